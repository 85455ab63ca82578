// Unitary forward scan on the bf16 matrix cores, two wavefronts per SIMD (N <= 16).
//
// Same mathematics, operand splitting and LDS record formats as scan_fwd_xdl.h.  What changes is
// the work split.  One wavefront per SIMD can issue a vector instruction only every ~5 cycles and
// leaves every LDS, matrix-pipe and barrier latency exposed; two wavefronts per SIMD issue at
// twice that rate and hide each other's waits.  A workgroup still owns (batch b, 64 channels), but
// has eight wavefronts: wavefronts cg and cg + 4 share the 16 channels of group cg and split each
// 32-step chunk by time.  Wavefront half hf = 0 owns timesteps 0..15 of the chunk (result tile 0),
// hf = 1 timesteps 16..31 (tile 1); lane (dl, g) owns t = 16 hf + 4 g + i, i = 0..3.
//   * per-timestep vector work (phases, sincos, rotated inputs, splitting, outputs) is halved;
//   * the products over s need V of the whole chunk: each wavefront writes its half of the V pieces
//     to an LDS exchange buffer while preparing chunk c + 1 and both read whole operands in step
//     c + 1 (the barrier between the steps is the one that already separates them);
//   * S is computed for the own tile only; the state update H += B^T V (24 matrix instructions) and
//     its rotation are done by both wavefronts redundantly, which is cheaper than exchanging H;
//   * hf = 1 needs the phase accumulated over tile 0: it reads those 16 theta values itself;
//   * the rotation over the whole chunk (P at timestep 31) comes from hf = 1 through LDS;
//   * G is produced as six half-jobs (3 tiles x re/im) on wavefronts 0..5, B/C staging is spread
//     over 512 threads (first mapping on threads 0..255, second on 256..511).
#pragma once
#include "scan_fwd_xdl.h"

namespace aussm {

template <int NP>
struct XdlBC2 {
  u4 cs_r[NP][XT * 4];   // row t: [ Cr[4g..4g+3], -Ci[4g..4g+3] ]
  u4 cs_i[NP][XT * 4];   // row t: [ Ci[4g..4g+3],  Cr[4g..4g+3] ]
  u4 bs[NP][XT * 4];     // row s: [ Br[4g..4g+3],  Bi[4g..4g+3] ]
  u4 bt_r[NP][XN * 4];   // row n: Br[t(g, e)][n], e = 0..7
  u4 bt_i[NP][XN * 4];   //        Bi
};
template <int NP>
struct XdlV {                       // V of one chunk: [re/im][piece][cg][lane] -> 8 K slots (16 bytes)
  u4 v[2][NP][4][64];
  float2 pT[4][16];                 // (cos, sin) of the phase at the last timestep, per channel
};

template <int NP, bool GATED>
__global__ __launch_bounds__(512) void unitary_fwd_xdl2_kernel(const FwdArgs p) {
  __shared__ XdlBC2<NP> s_bc[3];
  __shared__ XdlG<NP> s_g[2];
  __shared__ XdlV<NP> s_v[2];

  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int b = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int cg = wave & 3, hf = wave >> 2;
  const int dl = lane & 15, g = lane >> 4;
  const int D = p.D, N = p.N, L = p.L;
  const int d = d0 + cg * 16 + dl;
  const bool dok = d < D;
  const int dc = dok ? d : D - 1;
  const size_t row = ((size_t)b * D + dc) * L;
  const float* __restrict__ gu = static_cast<const float*>(p.u) + row;
  const float* __restrict__ gdl = static_cast<const float*>(p.delta) + row;
  const float* __restrict__ gth = p.theta + row;
  const float* __restrict__ gz = GATED ? p.z + row : nullptr;
  const float* __restrict__ gB = static_cast<const float*>(p.Bm);
  const float* __restrict__ gC = static_cast<const float*>(p.Cm);
  const float dsk = (p.Dskip && dok) ? p.Dskip[dc] : 0.0f;
  const int nchunks = (L + XT - 1) / XT;
  const SplitK sk = make_splitk();
  const float hff = hf ? 1.0f : 0.0f;

  // G tiles above the block diagonal are read (as zeros) but never written
  for (int i = tid; i < (int)(sizeof(s_g) / 16); i += 512) reinterpret_cast<u4*>(s_g)[i] = u4{0, 0, 0, 0};

  // ---- B/C staging.  Threads 0..255, first mapping: thread (t = tid % 32, g1 = (tid / 32) % 4) of C
  // (tid < 128) or B builds the records [row t][g1] from the four state rows 4 g1 .. 4 g1 + 3.
  // Threads 256..511, second mapping: thread (n = x % 16, g2 = (x / 16) % 4, half = (x / 64) % 2),
  // x = tid - 256, reads the four timesteps 16 half + 4 g2 .. + 3 of row n of B and writes the Br
  // (x < 128) or Bi half-record.
  const bool is_m1 = tid < 256;
  const int m1_t = tid & 31, m1_g = (tid >> 5) & 3;
  const bool m1_isB = (tid & 255) >= 128;
  const float* __restrict__ m1_src = m1_isB ? gB : gC;
  const uint32_t m1_s1 = m1_isB ? 0u : 0x80008000u;   // C records carry -Im
  const int m2_n = tid & 15, m2_g = (tid >> 4) & 3, m2_half = (tid >> 6) & 1;
  const bool m2_im = (tid & 255) >= 128;
  f4 raw[2];                        // first mapping: four (re, im) pairs; second: four complex timesteps
  auto bc_load = [&](int c) {
    if (is_m1) {
      const int l = c * XT + m1_t;
      const int lc = l < L ? l : 0;
      float2 t4[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int n = 4 * m1_g + k;
        const size_t o = (((size_t)b * N + (n < N ? n : 0)) * L + lc) * 2;
        t4[k] = *reinterpret_cast<const float2*>(m1_src + o);
      }
      raw[0] = f4{t4[0].x, t4[0].y, t4[1].x, t4[1].y};
      raw[1] = f4{t4[2].x, t4[2].y, t4[3].x, t4[3].y};
    } else {
      const int l2 = c * XT + 16 * m2_half + 4 * m2_g;
      const int l2c = l2 < L ? l2 : 0;
      const size_t o2 = (((size_t)b * N + (m2_n < N ? m2_n : 0)) * L + l2c) * 2;
      raw[0] = *reinterpret_cast<const f4*>(gB + o2);
      raw[1] = *reinterpret_cast<const f4*>(gB + o2 + 4);
    }
  };
  auto bc_store = [&](int c, XdlBC2<NP>& s) {
    if (is_m1) {
      const bool tok = c * XT + m1_t < L;
      float x[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const bool ok = tok && (4 * m1_g + k < N);
        x[k] = ok ? raw[k >> 1][2 * (k & 1)] : 0.0f;
        x[4 + k] = ok ? raw[k >> 1][2 * (k & 1) + 1] : 0.0f;
      }
      u4 pc[NP];
      split8<NP>(sk, x, pc);
      const int o = xrec(m1_t, m1_g, XT);
      u4* d1 = m1_isB ? &s.bs[0][0] : &s.cs_r[0][0];
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        d1[q * (XT * 4) + o] = u4{pc[q][0], pc[q][1], pc[q][2] ^ m1_s1, pc[q][3] ^ m1_s1};
        if (!m1_isB) s.cs_i[q][o] = u4{pc[q][2], pc[q][3], pc[q][0], pc[q][1]};
      }
    } else {
      const bool ok = (m2_n < N) && (c * XT + 16 * m2_half + 4 * m2_g < L);
      const int sel = m2_im ? 1 : 0;
      const float v0 = ok ? raw[0][sel] : 0.0f, v1 = ok ? raw[0][2 + sel] : 0.0f;
      const float v2 = ok ? raw[1][sel] : 0.0f, v3 = ok ? raw[1][2 + sel] : 0.0f;
      uint32_t a[NP], c2[NP];
      split2<NP>(sk, v0, v1, a);
      split2<NP>(sk, v2, v3, c2);
      const int o = xrec(m2_n, m2_g, XN) * 2 + m2_half;   // 8-byte half-record index
      u2* d1 = reinterpret_cast<u2*>(m2_im ? &s.bt_i[0][0] : &s.bt_r[0][0]);
#pragma unroll
      for (int q = 0; q < NP; ++q) d1[q * (XN * 4 * 2) + o] = u2{a[q], c2[q]};
    }
  };

  // ---- G: job j = min(wave, 5 - (7 - wave) ... ) : tile j / 2 of ((0,0), (1,0), (1,1)), part j % 2
  // (re, im); wavefronts 6 and 7 repeat jobs 4 and 5.
  const int gjob = wave < 6 ? wave : wave - 2;
  const int gtile = gjob >> 1, gpart = gjob & 1;
  const int gtt = gtile >= 1 ? 1 : 0, gst = gtile >= 2 ? 1 : 0;
  const int g_lim = (gtt == gst) ? dl : 64;   // diagonal tiles keep s <= t (a per-lane bound: no branch)
  auto make_g = [&](const XdlBC2<NP>& s, XdlG<NP>& o) {
    u4 a[NP], bq[NP];
    const u4* src = gpart ? &s.cs_i[0][0] : &s.cs_r[0][0];
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      a[q] = s.bs[q][xrec(16 * gst + dl, g, XT)];
      bq[q] = src[q * (XT * 4) + xrec(16 * gtt + dl, g, XT)];
    }
    f4 gx = xmm<NP>(a, bq, f4{0, 0, 0, 0});
#pragma unroll
    for (int i = 0; i < 4; ++i) gx[i] = (4 * g + i <= g_lim) ? gx[i] : 0.0f;
    uint32_t r0[NP], r1[NP];
    split2<NP>(sk, gx[0], gx[1], r0);
    split2<NP>(sk, gx[2], gx[3], r1);
    const int h = xrec(16 * gtt + dl, g, XT) * 2 + gst;   // 8-byte half-record index
    u2* dst = reinterpret_cast<u2*>(gpart ? &o.im[0][0] : &o.re[0][0]);
#pragma unroll
    for (int q = 0; q < NP; ++q) dst[q * (XT * 4 * 2) + h] = u2{r0[q], r1[q]};
  };

  // ---- channel data of one chunk: the own run of four timesteps (and theta of tile 0)
  struct In { f4 u, de, th, tha, z; };
  auto in_load = [&](In& r, int c) {
    const int l = c * XT + 16 * hf + 4 * g;
    const int lc = l < L ? l : 0;
    const int la = c * XT + 4 * g;
    const int lac = la < L ? la : 0;
    r.u = *reinterpret_cast<const f4*>(gu + lc);
    r.de = *reinterpret_cast<const f4*>(gdl + lc);
    r.th = *reinterpret_cast<const f4*>(gth + lc);
    r.tha = *reinterpret_cast<const f4*>(gth + lac);
    if (GATED) r.z = *reinterpret_cast<const f4*>(gz + lc);
  };

  // ---- per-channel vector work of one chunk
  struct Prep { float cs[4], sn[4]; f4 u, z; };
  auto prep = [&](const In& r, int c, Prep& o, XdlV<NP>& xv) {
    const bool ok = c * XT + 16 * hf + 4 * g < L;
    const bool oka = c * XT + 4 * g < L;
    float th[4], ta[4], w[4];
    bool big = false;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      th[i] = ok ? r.th[i] : 0.0f;
      ta[i] = oka ? r.tha[i] : 0.0f;
      big |= fabsf(th[i]) > 4.0f || fabsf(ta[i]) > 4.0f;
      w[i] = ok ? r.de[i] * r.u[i] : 0.0f;
    }
    // phases are reduced to (-pi, pi] when any of them is large so that the running sums stay
    // small enough for sincos_small and for fp32 sums of 32 terms
    if (__builtin_expect(__any(big), 0)) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        th[i] = (float)remainder((double)th[i], 6.283185307179586476925);
        ta[i] = (float)remainder((double)ta[i], 6.283185307179586476925);
      }
    }
    th[1] += th[0]; th[2] += th[1]; th[3] += th[2];
    float sa = th[3];
    {
      float t1 = __shfl_up(sa, 16);
      if (g >= 1) sa += t1;
      t1 = __shfl_up(sa, 32);
      if (g >= 2) sa += t1;
    }
    float tot0 = (ta[0] + ta[1]) + (ta[2] + ta[3]);   // phase accumulated over tile 0 (used by hf = 1)
    tot0 += __shfl_xor(tot0, 16);
    tot0 += __shfl_xor(tot0, 32);
    const float off = (sa - th[3]) + hff * tot0;
    float vr[4], vi[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sincos_small(th[i] + off, &o.sn[i], &o.cs[i]);
      vr[i] = o.cs[i] * w[i];
      vi[i] = -o.sn[i] * w[i];
    }
    o.u = r.u;
    if (GATED) o.z = r.z;
    uint32_t a0[NP], a1[NP], b0[NP], b1[NP];
    split2<NP>(sk, vr[0], vr[1], a0);
    split2<NP>(sk, vr[2], vr[3], a1);
    split2<NP>(sk, vi[0], vi[1], b0);
    split2<NP>(sk, vi[2], vi[3], b1);
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      reinterpret_cast<u2*>(&xv.v[0][q][cg][lane])[hf] = u2{a0[q], a1[q]};
      reinterpret_cast<u2*>(&xv.v[1][q][cg][lane])[hf] = u2{b0[q], b1[q]};
    }
    // rotation over the whole chunk: the element (hf 1, g 3, i 3) is timestep 31
    if (hf == 1 && g == 3) xv.pT[cg][dl] = make_float2(o.cs[3], o.sn[3]);
  };

  // ---- state: lane (dl, g) holds H[n = 4 g + i][channel dl] (both wavefronts of a group alike)
  f4 Hr = {0, 0, 0, 0}, Hi = {0, 0, 0, 0};
  if (p.h0 && dok) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        const size_t o = (((size_t)b * D + d) * N + n) * 2;
        Hr[i] = p.h0[o];
        Hi[i] = p.h0[o + 1];
      }
    }
  }

  int i0 = 0, i1 = 1, i2 = 2;   // LDS slots of chunks c, c+1, c+2
  const int ck_chunks = p.ck / XT;
  int ck_left = ck_chunks, kb = 0;   // chunks to the next checkpoint, its index

  // One chunk.  pc: vector work of chunk c (ready, its V in s_v[c & 1]); pn: receives that of chunk
  // c + 1, computed from in1; in2 receives the loads of chunk c + 2.
  auto step = [&](int c, In& in1, In& in2, Prep& pc, Prep& pn) {
    const int l0 = c * XT;
    const XdlBC2<NP>& s = s_bc[i0];
    const XdlG<NP>& G = s_g[c & 1];
    const XdlV<NP>& xv = s_v[c & 1];
    bc_store(c + 2, s_bc[i2]);
    bc_load(c + 3);
    in_load(in2, c + 2);

    // ---- operands of chunk c
    u4 Vr[NP], Vi[NP], nVi[NP], hk[NP], c_r[NP], c_i[NP], b_r[NP], b_i[NP], g_r[NP], g_i[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      Vr[q] = xv.v[0][q][cg][lane];
      Vi[q] = xv.v[1][q][cg][lane];
      nVi[q] = neg_bf16x8(Vi[q]);
      c_r[q] = s.cs_r[q][xrec(16 * hf + dl, g, XT)];
      c_i[q] = s.cs_i[q][xrec(16 * hf + dl, g, XT)];
      b_r[q] = s.bt_r[q][xrec(dl, g, XN)];
      b_i[q] = s.bt_i[q][xrec(dl, g, XN)];
      g_r[q] = G.re[q][xrec(16 * hf + dl, g, XT)];
      g_i[q] = G.im[q][xrec(16 * hf + dl, g, XT)];
    }
    const float2 pT = xv.pT[cg][dl];
    {
      const float x[8] = {Hr[0], Hr[1], Hr[2], Hr[3], Hi[0], Hi[1], Hi[2], Hi[3]};
      split8<NP>(sk, x, hk);
    }
    // ---- S (own tile) = C.H + G.V ;  H += B^T V
    f4 Sr = xmm<NP>(c_r, hk, f4{0, 0, 0, 0});
    f4 Si = xmm<NP>(c_i, hk, f4{0, 0, 0, 0});
    Hr = xmm<NP>(b_r, Vr, Hr);
    Hi = xmm<NP>(b_r, Vi, Hi);
    Sr = xmm<NP>(g_r, Vr, Sr);
    Si = xmm<NP>(g_r, Vi, Si);
    Hr = xmm<NP>(b_i, nVi, Hr);
    Hi = xmm<NP>(b_i, Vr, Hi);
    Sr = xmm<NP>(g_i, nVi, Sr);
    Si = xmm<NP>(g_i, Vr, Si);

    // ---- G of chunk c + 1, vector work of chunk c + 1 (independent of the products above)
    make_g(s_bc[i1], s_g[(c + 1) & 1]);
    prep(in1, c + 1, pn, s_v[(c + 1) & 1]);

    // ---- rotate the state to the end of the chunk
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float xr = Hr[i], xi = Hi[i];
      Hr[i] = pT.x * xr - pT.y * xi;
      Hi[i] = fmaf(pT.x, xi, pT.y * xr);
    }
    // ---- outputs: rows 16 hf + 4 g + i of channel dl are this lane's own timesteps
    if (p.y && dok) {
      const int l = l0 + 16 * hf + 4 * g;
      if (l < L) {
        f4 yo;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = pc.cs[i] * Sr[i] - pc.sn[i] * Si[i];
          v = fmaf(dsk, pc.u[i], v);
          if (GATED) v *= siluf_(pc.z[i]);
          yo[i] = v;
        }
        *reinterpret_cast<f4*>(p.y + row + l) = yo;
      }
    }
    // optional: Im(P_t S_t), which the backward pass would otherwise recompute
    if (p.aux && dok) {
      const int l = l0 + 16 * hf + 4 * g;
      if (l < L) {
        f4 ph;
#pragma unroll
        for (int i = 0; i < 4; ++i) ph[i] = pc.cs[i] * Si[i] + pc.sn[i] * Sr[i];
        *reinterpret_cast<f4*>(p.aux + row + l) = ph;
      }
    }
    // ---- checkpoint: state at the end of every ck-step block and at the end of the sequence
    const bool ck_now = l0 < L && (--ck_left == 0 || l0 + XT >= L);
    if (p.hck && dok && ck_now && hf == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = 4 * g + i;
        if (n < N) {
          const size_t o = ((((size_t)b * p.nck + kb) * N + n) * 2) * D + d;
          p.hck[o] = Hr[i];
          p.hck[o + D] = Hi[i];
        }
      }
    }
    if (ck_now) { ck_left = ck_chunks; ++kb; }
    const int tmp = i0; i0 = i1; i1 = i2; i2 = tmp;
    __syncthreads();
  };

  // ---- prologue
  In inA, inB;
  Prep P0, P1;
  bc_load(0);
  in_load(inB, 0);
  in_load(inA, 1);
  bc_store(0, s_bc[0]);
  bc_load(1);
  bc_store(1, s_bc[1]);
  bc_load(2);
  prep(inB, 0, P0, s_v[0]);
  __syncthreads();
  make_g(s_bc[0], s_g[0]);
  __syncthreads();

  // Two chunks per trip so that the register sets alternate without copies.  With an odd number of
  // chunks the last half-trip runs on an all-padding chunk: zero input, zero phase, no stores, and
  // the state passes through unchanged.
  for (int c = 0; c < nchunks; c += 2) {
    step(c, inA, inB, P0, P1);
    step(c + 1, inB, inA, P1, P0);
  }

  if (p.aux && blockIdx.x == 0 && tid == 0) p.aux[(size_t)p.B * D * L] = __uint_as_float(AUX_TAG);
  if (p.hL && dok && hf == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        const size_t o = (((size_t)b * D + d) * N + n) * 2;
        p.hL[o] = Hr[i];
        p.hL[o + 1] = Hi[i];
      }
    }
  }
}

}  // namespace aussm
