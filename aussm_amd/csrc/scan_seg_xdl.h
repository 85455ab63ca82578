// Splitting the sequence of a unitary scan over workgroups (few (batch, channel) pairs, long L).
//
// The recurrence is linear in the state, so a segment [l0, l0 + Ls) of the sequence acts on the
// state that enters it as  H_out = P H_in + Z  with P = exp(i sum theta) the segment's rotation
// and Z its end state from a zero start; the adjoint runs the other way, A_in = conj(P) A_out + Y
// with Y the adjoint at the segment start from a zero adjoint at its end.  The launcher therefore
//   1. computes (P, Z) or (P, Y) of every segment with unitary_seg_state_kernel (all segments in
//      parallel; only the sums  Z = P sum_s conj(P_s) delta_s u_s B_s,  Y = sum_t conj(P_t) dy_t conj(C_t)
//      are formed: per chunk one product with the channel as free index, on the matrix cores in
//      the layout of the scan kernels),
//   2. chains the segments of each (batch, channel, state) with seg_carry_*_kernel (ns steps),
//   3. runs the scan kernel proper with (batch, segment) pairs as its batch index, every segment
//      starting from its true incoming state or adjoint.
#pragma once
#include <type_traits>

#include "scan_fwd_xdl.h"

namespace aussm {


// ADJ = false: Z of each segment, chunks in forward order,  H <- P_T (H + B^T V).
// ADJ = true:  Y of each segment, chunks in reverse order,  A <- conj(P_T) A + conj(C)^T Q.
// Requires N <= 16, L % 4 == 0, 16-byte aligned tensors.  Tin: float or bf16_t (u, delta, B, C).
// Four wavefronts per SIMD (128 registers): the launch of a split call (1024 light workgroups for 64 fine segments
// of a batch of 4 x 4 channel groups) then fits the chip in one round instead of one and a third.
template <int NP, bool ADJ, typename Tin = float>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void unitary_seg_state_kernel(const SegArgs p) {
  // row n: M[t(g, e)][n], real and imaginary parts (the imaginary part negated for ADJ: conj(C))
  __shared__ u4 s_mr[2][NP][XN * 4];
  __shared__ u4 s_mi[2][NP][XN * 4];

  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int vb = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int dl = lane & 15, g = lane >> 4;
  const int D = p.D, N = p.N, L = p.L;
  const int d = d0 + wave * 16 + dl;
  const bool dok = d < D;
  const int dc = dok ? d : D - 1;
  const int bb = vb / p.ns;
  const size_t so = (size_t)(vb - bb * p.ns) * L;
  const size_t row = ((size_t)bb * D + dc) * p.ld + so;
  using TA = typename std::conditional<ADJ, float, Tin>::type;   // dy is always float
  const TA* __restrict__ gx1 = static_cast<const TA*>(p.x1) + row;
  const Tin* __restrict__ gx2 = ADJ ? nullptr : static_cast<const Tin*>(p.x2) + row;
  const Tin* __restrict__ gM = static_cast<const Tin*>(p.M);
  const float* __restrict__ gth = p.theta + row;
  const int nchunks = (L + XT - 1) / XT;
  const SplitK sk = make_splitk();

  // staging: thread (n = tid % 16, g2 = (tid / 16) % 4, half = (tid / 64) % 2) reads the four
  // timesteps 16 half + 4 g2 .. + 3 of row n; tid < 128 writes the real half-record, the others
  // the imaginary one
  const int m2_n = tid & 15, m2_g = (tid >> 4) & 3, m2_half = (tid >> 6) & 1;
  const bool m2_im = tid >= 128;
  RawC4<Tin> m2_raw;
  auto m_load = [&](int c) {
    const int cc = c < 0 ? 0 : (c >= nchunks ? nchunks - 1 : c);
    const int l2 = cc * XT + 16 * m2_half + 4 * m2_g;
    const int l2c = l2 < L ? l2 : 0;
    const size_t o2 = (((size_t)bb * N + (m2_n < N ? m2_n : 0)) * p.ld + so + l2c) * 2;
    m2_raw.load(gM + o2);
  };
  auto m_store = [&](int c, int slot) {
    const bool ok = (m2_n < N) && (c * XT + 16 * m2_half + 4 * m2_g < L);
    const float sg = (ADJ && m2_im) ? -1.0f : 1.0f;
    float v0 = m2_im ? m2_raw.im(0) : m2_raw.re(0), v1 = m2_im ? m2_raw.im(1) : m2_raw.re(1);
    float v2 = m2_im ? m2_raw.im(2) : m2_raw.re(2), v3 = m2_im ? m2_raw.im(3) : m2_raw.re(3);
    v0 = ok ? sg * v0 : 0.0f; v1 = ok ? sg * v1 : 0.0f; v2 = ok ? sg * v2 : 0.0f; v3 = ok ? sg * v3 : 0.0f;
    constexpr int NPS = sizeof(Tin) == 2 ? 1 : NP;   // bf16 values are a single exact piece
    uint32_t a0[NPS], a1[NPS];
    split2<NPS>(sk, v0, v1, a0);
    split2<NPS>(sk, v2, v3, a1);
    const int o = xrec(m2_n, m2_g, XN) * 2 + m2_half;   // 8-byte half-record index
    u4 (*dst)[XN * 4] = m2_im ? s_mi[slot] : s_mr[slot];
#pragma unroll
    for (int q = 0; q < NPS; ++q) reinterpret_cast<u2*>(dst[q])[o] = u2{a0[q], a1[q]};
  };

  struct In { f4 th[2]; Raw4<TA> a[2]; Raw4<Tin> b[2]; };
  auto in_load = [&](In& r, int c) {
    const int cc = c < 0 ? 0 : (c >= nchunks ? nchunks - 1 : c);
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int l = cc * XT + 16 * st + 4 * g;
      const int lc = l < L ? l : 0;
      r.th[st] = *reinterpret_cast<const f4*>(gth + lc);
      r.a[st].load(gx1 + lc);
      if (!ADJ) r.b[st].load(gx2 + lc);
    }
  };

  // lane (dl, g) holds the state (or adjoint) rows n = 4 g + i of channel dl
  f4 Sr = {0, 0, 0, 0}, Si = {0, 0, 0, 0};
  float pr = 1.0f, pi = 0.0f;   // rotation of the chunks done so far

  In cur;
  const int c_first = ADJ ? nchunks - 1 : 0, c_step = ADJ ? -1 : 1;
  m_load(c_first);
  in_load(cur, c_first);

  for (int k = 0; k < nchunks; ++k) {
    const int c = c_first + k * c_step;
    const int slot = k & 1;
    const int l0 = c * XT;
    m_store(c, slot);
    In nxt;
    m_load(c + c_step);
    in_load(nxt, c + c_step);
    __syncthreads();   // planes of this chunk visible; the other slot was last read one barrier ago

    float th[2][4], x[8];
    bool big = false;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const bool ok = dok && (l0 + 16 * st + 4 * g < L);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        th[st][i] = ok ? cur.th[st][i] : 0.0f;
        big |= fabsf(th[st][i]) > 4.0f;
        const float v = ADJ ? cur.a[st].get(i) : cur.a[st].get(i) * cur.b[st].get(i);
        x[4 * st + i] = ok ? v : 0.0f;
      }
    }
    if (__builtin_expect(__any(big), 0)) {
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int i = 0; i < 4; ++i) th[st][i] = (float)remainder((double)th[st][i], 6.283185307179586476925);
    }
    // running phase inside the chunk: the lane's two runs of four steps, then across the lane groups
#pragma unroll
    for (int st = 0; st < 2; ++st) { th[st][1] += th[st][0]; th[st][2] += th[st][1]; th[st][3] += th[st][2]; }
    float sa = th[0][3], sb = th[1][3];
    {
      float ta = __shfl_up(sa, 16), tb = __shfl_up(sb, 16);
      if (g >= 1) { sa += ta; sb += tb; }
      ta = __shfl_up(sa, 32); tb = __shfl_up(sb, 32);
      if (g >= 2) { sa += ta; sb += tb; }
    }
    const float tot_a = __shfl(sa, 48 + dl);
    const float off_a = sa - th[0][3];
    const float off_b = tot_a + sb - th[1][3];
    float xr[8], xi[8], c7 = 0.0f, s7 = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float ph = th[e >> 2][e & 3] + ((e >> 2) ? off_b : off_a);
      float sn, cs;
      if (e == 7) sincos_small(ph, &sn, &cs);       // (in lane group 3 the rotation of the whole chunk: it accumulates)
      else sincos_small_hw(ph, &sn, &cs);
      xr[e] = cs * x[e];        // x conj(P)
      xi[e] = -sn * x[e];
      if (e == 7) { c7 = cs; s7 = sn; }
    }
    const float cT = __shfl(c7, 48 + dl), sT = __shfl(s7, 48 + dl);   // rotation of the whole chunk
    u4 Xr[NP], Xi[NP], nXi[NP];
    split8<NP>(sk, xr, Xr);
    split8<NP>(sk, xi, Xi);
#pragma unroll
    for (int q = 0; q < NP; ++q) nXi[q] = neg_bf16x8(Xi[q]);
    u4 mr[NP], mi[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) { mr[q] = s_mr[slot][q][xrec(dl, g, XN)]; mi[q] = s_mi[slot][q][xrec(dl, g, XN)]; }
    if (ADJ) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float ar = Sr[i], ai = Si[i];
        Sr[i] = cT * ar + sT * ai;
        Si[i] = cT * ai - sT * ar;
      }
    }
    constexpr int NPA = sizeof(Tin) == 2 ? 1 : NP;   // bf16 B / C: a single exact piece
    Sr = xmm_p<NP, NPA>(mr, Xr, Sr);  Sr = xmm_p<NP, NPA>(mi, nXi, Sr);
    Si = xmm_p<NP, NPA>(mr, Xi, Si);  Si = xmm_p<NP, NPA>(mi, Xr, Si);
    if (!ADJ) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float hr = Sr[i], hi = Si[i];
        Sr[i] = cT * hr - sT * hi;
        Si[i] = cT * hi + sT * hr;
      }
    }
    {
      const float nr = pr * cT - pi * sT, ni = pr * sT + pi * cT;
      pr = nr; pi = ni;
    }
    cur = nxt;
  }

  if (dok) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        const size_t o = (((size_t)vb * D + d) * N + n) * 2;
        p.out[o] = Sr[i];
        p.out[o + 1] = Si[i];
      }
    }
    if (g == 0) {
      p.ptot[((size_t)vb * D + d) * 2] = pr;
      p.ptot[((size_t)vb * D + d) * 2 + 1] = pi;
    }
  }
}

// Chains the segments of one (batch, channel, state).  Forward (ADJ false): on entry seg[k] holds Z_k, on return the
// state that enters segment k; the state after the last segment goes to `last` (if wanted); `first` is the state
// before the first one (or null).  ADJ: on entry seg[k] holds Y_k, on return the adjoint that enters segment k at
// its end, walking from the last segment with conj(q_k); `first` is the adjoint after the last segment, `last`
// receives the adjoint of the initial state.
// The chain is short and there are few of them (B D N), so one thread per chain leaves the chip waiting on its
// loads: CARRY_SUBS threads share a chain - each composes its run of consecutive segments into one affine map
// h -> Q h + Z, the maps of the runs before it (LDS) give the state that enters its run, and it walks the run
// again writing every segment's incoming state.
constexpr int CARRY_SUBS = 8;          // threads per chain
constexpr int CARRY_RUN = 16;          // segments per thread at most: chains of up to 128 segments
template <bool ADJ>
__global__ __launch_bounds__(32 * CARRY_SUBS) void seg_carry_kernel(float* __restrict__ seg, const float* __restrict__ ptot,
                                                                    const float* __restrict__ first, float* __restrict__ last,
                                                                    int B, int D, int N, int ns) {
  __shared__ float4 s_map[CARRY_SUBS][32];          // (Re Q, Im Q, Re Z, Im Z) of every run
  const int cl = threadIdx.x & 31, sub = threadIdx.x >> 5;
  const size_t idx = (size_t)blockIdx.x * 32 + cl;
  const bool ok = idx < (size_t)B * D * N;
  const size_t ic = ok ? idx : 0;
  const int n = (int)(ic % N);
  const int d = (int)((ic / N) % D);
  const int b = (int)(ic / ((size_t)N * D));
  const int per = (ns + CARRY_SUBS - 1) / CARRY_SUBS;
  auto mul = [](float2 q, float hr, float hi) {          // q h, or conj(q) h for the adjoint
    return ADJ ? make_float2(q.x * hr + q.y * hi, q.x * hi - q.y * hr) : make_float2(q.x * hr - q.y * hi, q.x * hi + q.y * hr);
  };
  float2 z[CARRY_RUN], q[CARRY_RUN];
  size_t off[CARRY_RUN];
#pragma unroll
  for (int j = 0; j < CARRY_RUN; ++j) {
    const int pos = sub * per + j;
    const bool valid = j < per && pos < ns;
    const int k = valid ? (ADJ ? ns - 1 - pos : pos) : 0;
    const size_t v = ((size_t)b * ns + k) * D + d;
    off[j] = valid ? (v * N + n) * 2 : ~(size_t)0;
    z[j] = valid ? *reinterpret_cast<const float2*>(seg + (v * N + n) * 2) : make_float2(0.f, 0.f);
    q[j] = valid ? *reinterpret_cast<const float2*>(ptot + v * 2) : make_float2(1.f, 0.f);
  }
  float Qr = 1.f, Qi = 0.f, Zr = 0.f, Zi = 0.f;
#pragma unroll
  for (int j = 0; j < CARRY_RUN; ++j) {
    const float2 a = mul(q[j], Qr, Qi), c = mul(q[j], Zr, Zi);
    Qr = a.x; Qi = a.y; Zr = c.x + z[j].x; Zi = c.y + z[j].y;
  }
  s_map[sub][cl] = make_float4(Qr, Qi, Zr, Zi);
  __syncthreads();
  float hr = first ? first[ic * 2] : 0.0f, hi = first ? first[ic * 2 + 1] : 0.0f;
  for (int s_ = 0; s_ < sub; ++s_) {
    const float4 m = s_map[s_][cl];
    // (the maps hold q's products already conjugated for the adjoint: plain complex multiplication here)
    const float nr = m.x * hr - m.y * hi + m.z, ni = m.x * hi + m.y * hr + m.w;
    hr = nr; hi = ni;
  }
#pragma unroll
  for (int j = 0; j < CARRY_RUN; ++j) {
    if (off[j] != ~(size_t)0) {
      if (ok) *reinterpret_cast<float2*>(seg + off[j]) = make_float2(hr, hi);
      const float2 a = mul(q[j], hr, hi);
      hr = a.x + z[j].x; hi = a.y + z[j].y;
    }
  }
  if (last && ok && sub == CARRY_SUBS - 1) { last[idx * 2] = hr; last[idx * 2 + 1] = hi; }
}

}  // namespace aussm
