// Unitary backward scan in chunked matrix form on the bf16 matrix cores, fp32-accurate (N <= 16).
//
// Chunks of XT = 32 timesteps are visited in reverse.  With the forward quantities of a chunk
// (Theta_t running phase, P_t = exp(i Theta_t), w = delta u, V_s = conj(P_s) w_s, H the state at
// the chunk start, K_t = H + sum_{s<=t} B_s V_s, S_t = sum_n C_t[n] K_t[n], H_end = P_T K_T) and
// the incoming adjoints dy_t and A' (of H_end), in the convention dl = Re(conj(g) dz):
//     Q_t   = dy_t conj(P_t)                         adjoint of S_t
//     J     = conj(P_T) A'                           adjoint of K_T through H_end
//     H     = conj(P_T) H_end - sum_s B_s V_s        the state is recomputed backwards
//     gV_s  = sum_n conj(B_s[n]) J[n] + sum_{t>=s} conj(G[t,s]) Q_t
//     A     = J + sum_t conj(C_t) Q_t                adjoint of H (A' of the previous chunk)
//     dw_s  = Re(gV_s P_s),  du = delta dw + D dy,  ddelta = u dw
//     gTh_t = Im(conj(gV_t) V_t) - dy_t Im(P_t S_t)  [- sum_n Im(conj(A') H_end) at t = T]
//     dtheta_r = sum_{t>=r in chunk} gTh_t
//     dC_t[n] = sum_d Q_t conj(H[n])  + sum_{s<=t} M[t,s] conj(B_s[n])
//     dB_s[n] = sum_d conj(V_s) J[n]  + sum_{t>=s} M[t,s] conj(C_t[n]),   M[t,s] = sum_d Q_t conj(V_s)
// Sums over n, s or t with the channel as free index run on the matrix cores in the layout of the
// forward kernel (lane = channel, eight owned timesteps = K slots / result rows).  The sums over
// the channel d (M and the two H/J terms) need the channel in the K slots instead: each wavefront
// transposes its own Q, V, H, J through a private LDS scratch, multiplies, and the four partial
// results of a workgroup are added and finished with two more small products before one atomic
// add per dB/dC element and workgroup.
#pragma once
#include "scan_bwd_unitary.h"
#include "scan_fwd_xdl.h"

namespace aussm {

template <int NP>
struct XbBC {
  u4 cs_r[NP][XT * 4];   // row t: [ Cr[4g..], -Ci[4g..] ]
  u4 cs_i[NP][XT * 4];   // row t: [ Ci[4g..],  Cr[4g..] ]
  u4 bs[NP][XT * 4];     // row s: [ Br[4g..],  Bi[4g..] ]
  u4 bs_c[NP][XT * 4];   // row s: [-Bi[4g..],  Br[4g..] ]
  u4 bt_r[NP][XN * 4];   // row n: Br[t(g,e)][n]
  u4 bt_i[NP][XN * 4];
  u4 ct_r[NP][XN * 4];   // row n: Cr[t(g,e)][n]
  u4 ct_i[NP][XN * 4];
};
template <int NP>
struct XbG {
  u4 gt_r[NP][XT * 4];   // row t, slots s: G[t][s] (zero where s > t)
  u4 gt_i[NP][XT * 4];
  u4 g_r[NP][XT * 4];    // row s, slots t: G[t][s] (zero where t < s)
  u4 g_i[NP][XT * 4];
};

constexpr int XB_TS = 33;                 // rows per channel group of the [t][d] scratch (32 + pad)
constexpr int XB_NS = 17;                 // rows per channel group of the [n][d] scratch
constexpr int XB_TD = 4 * XB_TS * 4;      // floats of one [t][d] array
constexpr int XB_ND = 4 * XB_NS * 4;      // floats of one [n][d] array
constexpr int XB_JOBS = 14;               // M (3 tiles x re, im), X1 (2 x 2), X2 (2 x 2)
constexpr int XB_WS = XB_JOBS * 64 * 4;   // floats of one wavefront's scratch (>= 4 XB_TD + 4 XB_ND)
constexpr int XB_AS = 36;                 // row stride of the dB/dC output tiles
constexpr int XB_MS = 36;                 // row stride of the summed M arrays
static_assert(4 * XB_TD + 4 * XB_ND <= XB_WS, "transpose arrays must fit the partial-sum region");

__device__ __forceinline__ u4 negp(const u4& v) { return v ^ u4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u}; }
template <int NP>
__device__ __forceinline__ void nega(const u4 (&a)[NP], u4 (&o)[NP]) {
#pragma unroll
  for (int q = 0; q < NP; ++q) o[q] = negp(a[q]);
}
// record [x0..x3, y0..y3] -> [-y0..-y3, x0..x3]  (multiplication of the packed complex by i)
template <int NP>
__device__ __forceinline__ void rot_i(const u4 (&a)[NP], u4 (&o)[NP]) {
#pragma unroll
  for (int q = 0; q < NP; ++q) o[q] = u4{a[q][2] ^ 0x80008000u, a[q][3] ^ 0x80008000u, a[q][0], a[q][1]};
}
// record [x0..x3, y0..y3] -> [y0..y3, -x0..-x3]  (multiplication by -i)
template <int NP>
__device__ __forceinline__ void rot_mi(const u4 (&a)[NP], u4 (&o)[NP]) {
#pragma unroll
  for (int q = 0; q < NP; ++q) o[q] = u4{a[q][2], a[q][3], a[q][0] ^ 0x80008000u, a[q][1] ^ 0x80008000u};
}
template <int NP>
__device__ __forceinline__ void ldrec(const u4 (*plane)[XT * 4], int idx, u4 (&o)[NP]) {
#pragma unroll
  for (int q = 0; q < NP; ++q) o[q] = plane[q][idx];
}
template <int NP>
__device__ __forceinline__ void ldrec16(const u4 (*plane)[XN * 4], int idx, u4 (&o)[NP]) {
#pragma unroll
  for (int q = 0; q < NP; ++q) o[q] = plane[q][idx];
}

// Prefetch loads whose results must sit untouched for a whole step.  The register file of this
// kernel is full (arch + accumulation registers); left to the compiler such a load lands in an
// arch register and is copied to an accumulation register a few instructions later, which makes
// the wavefront wait for the full memory latency at once.  These helpers load straight into
// accumulation registers; the compiler does not know the data is still in flight, so every value
// loaded this way passes through landed() (a wait for all vector-memory operations that also pins
// the values) before its first use.
__device__ __forceinline__ void ldg_acc(f4& dst, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=a"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void ldg_acc(float2& dst, const void* p) {
  asm volatile("global_load_dwordx2 %0, %1, off" : "=a"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void ldg_acc(float& dst, const void* p) {
  asm volatile("global_load_dword %0, %1, off" : "=a"(dst) : "v"(p) : "memory");
}
// The raw inputs of scan_fwd_xdl.h (Raw4, RawC, RawC4) loaded this way: float tensors as they are,
// bf16 tensors as packed words held in float-typed registers and widened where they are used.
template <typename Tin> struct AccRaw4;
template <> struct AccRaw4<float> {
  f4 v;
  __device__ __forceinline__ void load(const float* p) { ldg_acc(v, p); }
  __device__ __forceinline__ float get(int i) const { return v[i]; }
};
template <> struct AccRaw4<bf16_t> {
  float2 v;
  __device__ __forceinline__ void load(const bf16_t* p) { ldg_acc(v, p); }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = __float_as_uint(i < 2 ? v.x : v.y);
    return (i & 1) ? bf16_hi(w) : bf16_lo(w);
  }
};
template <typename Tin> struct AccRawC;
template <> struct AccRawC<float> {
  float2 v;
  __device__ __forceinline__ void load(const float* p) { ldg_acc(v, p); }
  __device__ __forceinline__ float re() const { return v.x; }
  __device__ __forceinline__ float im() const { return v.y; }
};
template <> struct AccRawC<bf16_t> {
  float v;
  __device__ __forceinline__ void load(const bf16_t* p) { ldg_acc(v, p); }
  __device__ __forceinline__ float re() const { return bf16_lo(__float_as_uint(v)); }
  __device__ __forceinline__ float im() const { return bf16_hi(__float_as_uint(v)); }
};
template <typename Tin> struct AccRawC4;
template <> struct AccRawC4<float> {
  f4 a, b;
  __device__ __forceinline__ void load(const float* p) { ldg_acc(a, p); ldg_acc(b, p + 4); }
  __device__ __forceinline__ float re(int j) const { return j < 2 ? a[2 * j] : b[2 * j - 4]; }
  __device__ __forceinline__ float im(int j) const { return j < 2 ? a[2 * j + 1] : b[2 * j - 3]; }
};
template <> struct AccRawC4<bf16_t> {
  f4 a;
  __device__ __forceinline__ void load(const bf16_t* p) { ldg_acc(a, p); }
  __device__ __forceinline__ float re(int j) const { return bf16_lo(__float_as_uint(a[j])); }
  __device__ __forceinline__ float im(int j) const { return bf16_hi(__float_as_uint(a[j])); }
};

// Requires: N <= 16, L % 4 == 0, 16-byte aligned tensors, ck % 32 == 0.  Tin: float or bf16_t (u, delta, B, C).
// NP: operand pieces of the products along the sequence (3 = fp32-accurate); NPC: pieces of the
// products that sum over the channel (M, X1, X2 and the two closing products of dB / dC).
template <int NP, int NPC, typename Tin = float>
__global__ __launch_bounds__(256) void unitary_bwd_xdl_kernel(const UniBwdArgs p) {
  __shared__ XbBC<NP> s_bc;
  __shared__ XbG<NP> s_g;
  __shared__ __attribute__((aligned(16))) float s_ws[4][XB_WS];
  __shared__ __attribute__((aligned(16))) float s_ms[4][XT * XB_MS];   // MS re, MS im, MT re, MT im
  __shared__ __attribute__((aligned(16))) float s_at[4][XN * XB_AS];

  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int b = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int dl = lane & 15, g = lane >> 4;
  const int D = p.D, N = p.N, L = p.L;
  const int d = d0 + wave * 16 + dl;
  const bool dok = d < D;
  const int dc = dok ? d : D - 1;
  // b counts (batch element, segment of L steps) pairs when the launcher has split the sequence:
  // states and checkpoints are indexed by b, the [.., ld] tensors by (bb, segment offset so)
  const int bb = b / p.ns;
  const size_t so = (size_t)(b - bb * p.ns) * L;
  const size_t row = ((size_t)bb * D + dc) * p.ld + so;
  const Tin* __restrict__ gu = static_cast<const Tin*>(p.u) + row;
  const Tin* __restrict__ gdl = static_cast<const Tin*>(p.delta) + row;
  const float* __restrict__ gth = p.theta + row;
  const float* __restrict__ gdy = p.dy + row;
  const Tin* __restrict__ gB = static_cast<const Tin*>(p.Bm);
  const Tin* __restrict__ gC = static_cast<const Tin*>(p.Cm);
  const float dsk = (p.Dskip && dok) ? p.Dskip[dc] : 0.0f;
  const int nchunks = (L + XT - 1) / XT;
  const SplitK sk = make_splitk();
  // non-zero pieces of the staged B / C records: bf16 inputs are a single exact piece
  constexpr int NPA = sizeof(Tin) == 2 ? 1 : NP, NPAC = sizeof(Tin) == 2 ? 1 : NPC;
  // Im(P_t S_t) left by the forward kernel (if it filled the buffer): saves recomputing S here
  const bool use_phi = p.aux != nullptr &&
      __builtin_amdgcn_readfirstlane(__float_as_uint(p.aux[(size_t)p.B * D * L])) == p.auxtag;
  if (p.tag_mode == 2 && use_phi) return;      // the kernel that needs the buffer's contents has done the work
  // (always a valid address: the load below is unconditional, its result unused without the tag)
  const float* __restrict__ gph = use_phi ? p.aux + row : gth;
  float* __restrict__ ws = s_ws[wave];

  // zero what is read but never written: G tiles off the causal side, the same tile of MS / MT
  for (int i = tid; i < (int)(sizeof(s_g) / 16); i += 256) reinterpret_cast<u4*>(&s_g)[i] = u4{0, 0, 0, 0};
  for (int i = tid; i < 4 * XT * XB_MS; i += 256) (&s_ms[0][0])[i] = 0.0f;

  // ---- B/C staging.  First mapping: thread (t = tid % 32, g1 = (tid / 32) % 4) of C (tid < 128) or B
  // builds the records [row t][g1] from state rows 4 g1 .. 4 g1 + 3.  Second mapping: thread
  // (n = tid % 16, g2 = (tid / 16) % 4, half = (tid / 64) % 2) of B (tid < 128) or C builds the
  // half-records [row n][g2] from the four timesteps 16 half + 4 g2 .. + 3.
  const int m1_t = tid & 31, m1_g = (tid >> 5) & 3;
  const bool m1_isB = tid >= 128;
  const Tin* __restrict__ m1_src = m1_isB ? gB : gC;
  const int m2_n = tid & 15, m2_g = (tid >> 4) & 3, m2_half = (tid >> 6) & 1;
  const bool m2_isC = tid >= 128;
  const Tin* __restrict__ m2_src = m2_isC ? gC : gB;
  AccRawC<Tin> m1_raw[4];
  AccRawC4<Tin> m2_raw;
  auto bc_load = [&](int c) {
    const int cc = c < 0 ? 0 : c;
    const int l = cc * XT + m1_t;
    const int lc = l < L ? l : 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int n = 4 * m1_g + k;
      const size_t o = (((size_t)bb * N + (n < N ? n : 0)) * p.ld + so + lc) * 2;
      m1_raw[k].load(m1_src + o);
    }
    const int l2 = cc * XT + 16 * m2_half + 4 * m2_g;
    const int l2c = l2 < L ? l2 : 0;
    const size_t o2 = (((size_t)bb * N + (m2_n < N ? m2_n : 0)) * p.ld + so + l2c) * 2;
    m2_raw.load(m2_src + o2);
  };
  // (only the NPA pieces that can be non-zero are formed and stored; the others are never read)
  auto bc_store = [&](int c) {
    {
      const bool tok = c * XT + m1_t < L;
      float x[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const bool ok = tok && (4 * m1_g + k < N);
        x[k] = ok ? m1_raw[k].re() : 0.0f;
        x[4 + k] = ok ? m1_raw[k].im() : 0.0f;
      }
      u4 pc[NPA], pi[NPA], pcs[NPA];
      split8<NPA>(sk, x, pc);                 // [re, im]
      rot_i<NPA>(pc, pi);                 // [-im, re]
      const int o = xrec(m1_t, m1_g, XT);
      if (m1_isB) {
#pragma unroll
        for (int q = 0; q < NPA; ++q) { s_bc.bs[q][o] = pc[q]; s_bc.bs_c[q][o] = pi[q]; }
      } else {
#pragma unroll
        for (int q = 0; q < NPA; ++q) {
          pcs[q] = u4{pc[q][0], pc[q][1], pc[q][2] ^ 0x80008000u, pc[q][3] ^ 0x80008000u};   // [re, -im]
          s_bc.cs_r[q][o] = pcs[q];
          s_bc.cs_i[q][o] = u4{pc[q][2], pc[q][3], pc[q][0], pc[q][1]};                        // [im, re]
        }
      }
    }
    {
      const bool ok = (m2_n < N) && (c * XT + 16 * m2_half + 4 * m2_g < L);
      const float r0 = ok ? m2_raw.re(0) : 0.0f, r1 = ok ? m2_raw.re(1) : 0.0f;
      const float r2 = ok ? m2_raw.re(2) : 0.0f, r3 = ok ? m2_raw.re(3) : 0.0f;
      const float j0 = ok ? m2_raw.im(0) : 0.0f, j1 = ok ? m2_raw.im(1) : 0.0f;
      const float j2 = ok ? m2_raw.im(2) : 0.0f, j3 = ok ? m2_raw.im(3) : 0.0f;
      uint32_t a0[NPA], a1[NPA], b0[NPA], b1[NPA];
      split2<NPA>(sk, r0, r1, a0);
      split2<NPA>(sk, r2, r3, a1);
      split2<NPA>(sk, j0, j1, b0);
      split2<NPA>(sk, j2, j3, b1);
      const int o = xrec(m2_n, m2_g, XN) * 2 + m2_half;   // 8-byte half-record index
#pragma unroll
      for (int q = 0; q < NPA; ++q) {
        if (m2_isC) {
          reinterpret_cast<u2*>(s_bc.ct_r[q])[o] = u2{a0[q], a1[q]};
          reinterpret_cast<u2*>(s_bc.ct_i[q])[o] = u2{b0[q], b1[q]};
        } else {
          reinterpret_cast<u2*>(s_bc.bt_r[q])[o] = u2{a0[q], a1[q]};
          reinterpret_cast<u2*>(s_bc.bt_i[q])[o] = u2{b0[q], b1[q]};
        }
      }
    }
  };

  // ---- G tile of one wavefront in both orientations: wave 0 -> (tt 0, st 0), 1 -> (1, 0), 2 and 3
  // -> (1, 1) (the same values twice).
  const int gtt = wave >= 1 ? 1 : 0, gst = wave >= 2 ? 1 : 0;
  const int g_lim = (gtt == gst) ? dl : 64;          // keep rows s = 4 g + i <= column t = dl
  const int g_low = (gtt == gst) ? dl : -1;          // keep rows t = 4 g + i >= column s = dl
  auto put_half = [&](u4 (*pr)[XT * 4], u4 (*pi)[XT * 4], int h, const f4& vr, const f4& vi) {
    uint32_t r0[NP], r1[NP], i0[NP], i1[NP];
    split2<NP>(sk, vr[0], vr[1], r0);
    split2<NP>(sk, vr[2], vr[3], r1);
    split2<NP>(sk, vi[0], vi[1], i0);
    split2<NP>(sk, vi[2], vi[3], i1);
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      reinterpret_cast<u2*>(pr[q])[h] = u2{r0[q], r1[q]};
      reinterpret_cast<u2*>(pi[q])[h] = u2{i0[q], i1[q]};
    }
  };
  auto make_g = [&]() {
    u4 a[NP], cr[NP], ci[NP];
    ldrec<NP>(s_bc.bs, xrec(16 * gst + dl, g, XT), a);
    ldrec<NP>(s_bc.cs_r, xrec(16 * gtt + dl, g, XT), cr);
    ldrec<NP>(s_bc.cs_i, xrec(16 * gtt + dl, g, XT), ci);
    // rows t, columns s  ->  lane: G[t = 4 g + i][s = dl]
    f4 yr = xmm_pp<NP, NPA>(cr, a, f4{0, 0, 0, 0}), yi = xmm_pp<NP, NPA>(ci, a, f4{0, 0, 0, 0});
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool k2 = 4 * g + i >= g_low;
      yr[i] = k2 ? yr[i] : 0.0f; yi[i] = k2 ? yi[i] : 0.0f;
    }
    put_half(s_g.g_r, s_g.g_i, xrec(16 * gst + dl, g, XT) * 2 + gtt, yr, yi);
    if (!use_phi) {
      // rows s, columns t  ->  lane: G[t = dl][s = 4 g + i]   (only the S recomputation reads it)
      f4 xr = xmm_pp<NP, NPA>(a, cr, f4{0, 0, 0, 0}), xi = xmm_pp<NP, NPA>(a, ci, f4{0, 0, 0, 0});
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool k1 = 4 * g + i <= g_lim;
        xr[i] = k1 ? xr[i] : 0.0f; xi[i] = k1 ? xi[i] : 0.0f;
      }
      put_half(s_g.gt_r, s_g.gt_i, xrec(16 * gtt + dl, g, XT) * 2 + gst, xr, xi);
    }
  };

  // ---- channel data of one chunk
  struct In { AccRaw4<Tin> u[2], de[2]; f4 th[2], dy[2], ph[2]; };
  auto in_load = [&](In& r, int c) {
    const int cc = c < 0 ? 0 : c;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int l = cc * XT + 16 * st + 4 * g;
      const int lc = l < L ? l : 0;
      r.u[st].load(gu + lc);
      r.de[st].load(gdl + lc);
      ldg_acc(r.th[st], gth + lc);
      ldg_acc(r.dy[st], gdy + lc);
      ldg_acc(r.ph[st], gph + lc);   // unconditional: a value defined on one path only would be copied at the join, before it has landed
    }
  };
  // everything ldg_acc has requested (B/C staging data and one chunk of channel data) has landed
  auto landed = [&](In& r) {
    if constexpr (sizeof(Tin) == 4) {
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+a"(r.u[0].v), "+a"(r.u[1].v), "+a"(r.de[0].v), "+a"(r.de[1].v), "+a"(r.th[0]), "+a"(r.th[1]),
                     "+a"(r.dy[0]), "+a"(r.dy[1]), "+a"(r.ph[0]), "+a"(r.ph[1]),
                     "+a"(m1_raw[0].v), "+a"(m1_raw[1].v), "+a"(m1_raw[2].v), "+a"(m1_raw[3].v),
                     "+a"(m2_raw.a), "+a"(m2_raw.b)
                   :
                   : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+a"(r.u[0].v), "+a"(r.u[1].v), "+a"(r.de[0].v), "+a"(r.de[1].v), "+a"(r.th[0]), "+a"(r.th[1]),
                     "+a"(r.dy[0]), "+a"(r.dy[1]), "+a"(r.ph[0]), "+a"(r.ph[1]),
                     "+a"(m1_raw[0].v), "+a"(m1_raw[1].v), "+a"(m1_raw[2].v), "+a"(m1_raw[3].v),
                     "+a"(m2_raw.a)
                   :
                   : "memory");
    }
  };

  // ---- state at the end of the current chunk and its adjoint: lane (dl, g) holds n = 4 g + i
  f4 Hr = {0, 0, 0, 0}, Hi = {0, 0, 0, 0}, Ar = {0, 0, 0, 0}, Ai = {0, 0, 0, 0};
  // checkpoint kb: fetched early into temporaries (eight loads in flight at once), applied later
  // rows of checkpoint 0 for this lane (clamped to valid rows; rows >= N are zeroed on use)
  const float* __restrict__ ck_row[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = 4 * g + i;
    ck_row[i] = p.hck + ((((size_t)b * p.nck) * N + (n < N ? n : 0)) * 2) * D + dc;
  }
  const size_t ck_stride = (size_t)N * 2 * D;
#pragma unroll
  for (int i = 0; i < 4; ++i) {                      // the state at the end of the sequence
    const size_t o = (size_t)(p.nck - 1) * ck_stride;
    const float vr = ck_row[i][o], vi = ck_row[i][o + D];
    Hr[i] = 4 * g + i < N ? vr : 0.0f;
    Hi[i] = 4 * g + i < N ? vi : 0.0f;
  }
  if (p.dhL && dok) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        const size_t o = ((((size_t)b * p.hs + p.ho) * D + d) * N + n) * 2;
        Ar[i] = p.dhL[o];
        Ai[i] = p.dhL[o + 1];
      }
    }
  }
  float accD = 0.0f;
  // dB / dC output: lane (at_n, at_x) of a closing wavefront adds element (row n = 2 k + at_n,
  // timestep at_x / 2, part at_x % 2) of its tile, k = 0..7
  const int at_n = lane >> 5, at_x = lane & 31;
  const size_t at_off = (((size_t)bb * N + at_n) * p.ld + so + 16 * (wave & 1) + (at_x >> 1)) * 2 + (at_x & 1);

  // dB / dC tile of the chunk starting at l_at, waiting in s_at[wave] (written by this wavefront)
  auto flush_dbc = [&](int l_at) {
    const float* __restrict__ at = s_at[wave];
    float* __restrict__ dst = (wave < 2 ? p.dC : p.dB) + at_off + (size_t)l_at * 2;
    const bool lok = l_at + 16 * (wave & 1) + (at_x >> 1) < L;
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = at[(2 * k + at_n) * XB_AS + at_x];   // all reads, then one wait
    sched_fence();
    if (lok) {
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (2 * k + at_n < N) atomicAdd(dst + (size_t)k * 4 * p.ld, v[k]);
    }
  };
  // checkpoints: the chunk that starts at a multiple of ck takes its start state from the store
  const int ck_chunks = p.ck / XT;
  int ck_left = (nchunks - 1) % ck_chunks + 1;      // chunks down to the next multiple of ck
  int kb_next = (nchunks - 1) / ck_chunks - 1;      // checkpoint holding the state before that chunk

  In inA, inB;
  bc_load(nchunks - 1);
  in_load(inA, nchunks - 1);
  landed(inA);
  __syncthreads();

  auto step = [&](int c, In& cur, In& nxt) {
    const int l0 = c * XT;
    // ================= phase 1: stage B/C, everything that does not need G
    bc_store(c);
    bc_load(c - 1);
    in_load(nxt, c - 1);
    const bool ck_here = (ck_left == 1) && l0 > 0;   // this chunk starts a checkpoint block
    float tr[4] = {0, 0, 0, 0}, ti[4] = {0, 0, 0, 0};
    if (ck_here) {                                   // its start state comes from the store: request it now
      const size_t o = (size_t)kb_next * ck_stride;
#pragma unroll
      for (int i = 0; i < 4; ++i) { tr[i] = ck_row[i][o]; ti[i] = ck_row[i][o + D]; }
    }
    if (c + 1 < nchunks) flush_dbc(l0 + XT);                           // dB / dC of the previous step
    __syncthreads();                                                   // (a) planes of chunk c visible
    make_g();

    // ---- per-channel vector work
    float th[2][4], w[8], dy[8], uu[8], de[8];
    bool big = false;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const bool ok = dok && (l0 + 16 * st + 4 * g < L);   // idle lanes must not feed the channel sums
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        th[st][i] = ok ? cur.th[st][i] : 0.0f;
        big |= fabsf(th[st][i]) > 4.0f;
        uu[4 * st + i] = ok ? cur.u[st].get(i) : 0.0f;
        de[4 * st + i] = ok ? cur.de[st].get(i) : 0.0f;
        dy[4 * st + i] = ok ? cur.dy[st][i] : 0.0f;
        w[4 * st + i] = de[4 * st + i] * uu[4 * st + i];
      }
    }
    if (__builtin_expect(__any(big), 0)) {
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int i = 0; i < 4; ++i) th[st][i] = (float)remainder((double)th[st][i], 6.283185307179586476925);
    }
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
    float cs[8], sn[8], vr[8], vi[8], qr[8], qi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float ph = th[e >> 2][e & 3] + ((e >> 2) ? off_b : off_a);
      sincos_small(ph, &sn[e], &cs[e]);
      vr[e] = cs[e] * w[e];
      vi[e] = -sn[e] * w[e];
      qr[e] = cs[e] * dy[e];
      qi[e] = -sn[e] * dy[e];
      accD = fmaf(dy[e], uu[e], accD);
    }
    const float cT = __shfl(cs[7], 48 + dl), sT = __shfl(sn[7], 48 + dl);
    u4 Vr[NP], Vi[NP], nVr[NP], nVi[NP], Qr[NP], Qi[NP], nQr[NP];
    split8<NP>(sk, vr, Vr); split8<NP>(sk, vi, Vi); split8<NP>(sk, qr, Qr); split8<NP>(sk, qi, Qi);
    nega<NP>(Vr, nVr); nega<NP>(Vi, nVi); nega<NP>(Qr, nQr);

    // ---- term of the phase gradient at the last step: - sum_n Im(conj(A') H_end)
    float tq = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) tq -= Ar[i] * Hi[i] - Ai[i] * Hr[i];
    tq += __shfl_xor(tq, 16);
    tq += __shfl_xor(tq, 32);

    // ---- into the frame of the chunk start: K_T = conj(P_T) H_end, J = conj(P_T) A'
    f4 Jr, Ji;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float hr = Hr[i], hi = Hi[i], ar = Ar[i], ai = Ai[i];
      Hr[i] = cT * hr + sT * hi;  Hi[i] = cT * hi - sT * hr;
      Jr[i] = cT * ar + sT * ai;  Ji[i] = cT * ai - sT * ar;
    }
    // ---- H = K_T - B^T V ;  A = J + conj(C)^T Q
    {
      u4 br[NP], bi[NP], cr[NP], ci[NP];
      ldrec16<NP>(s_bc.bt_r, xrec(dl, g, XN), br);
      ldrec16<NP>(s_bc.bt_i, xrec(dl, g, XN), bi);
      ldrec16<NP>(s_bc.ct_r, xrec(dl, g, XN), cr);
      ldrec16<NP>(s_bc.ct_i, xrec(dl, g, XN), ci);
      Hr = xmm_p<NP, NPA>(br, nVr, Hr);  Hr = xmm_p<NP, NPA>(bi, Vi, Hr);
      Hi = xmm_p<NP, NPA>(br, nVi, Hi);  Hi = xmm_p<NP, NPA>(bi, nVr, Hi);
      Ar = xmm_p<NP, NPA>(cr, Qr, Jr);   Ar = xmm_p<NP, NPA>(ci, Qi, Ar);
      Ai = xmm_p<NP, NPA>(cr, Qi, Ji);   Ai = xmm_p<NP, NPA>(ci, nQr, Ai);
    }
    // ---- gV, first term: sum_n conj(B_s[n]) J[n]
    f4 gVr[2], gVi[2];
    {
      const float x[8] = {Jr[0], Jr[1], Jr[2], Jr[3], Ji[0], Ji[1], Ji[2], Ji[3]};
      u4 jk[NP];
      split8<NP>(sk, x, jk);
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        u4 a[NP], ac[NP];
        ldrec<NP>(s_bc.bs, xrec(16 * st + dl, g, XT), a);
        ldrec<NP>(s_bc.bs_c, xrec(16 * st + dl, g, XT), ac);
        gVr[st] = xmm_p<NP, NPA>(a, jk, f4{0, 0, 0, 0});
        gVi[st] = xmm_p<NP, NPA>(ac, jk, f4{0, 0, 0, 0});
      }
    }
    // ---- sums over the channel: transpose Q, V, H, J through the private scratch
    {
      float* tqr = ws;
      float* tqi = ws + XB_TD;
      float* tvr = ws + 2 * XB_TD;
      float* tvi = ws + 3 * XB_TD;
      float* thr = ws + 4 * XB_TD;
      float* thi = thr + XB_ND;
      float* tjr = thr + 2 * XB_ND;
      float* tji = thr + 3 * XB_ND;
      const int dg = dl >> 2, dm = dl & 3;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int t = 16 * (e >> 2) + 4 * g + (e & 3);
        const int o = (dg * XB_TS + t) * 4 + dm;
        tqr[o] = qr[e]; tqi[o] = qi[e]; tvr[o] = vr[e]; tvi[o] = vi[e];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = (dg * XB_NS + 4 * g + i) * 4 + dm;
        thr[o] = Hr[i]; thi[o] = Hi[i]; tjr[o] = Jr[i]; tji[o] = Ji[i];
      }
      __builtin_amdgcn_wave_barrier();
      auto rec_t = [&](const float* re, const float* im, int tile, u4 (&o)[NPC]) {
        const f4 a = *reinterpret_cast<const f4*>(re + (g * XB_TS + 16 * tile + dl) * 4);
        const f4 bq = *reinterpret_cast<const f4*>(im + (g * XB_TS + 16 * tile + dl) * 4);
        const float x[8] = {a[0], a[1], a[2], a[3], bq[0], bq[1], bq[2], bq[3]};
        split8<NPC>(sk, x, o);
      };
      auto rec_n = [&](const float* re, const float* im, u4 (&o)[NPC]) {
        const f4 a = *reinterpret_cast<const f4*>(re + (g * XB_NS + dl) * 4);
        const f4 bq = *reinterpret_cast<const f4*>(im + (g * XB_NS + dl) * 4);
        const float x[8] = {a[0], a[1], a[2], a[3], bq[0], bq[1], bq[2], bq[3]};
        split8<NPC>(sk, x, o);
      };
      // Products in an order that keeps few operand records alive at a time.
      const f4 z = {0, 0, 0, 0};
      f4 pj[XB_JOBS];
      {
        u4 Q0[NPC], V0[NPC], V0i[NPC], Jc[NPC], Jci[NPC];
        rec_t(tqr, tqi, 0, Q0);
        rec_t(tvr, tvi, 0, V0);
        rot_i<NPC>(V0, V0i);                        // [-Vi, Vr]
        pj[0] = xmm<NPC>(Q0, V0, z);  pj[1] = xmm<NPC>(Q0, V0i, z);     // M tile (0,0): lane col s, rows t
        rec_n(tjr, tji, Jc);
        rot_mi<NPC>(Jc, Jci);                       // [ Ji, -Jr]
        pj[10] = xmm<NPC>(V0, Jc, z); pj[11] = xmm<NPC>(V0, Jci, z);    // X2 tile 0: lane col n, rows s
        {
          u4 Hc[NPC], Hci[NPC], Q1[NPC];
          rec_n(thr, thi, Hc);
          rot_i<NPC>(Hc, Hci);                      // [-Hi, Hr]
          pj[6] = xmm<NPC>(Q0, Hc, z);  pj[7] = xmm<NPC>(Q0, Hci, z);   // X1 tile 0: lane col n, rows t
          rec_t(tqr, tqi, 1, Q1);
          pj[8] = xmm<NPC>(Q1, Hc, z);  pj[9] = xmm<NPC>(Q1, Hci, z);   // X1 tile 1
          pj[2] = xmm<NPC>(Q1, V0, z);  pj[3] = xmm<NPC>(Q1, V0i, z);   // M tile (1,0)
          u4 V1[NPC], V1i[NPC];
          rec_t(tvr, tvi, 1, V1);
          rot_i<NPC>(V1, V1i);
          pj[4] = xmm<NPC>(Q1, V1, z);  pj[5] = xmm<NPC>(Q1, V1i, z);   // M tile (1,1)
          pj[12] = xmm<NPC>(V1, Jc, z); pj[13] = xmm<NPC>(V1, Jci, z);  // X2 tile 1
        }
      }
      // causal mask of the diagonal M tiles: keep rows t = 4 g + i >= column s = dl
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool keep = 4 * g + i >= dl;
        pj[0][i] = keep ? pj[0][i] : 0.0f; pj[1][i] = keep ? pj[1][i] : 0.0f;
        pj[4][i] = keep ? pj[4][i] : 0.0f; pj[5][i] = keep ? pj[5][i] : 0.0f;
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < XB_JOBS; ++j) *reinterpret_cast<f4*>(ws + (j * 64 + lane) * 4) = pj[j];
    }
    __syncthreads();                                                   // (b) G planes and partial sums visible

    // ================= phase 2
    // ---- Im(P_t S_t): read back from the forward pass, or recomputed (S = C.H + G.V)
    float phi[8];
    if (use_phi) {
#pragma unroll
      for (int e = 0; e < 8; ++e) phi[e] = cur.ph[e >> 2][e & 3];
    } else {
      const float x[8] = {Hr[0], Hr[1], Hr[2], Hr[3], Hi[0], Hi[1], Hi[2], Hi[3]};
      u4 hk[NP];
      split8<NP>(sk, x, hk);
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        u4 ar[NP], ai[NP], gr[NP], gi[NP];
        ldrec<NP>(s_bc.cs_r, xrec(16 * tt + dl, g, XT), ar);
        ldrec<NP>(s_bc.cs_i, xrec(16 * tt + dl, g, XT), ai);
        ldrec<NP>(s_g.gt_r, xrec(16 * tt + dl, g, XT), gr);
        ldrec<NP>(s_g.gt_i, xrec(16 * tt + dl, g, XT), gi);
        f4 Sr = xmm_p<NP, NPA>(ar, hk, f4{0, 0, 0, 0});
        f4 Si = xmm_p<NP, NPA>(ai, hk, f4{0, 0, 0, 0});
        Sr = xmm<NP>(gr, Vr, Sr);  Sr = xmm<NP>(gi, nVi, Sr);
        Si = xmm<NP>(gr, Vi, Si);  Si = xmm<NP>(gi, Vr, Si);
#pragma unroll
        for (int i = 0; i < 4; ++i) phi[4 * tt + i] = cs[4 * tt + i] * Si[i] + sn[4 * tt + i] * Sr[i];
      }
    }
    // ---- gV, second term: sum_{t>=s} conj(G[t,s]) Q_t
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      u4 gr[NP], gi[NP];
      ldrec<NP>(s_g.g_r, xrec(16 * st + dl, g, XT), gr);
      ldrec<NP>(s_g.g_i, xrec(16 * st + dl, g, XT), gi);
      gVr[st] = xmm<NP>(gr, Qr, gVr[st]);  gVr[st] = xmm<NP>(gi, Qi, gVr[st]);
      gVi[st] = xmm<NP>(gr, Qi, gVi[st]);  gVi[st] = xmm<NP>(gi, nQr, gVi[st]);
    }
    // ---- per-element results
    float dw[8], gth[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gr = gVr[e >> 2][e & 3], gi = gVi[e >> 2][e & 3];
      dw[e] = gr * cs[e] - gi * sn[e];
      gth[e] = gr * vi[e] - gi * vr[e] - dy[e] * phi[e];
    }
    gth[7] += (g == 3) ? tq : 0.0f;
    // suffix sums over the chunk: runs (st 1: g 3..0) then (st 0: g 3..0) in reverse time
    gth[2] += gth[3]; gth[1] += gth[2]; gth[0] += gth[1];
    gth[6] += gth[7]; gth[5] += gth[6]; gth[4] += gth[5];
    float ra = gth[0], rb = gth[4];
    {
      float ta = __shfl_down(ra, 16), tb = __shfl_down(rb, 16);
      if (g <= 2) { ra += ta; rb += tb; }
      ta = __shfl_down(ra, 32); tb = __shfl_down(rb, 32);
      if (g <= 1) { ra += ta; rb += tb; }
    }
    const float tot_b = __shfl(rb, dl);
    const float offb = rb - gth[4];
    const float offa = tot_b + ra - gth[0];
    f4 o_du[2], o_dd[2], o_dt[2];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      o_du[e >> 2][e & 3] = fmaf(de[e], dw[e], dsk * dy[e]);
      o_dd[e >> 2][e & 3] = uu[e] * dw[e];
      o_dt[e >> 2][e & 3] = gth[e] + ((e >> 2) ? offb : offa);
    }
    // ---- add the four partial M of the workgroup; keep them as [t][s] and [s][t]
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int idx = tid + 256 * k;                 // (job, lane') of the M jobs 0..5
      if (idx < 6 * 64) {
        const int job = idx >> 6, ln = idx & 63;
        f4 sum = *reinterpret_cast<const f4*>(&s_ws[0][idx * 4]);
#pragma unroll
        for (int wv = 1; wv < 4; ++wv) sum += *reinterpret_cast<const f4*>(&s_ws[wv][idx * 4]);
        const int tile = job >> 1, im = job & 1;     // tiles (0,0), (1,0), (1,1)
        const int tt = tile >= 1 ? 1 : 0, st = tile >= 2 ? 1 : 0;
        const int s = 16 * st + (ln & 15), t = 16 * tt + 4 * (ln >> 4);
        *reinterpret_cast<f4*>(&s_ms[2 + im][s * XB_MS + t]) = sum;
#pragma unroll
        for (int i = 0; i < 4; ++i) s_ms[im][(t + i) * XB_MS + s] = sum[i];
      }
    }
    // collect the loads issued at the top (long landed) before the stores join the in-order queue:
    // otherwise the next step's first use would have to wait for "everything", stores included
    landed(nxt);
#pragma unroll
    for (int i = 0; i < 4; ++i) { touch_vgpr(tr[i]); touch_vgpr(ti[i]); }
    if (dok) {
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const int l = l0 + 16 * st + 4 * g;
        if (l < L) {
          *reinterpret_cast<f4*>(p.du + row + l) = o_du[st];
          *reinterpret_cast<f4*>(p.ddelta + row + l) = o_dd[st];
          *reinterpret_cast<f4*>(p.dtheta + row + l) = o_dt[st];
        }
      }
    }
    __syncthreads();                                                   // (c) summed M visible

    // ---- dC (waves 0, 1: tiles 0, 1) and dB (waves 2, 3): X + M conj(B) / X + M^T conj(C)
    {
      const bool isC = wave < 2;
      const int tile = wave & 1;
      const int jx = (isC ? 6 : 10) + 2 * tile;
      f4 xr = *reinterpret_cast<const f4*>(&s_ws[0][(jx * 64 + lane) * 4]);
      f4 xi = *reinterpret_cast<const f4*>(&s_ws[0][((jx + 1) * 64 + lane) * 4]);
#pragma unroll
      for (int wv = 1; wv < 4; ++wv) {
        xr += *reinterpret_cast<const f4*>(&s_ws[wv][(jx * 64 + lane) * 4]);
        xi += *reinterpret_cast<const f4*>(&s_ws[wv][((jx + 1) * 64 + lane) * 4]);
      }
      const float* mre = s_ms[isC ? 0 : 2] + (16 * tile + dl) * XB_MS;
      const float* mim = s_ms[isC ? 1 : 3] + (16 * tile + dl) * XB_MS;
      u4 mr[NPC], mi[NPC], nmr[NPC], er[NPC], ei[NPC];
      {
        const f4 a = *reinterpret_cast<const f4*>(mre + 4 * g), a2 = *reinterpret_cast<const f4*>(mre + 16 + 4 * g);
        const f4 c2 = *reinterpret_cast<const f4*>(mim + 4 * g), c3 = *reinterpret_cast<const f4*>(mim + 16 + 4 * g);
        const float x[8] = {a[0], a[1], a[2], a[3], a2[0], a2[1], a2[2], a2[3]};
        const float y[8] = {c2[0], c2[1], c2[2], c2[3], c3[0], c3[1], c3[2], c3[3]};
        split8<NPC>(sk, x, mr);
        split8<NPC>(sk, y, mi);
        nega<NPC>(mr, nmr);
      }
      ldrec16<NPC>(isC ? s_bc.bt_r : s_bc.ct_r, xrec(dl, g, XN), er);
      ldrec16<NPC>(isC ? s_bc.bt_i : s_bc.ct_i, xrec(dl, g, XN), ei);
      xr = xmm_q<NPC, NPAC>(mr, er, xr);  xr = xmm_q<NPC, NPAC>(mi, ei, xr);
      xi = xmm_q<NPC, NPAC>(mi, er, xi);  xi = xmm_q<NPC, NPAC>(nmr, ei, xi);
      // Through a small LDS tile so that one atomic instruction covers two whole rows n of the
      // tile (16 timesteps x (re, im) = one 128-byte line each) instead of sixteen lines.
      float* __restrict__ at = s_at[wave];
      *reinterpret_cast<f4*>(at + dl * XB_AS + 8 * g) = f4{xr[0], xi[0], xr[1], xi[1]};
      *reinterpret_cast<f4*>(at + dl * XB_AS + 8 * g + 4) = f4{xr[2], xi[2], xr[3], xi[3]};
      // (the atomic adds themselves are issued by flush_dbc() in the next step, behind its loads)
    }
    // ---- next chunk: its end state is this chunk's start state (or the stored checkpoint)
    if (ck_here) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { Hr[i] = 4 * g + i < N ? tr[i] : 0.0f; Hi[i] = 4 * g + i < N ? ti[i] : 0.0f; }
      --kb_next;
    }
    if (--ck_left == 0) ck_left = ck_chunks;
    __syncthreads();                                                   // (d) planes, scratch and M free
  };

  for (int c = nchunks - 1; c >= 0; c -= 2) {
    step(c, inA, inB);
    if (c >= 1) step(c - 1, inB, inA);
  }
  flush_dbc(0);

  if (p.dh0 && dok) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        const size_t o = (((size_t)b * D + d) * N + n) * 2;
        p.dh0[o] = Ar[i];
        p.dh0[o + 1] = Ai[i];
      }
    }
  }
  if (p.dD && dok) {
    accD += __shfl_xor(accD, 16);
    accD += __shfl_xor(accD, 32);
    if (g == 0) atomicAdd(p.dD + d, accD);
  }
}

}  // namespace aussm
