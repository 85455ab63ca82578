// Unitary scan on the matrix cores with operands prepared once per batch element.
//
// Mathematics, operand splitting and lane layout are those of scan_fwd_xdl.h / scan_bwd_xdl.h.
// Two things differ.
//
// 1. The channel-independent operands of a 32-step chunk -- B_t and C_t in the record orders the
//    products need, G[t,s] = sum_n C_t[n] B_s[n] in both orientations, all split into bf16
//    pieces -- do not depend on the channel group, yet every workgroup of a batch element used to
//    rebuild them (staging, two products, a dozen splits per chunk).  A light pre-pass
//    (unitary_px_prep_kernel, one workgroup per (batch, chunk)) now writes them once, as "images"
//    that have exactly the layout the scan kernels keep in LDS; a scan workgroup fetches an image
//    with loads that go from global memory straight into LDS.
//
// 2. Two wavefronts per SIMD.  A workgroup still owns (batch b, 64 channels) but has eight
//    wavefronts: w and w + 4 share the 16 channels of group w and take the chunks in turn.  The
//    work of a chunk c is cut into a part that does not need the carried state,
//        phase A:  phases, rotations, V = conj(P) delta u (split), Z = B^T V, then the carry
//                  H_{c+1} = P_T (H_c + Z)  (a handful of vector instructions),
//    and the rest,
//        phase B:  S = C.H_c + G.V, y = Re(P S) + D u.
//    Time is cut into intervals separated by workgroup barriers; in interval i the wavefront with
//    i % 2 == its half runs phase A of chunk i while its partner runs phase B of chunk i - 1.
//    One of the two is busy on the vector ALU while the other feeds the matrix pipe, the carry
//    passes through LDS once per chunk, and the same barrier publishes the next images.
#pragma once
#include "scan_bwd_xdl.h"
#include "scan_fwd_xdl.h"

namespace aussm {

// One workgroup (256 threads) per (batch element, chunk).  CHECK: the launch of a backward call, which has
// nothing to do when the forward call of the same tensors has left the images (its own instance, so that a
// profile tells the two launches of a training step apart).
template <typename Tin, bool CHECK>
__global__ __launch_bounds__(256) void unitary_px_prep_kernel(const PrepArgs p) {
  constexpr int NP = PX_NP;
  // (the records the images do not hold - [Ci, Cr] and [-Bi, Br] - are formed in registers where the products
  // need them: 48 KiB instead of 60 per workgroup, three workgroups per compute unit instead of two, so that one
  // workgroup's stores - half of its life - overlap the others' loads and products)
  struct PrepBC {
    u4 cs_r[NP][XT * 4];   // row t: [ Cr[4g..], -Ci[4g..] ]
    u4 bs[NP][XT * 4];     // row s: [ Br[4g..],  Bi[4g..] ]
    u4 bt_r[NP][XN * 4];   // row n: Br[t(g,e)][n]
    u4 bt_i[NP][XN * 4];
    u4 ct_r[NP][XN * 4];   // row n: Cr[t(g,e)][n]
    u4 ct_i[NP][XN * 4];
  };
  __shared__ PrepBC s_bc;
  __shared__ XbG<NP> s_g;

  // the images a forward call left behind are still those of these tensors: nothing to do
  if (CHECK && p.have) {
    bool same = true;
#pragma unroll
    for (int i = 0; i < 8; ++i) same &= __builtin_amdgcn_readfirstlane(p.have[i]) == p.want.w[i];
    if (same) return;
  }
  const int bb = blockIdx.x / p.nch, c = blockIdx.x % p.nch;
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int dl = lane & 15, g = lane >> 4;
  const int N = p.N, L = p.ld;
  const Tin* __restrict__ gB = static_cast<const Tin*>(p.Bm);
  const Tin* __restrict__ gC = static_cast<const Tin*>(p.Cm);
  const SplitK sk = make_splitk();

  for (int i = tid; i < (int)(sizeof(s_g) / 16); i += 256) reinterpret_cast<u4*>(&s_g)[i] = u4{0, 0, 0, 0};

  // ---- records of B_t and C_t (the two thread mappings of scan_bwd_xdl.h)
  {
    const int m1_t = tid & 31, m1_g = (tid >> 5) & 3;
    const bool m1_isB = tid >= 128;
    const Tin* __restrict__ src = m1_isB ? gB : gC;
    const int l = c * XT + m1_t;
    const bool tok = l < L;
    float x[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int n = 4 * m1_g + k;
      const bool ok = tok && n < N;
      RawC<Tin> r;
      r.load(src + (((size_t)bb * N + (ok ? n : 0)) * L + (ok ? l : 0)) * 2);
      x[k] = ok ? r.re() : 0.0f;
      x[4 + k] = ok ? r.im() : 0.0f;
    }
    u4 pc[NP];
    split8<NP>(sk, x, pc);                  // [re, im]
    const int o = xrec(m1_t, m1_g, XT);
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      if (m1_isB) s_bc.bs[q][o] = pc[q];
      else s_bc.cs_r[q][o] = u4{pc[q][0], pc[q][1], pc[q][2] ^ 0x80008000u, pc[q][3] ^ 0x80008000u};   // [re, -im]
    }
  }
  {
    const int m2_n = tid & 15, m2_g = (tid >> 4) & 3, m2_half = (tid >> 6) & 1;
    const bool m2_isC = tid >= 128;
    const Tin* __restrict__ src = m2_isC ? gC : gB;
    const int l2 = c * XT + 16 * m2_half + 4 * m2_g;
    const bool ok = m2_n < N && l2 < L;               // L is a multiple of 4: a run is in range as a whole
    RawC4<Tin> r;
    r.load(src + (((size_t)bb * N + (ok ? m2_n : 0)) * L + (ok ? l2 : 0)) * 2);
    float re[4], im[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) { re[j] = ok ? r.re(j) : 0.0f; im[j] = ok ? r.im(j) : 0.0f; }
    uint32_t a0[NP], a1[NP], b0[NP], b1[NP];
    split2<NP>(sk, re[0], re[1], a0);
    split2<NP>(sk, re[2], re[3], a1);
    split2<NP>(sk, im[0], im[1], b0);
    split2<NP>(sk, im[2], im[3], b1);
    const int o = xrec(m2_n, m2_g, XN) * 2 + m2_half;   // 8-byte half-record index
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      if (m2_isC) {
        reinterpret_cast<u2*>(s_bc.ct_r[q])[o] = u2{a0[q], a1[q]};
        reinterpret_cast<u2*>(s_bc.ct_i[q])[o] = u2{b0[q], b1[q]};
      } else {
        reinterpret_cast<u2*>(s_bc.bt_r[q])[o] = u2{a0[q], a1[q]};
        reinterpret_cast<u2*>(s_bc.bt_i[q])[o] = u2{b0[q], b1[q]};
      }
    }
  }
  __syncthreads();

  // ---- G in both orientations: wave 0 -> tile (tt 0, st 0), 1 -> (1, 0), 2 -> (1, 1)
  if (wave < 3) {
    const int gtt = wave >= 1 ? 1 : 0, gst = wave >= 2 ? 1 : 0;
    const int g_lim = (gtt == gst) ? dl : 64;          // keep rows s = 4 g + i <= column t = dl
    const int g_low = (gtt == gst) ? dl : -1;          // keep rows t = 4 g + i >= column s = dl
    u4 a[NP], cr[NP], ci[NP];
    ldrec<NP>(s_bc.bs, xrec(16 * gst + dl, g, XT), a);
    ldrec<NP>(s_bc.cs_r, xrec(16 * gtt + dl, g, XT), cr);
#pragma unroll
    for (int q = 0; q < NP; ++q) ci[q] = u4{cr[q][2] ^ 0x80008000u, cr[q][3] ^ 0x80008000u, cr[q][0], cr[q][1]};   // [im, re]
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
    // rows t, columns s  ->  lane: G[t = 4 g + i][s = dl]: half a record of row s (slots t)
    f4 yr = xmm<NP>(cr, a, f4{0, 0, 0, 0}), yi = xmm<NP>(ci, a, f4{0, 0, 0, 0});
    // rows s, columns t  ->  lane: G[t = dl][s = 4 g + i]: half a record of row t (slots s)
    f4 xr = xmm<NP>(a, cr, f4{0, 0, 0, 0}), xi = xmm<NP>(a, ci, f4{0, 0, 0, 0});
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool k2 = 4 * g + i >= g_low, k1 = 4 * g + i <= g_lim;
      yr[i] = k2 ? yr[i] : 0.0f; yi[i] = k2 ? yi[i] : 0.0f;
      xr[i] = k1 ? xr[i] : 0.0f; xi[i] = k1 ? xi[i] : 0.0f;
    }
    put_half(s_g.g_r, s_g.g_i, xrec(16 * gst + dl, g, XT) * 2 + gtt, yr, yi);
    put_half(s_g.gt_r, s_g.gt_i, xrec(16 * gtt + dl, g, XT) * 2 + gst, xr, xi);
  }
  __syncthreads();

  // ---- images
  const size_t ic = (size_t)bb * p.nch + c;
  if (p.fimg) {
    u4* __restrict__ o = p.fimg + ic * PXF_REC;
    constexpr int S16 = NP * XN * 4, S32 = NP * XT * 4;
    for (int i = tid; i < S16; i += 256) { o[i] = (&s_bc.bt_r[0][0])[i]; o[S16 + i] = (&s_bc.bt_i[0][0])[i]; }
    o += PXF_A;
    for (int i = tid; i < S32; i += 256) {
      o[i] = (&s_bc.cs_r[0][0])[i];
      o[S32 + i] = (&s_g.gt_r[0][0])[i];
      o[2 * S32 + i] = (&s_g.gt_i[0][0])[i];
    }
  }
  if (p.bimg) {
    u4* __restrict__ o = p.bimg + ic * PXB_REC;
    constexpr int S16 = NP * XN * 4, S32 = NP * XT * 4;
    for (int i = tid; i < S16; i += 256) {
      o[i] = (&s_bc.bt_r[0][0])[i];
      o[S16 + i] = (&s_bc.bt_i[0][0])[i];
      o[2 * S16 + i] = (&s_bc.ct_r[0][0])[i];
      o[3 * S16 + i] = (&s_bc.ct_i[0][0])[i];
    }
    o += PXB_A;
    for (int i = tid; i < S32; i += 256) {
      o[i] = (&s_bc.bs[0][0])[i];
      o[S32 + i] = (&s_g.g_r[0][0])[i];
      o[2 * S32 + i] = (&s_g.g_i[0][0])[i];
    }
  }
}

// ---- global memory -> LDS without passing through registers: a wavefront moves 64 records (1 KiB)
// per instruction, lane i's record to lds + i.  The data is in LDS once the wavefront's vector-memory
// counter says so (px_loads_done / px_wait) and a barrier has published it.  The instruction is
// written out: left to the compiler, every later LDS read of the wavefront waits for ALL of its
// outstanding loads of this kind, which would serialise the prefetch.
__device__ __forceinline__ void px_load_block(const u4* __restrict__ src, u4* lds, int lane) {
  const uint32_t dst = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds);
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src + lane), "s"(dst) : "memory");
}
__device__ __forceinline__ void px_loads_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// ... or all but the K youngest vector-memory operations of the wavefront have completed
template <int K>
__device__ __forceinline__ void px_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K) : "memory"); }
// Workgroup barrier that publishes LDS contents only.  __syncthreads() also drains the
// vector-memory counter, i.e. waits for every prefetch and store in flight.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Input loads whose completion is tracked by hand: the compiler is not told that they are loads, so
// it places no wait of its own (it cannot count the image loads above and would wait for all of
// them); every value loaded this way passes through px_landed() before its first use.
__device__ __forceinline__ void px_ldg(f4& dst, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void px_ldg(float2& dst, const void* p) {
  asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
// ... with a wave-uniform base pointer and a 32-bit byte offset per lane (one address register
// instead of two, and no 64-bit pointer kept per tensor)
__device__ __forceinline__ void px_ldg(f4& dst, const void* base, uint32_t off) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void px_ldg(float2& dst, const void* base, uint32_t off) {
  asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
template <typename Tin> struct PxRaw4;
template <> struct PxRaw4<float> {
  f4 v;
  __device__ __forceinline__ void load(const float* p) { px_ldg(v, p); }
  __device__ __forceinline__ void load(const void* base, uint32_t off) { px_ldg(v, base, off); }
  __device__ __forceinline__ float get(int i) const { return v[i]; }
};
template <> struct PxRaw4<bf16_t> {
  float2 v;
  __device__ __forceinline__ void load(const bf16_t* p) { px_ldg(v, p); }
  __device__ __forceinline__ void load(const void* base, uint32_t off) { px_ldg(v, base, off); }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = __float_as_uint(i < 2 ? v.x : v.y);
    return (i & 1) ? bf16_hi(w) : bf16_lo(w);
  }
};

// [x0..x3, y0..y3] with (x, y) = (Cr, -Ci)  ->  (Ci, Cr): the imaginary-part record of C from the real-part one
template <int NP>
__device__ __forceinline__ void cs_i_from_r(const u4 (&a)[NP], u4 (&o)[NP]) {
#pragma unroll
  for (int q = 0; q < NP; ++q) o[q] = u4{a[q][2] ^ 0x80008000u, a[q][3] ^ 0x80008000u, a[q][0], a[q][1]};
}

// Requires what unitary_fwd_xdl_kernel requires, and the forward images of the call's B_t / C_t.
// img: [B / ns batch elements][ceil(ld / 32)] images.
template <bool GATED, typename Tin = float>
__global__ __launch_bounds__(512) void unitary_fwd_px_kernel(const FwdArgs p, const u4* __restrict__ img, const ImgNote note) {
  constexpr int NP = PX_NP;
  constexpr int NPA = sizeof(Tin) == 2 ? 1 : NP;   // non-zero pieces of the B / C records
  __shared__ u4 s_a[3][PXF_A];                     // phase-A part of chunk i in slot i % 3
  __shared__ u4 s_b[3][PXF_B];                     // phase-B part of chunk i in slot i % 3
  __shared__ f4 s_h[2][4][2][64];                  // carried state H_c in [c % 2][channel group][re, im][lane]

  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int b = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int cg = wave & 3, hf = wave >> 2;
  const int dl = lane & 15, g = lane >> 4;
  const int D = p.D, N = p.N, L = p.L;
  const int d = d0 + cg * 16 + dl;
  const bool dok = d < D;
  const int dc = dok ? d : D - 1;
  const int bb = b / p.ns;
  const size_t so = (size_t)(b - bb * p.ns) * L;
  const size_t row = ((size_t)bb * D + dc) * p.ld + so;
  const Tin* __restrict__ gu = static_cast<const Tin*>(p.u) + row;
  const Tin* __restrict__ gdl = static_cast<const Tin*>(p.delta) + row;
  const float* __restrict__ gth = p.theta + row;
  const float* __restrict__ gz = GATED ? p.z + row : nullptr;
  const float dsk = (p.Dskip && dok) ? p.Dskip[dc] : 0.0f;
  const int nchunks = (L + XT - 1) / XT;
  const SplitK sk = make_splitk();
  // images of this (batch element, segment): chunk c of the segment is chunk so / 32 + c of the batch element
  const u4* __restrict__ gimg = img + ((size_t)bb * ((p.ld + XT - 1) / XT) + so / XT) * PXF_REC;

  // Image traffic of one interval: the phase-A part of chunk ca and the phase-B part of chunk cb,
  // 24 blocks of 64 records over the eight wavefronts, three per wavefront.  A block is loaded
  // into registers in one interval (img_load), written to its LDS slot at the start of the next
  // (img_store, once the load has landed) and published by the barrier that ends that interval.
  // Chunks past the end are clamped: their slots are free and the data is never used.  (Loads
  // that write LDS directly would spare the registers, but they are executed one at a time by
  // the memory pipeline and held up every other load and store of the compute unit.)
  u4 ireg[3];
  auto img_load = [&](int ca, int cb) {
    const int cac = ca < nchunks ? ca : nchunks - 1, cbc = cb < nchunks ? cb : nchunks - 1;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const int j = wave + 8 * k;                                     // wave-uniform block index
      const u4* src = j < PXF_A / 64 ? gimg + (size_t)cac * PXF_REC + j * 64
                                     : gimg + (size_t)cbc * PXF_REC + PXF_A + (j - PXF_A / 64) * 64;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(ireg[k]) : "v"(src + lane) : "memory");
    }
  };
  // K: vector-memory operations of the wavefront younger than the image loads being collected
  auto img_store = [&](int ca, int cb, auto kc) {
    constexpr int K = decltype(kc)::value;
    asm volatile("s_waitcnt vmcnt(%3)" : "+v"(ireg[0]), "+v"(ireg[1]), "+v"(ireg[2]) : "n"(K) : "memory");
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const int j = wave + 8 * k;
      if (j < PXF_A / 64) s_a[ca % 3][j * 64 + lane] = ireg[k];
      else s_b[cb % 3][(j - PXF_A / 64) * 64 + lane] = ireg[k];
    }
  };
  constexpr int N_IMG = 3;                          // image loads per wavefront and interval
  constexpr int N_IN = GATED ? 8 : 6;               // input loads per chunk

  // ---- channel data of one chunk: two runs of four timesteps per lane (clamped, zeroed on use)
  struct In { PxRaw4<Tin> u[2], de[2]; f4 th[2], z[2]; };
  auto in_load = [&](In& r, int c) {
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int l = c * XT + 16 * st + 4 * g;
      const int lc = l < L ? l : 0;
      r.u[st].load(gu + lc);
      r.de[st].load(gdl + lc);
      px_ldg(r.th[st], gth + lc);
      if (GATED) px_ldg(r.z[st], gz + lc);
    }
  };
  // the input loads have landed when at most K younger vector-memory operations are outstanding
  auto in_landed = [&](In& r, auto kc) {
    constexpr int K = decltype(kc)::value;
    if constexpr (GATED)
      asm volatile("s_waitcnt vmcnt(%8)"
                   : "+v"(r.u[0].v), "+v"(r.u[1].v), "+v"(r.de[0].v), "+v"(r.de[1].v), "+v"(r.th[0]), "+v"(r.th[1]),
                     "+v"(r.z[0]), "+v"(r.z[1])
                   : "n"(K)
                   : "memory");
    else
      asm volatile("s_waitcnt vmcnt(%6)"
                   : "+v"(r.u[0].v), "+v"(r.u[1].v), "+v"(r.de[0].v), "+v"(r.de[1].v), "+v"(r.th[0]), "+v"(r.th[1])
                   : "n"(K)
                   : "memory");
  };

  // ---- registers that pass from one phase of a wavefront to its next:
  //   gather (end of phase B, prologue) -> phase A of the next chunk: ph (running phases), w = delta u, un, zn
  //   phase A -> phase B of the same chunk: cs, sn, Vr, Vi, H (state at the chunk start), uu, zz
  float ph[8], w[8], un[8], zn[8];
  float cs[8], sn[8], uu[8], zz[8];
  u4 Vr[NP], Vi[NP];
  f4 Hr = {0, 0, 0, 0}, Hi = {0, 0, 0, 0};           // H_c: lane (dl, g) holds n = 4 g + i of channel dl
  In in;

  // Gather: the loaded inputs of chunk c become masked values and running phases (the registers are
  // refilled with the inputs of the chunk after it at the start of the wavefront's next phase A).
  auto gather = [&](int c, auto kc) {
    in_landed(in, kc);
    float th[2][4];
    bool big = false;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const bool ok = c * XT + 16 * st + 4 * g < L;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        th[st][k] = ok ? in.th[st][k] : 0.0f;
        big |= fabsf(th[st][k]) > 4.0f;
        un[4 * st + k] = in.u[st].get(k);
        w[4 * st + k] = ok ? in.de[st].get(k) * un[4 * st + k] : 0.0f;
        if (GATED) zn[4 * st + k] = in.z[st][k];
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      asm volatile("" : "+v"(un[e]), "+v"(w[e]), "+v"(th[e >> 2][e & 3]));
      if (GATED) asm volatile("" : "+v"(zn[e]));
    }
    // large phases are first reduced to (-pi, pi] so that the running sums stay small enough for
    // sincos_small and for fp32 sums of 32 terms (rare, uniform branch)
    if (__builtin_expect(__any(big), 0)) {
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int k = 0; k < 4; ++k) th[st][k] = (float)remainder((double)th[st][k], 6.283185307179586476925);
    }
#pragma unroll
    for (int st = 0; st < 2; ++st) { th[st][1] += th[st][0]; th[st][2] += th[st][1]; th[st][3] += th[st][2]; }
    // exclusive offsets over the order (st 0: g 0..3), (st 1: g 0..3)
    float sa, sb, tot_a, tot_b_;
    rows_prefix(th[0][3], g, &sa, &tot_a);
    rows_prefix(th[1][3], g, &sb, &tot_b_);
    const float off_a = sa - th[0][3];
    const float off_b = tot_a + sb - th[1][3];
#pragma unroll
    for (int e = 0; e < 8; ++e) ph[e] = th[e >> 2][e & 3] + ((e >> 2) ? off_b : off_a);
  };

  // ---- prologue: start state, first images, inputs of this wavefront's first chunk
  if (hf == 0) {
    f4 hr = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
    if (p.h0 && dok) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = 4 * g + i;
        if (n < N) {
          const size_t o = ((((size_t)b * p.hs + p.ho) * D + d) * N + n) * 2;
          hr[i] = p.h0[o];
          hi[i] = p.h0[o + 1];
        }
      }
    }
    s_h[0][cg][0][lane] = hr;
    s_h[0][cg][1][lane] = hi;
  }
  img_load(0, 0);
  img_store(0, 0, std::integral_constant<int, 0>{});
  img_load(1, 0);
  img_store(1, 0, std::integral_constant<int, 0>{});
  img_load(2, 1);                                   // collected in interval 0
  in_load(in, hf);
  gather(hf, std::integral_constant<int, 0>{});
  __syncthreads();

  const int ck_chunks = p.ck / XT;
  f4 yo[2], po[2];                                    // outputs of the last phase B, not yet stored
  int out_l0 = -1;
  auto flush_out = [&]() {
    if (out_l0 >= 0 && dok) {
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const int l = out_l0 + 16 * tt + 4 * g;
        if (l < L) {
          if (p.y) *reinterpret_cast<f4*>(p.y + row + l) = yo[tt];
          if (p.aux) *reinterpret_cast<f4*>(p.aux + row + l) = po[tt];     // Im(P_t S_t) for the backward pass
        }
      }
    }
    out_l0 = -1;
  };
  // ---- phase A of chunk c (interval i = c): rotations, V, Z = B^T V, carry.  Chunks past the end
  // run on zero input and zero phase: the state passes through unchanged, nothing is stored.
  auto phase_a = [&](int c) {
    const int i = c;
    // (nothing of the phase B before it is in flight but its image loads: it collected its inputs at its end)
    img_store(i + 2, i + 1, std::integral_constant<int, 0>{});
    flush_out();
    img_load(i + 3, i + 2);
    // the inputs of this wavefront's next chunk: behind the image loads, so that the wait for those at the start
    // of the next phase can leave them in flight - they are collected at that phase's end, two intervals from here
    in_load(in, c + 2);
    float vr[8], vi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      // (the lane's last step through the polynomial: in lane group 3 it is the rotation of the whole chunk,
      // which multiplies the carried state chunk after chunk - the hardware sine / cosine's 3e-7 against 9e-8
      // would show after a few thousand steps; everywhere else an error of that size does not accumulate)
      if (e == 7) sincos_small(ph[e], &sn[e], &cs[e]);
      else sincos_small_hw(ph[e], &sn[e], &cs[e]);
      vr[e] = cs[e] * w[e];
      vi[e] = -sn[e] * w[e];
      uu[e] = un[e];
      if (GATED) zz[e] = zn[e];
    }
    split8<NP>(sk, vr, Vr);
    split8<NP>(sk, vi, Vi);
    // rotation over the whole chunk: the element (st 1, g 3, i 3) is timestep 31
    const float cT = rows_last(cs[7]), sT = rows_last(sn[7]);
    // ---- Z = B^T V  (four independent accumulation chains)
    f4 z0 = {0, 0, 0, 0}, z1 = {0, 0, 0, 0}, z2 = {0, 0, 0, 0}, z3 = {0, 0, 0, 0};
    {
      const u4* sa_ = s_a[c % 3];
      u4 b_r[NP], b_i[NP], nVi[NP];
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        b_r[q] = sa_[q * (XN * 4) + xrec(dl, g, XN)];
        b_i[q] = sa_[(NP + q) * (XN * 4) + xrec(dl, g, XN)];
        nVi[q] = neg_bf16x8(Vi[q]);
      }
#pragma unroll
      for (int s = NP - 1; s >= 0; --s)
#pragma unroll
        for (int k = 0; k <= s; ++k)
          if (k < NPA) {
            z0 = xdl(b_r[k], Vr[s - k], z0);
            z1 = xdl(b_r[k], Vi[s - k], z1);
            z2 = xdl(b_i[k], nVi[s - k], z2);
            z3 = xdl(b_i[k], Vr[s - k], z3);
          }
    }
    // ---- carry: H_{c+1} = P_T (H_c + Z)
    Hr = s_h[c & 1][cg][0][lane];
    Hi = s_h[c & 1][cg][1][lane];
    f4 nr, ni;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float xr = Hr[k] + (z0[k] + z2[k]), xi = Hi[k] + (z1[k] + z3[k]);
      nr[k] = cT * xr - sT * xi;
      ni[k] = fmaf(cT, xi, sT * xr);
    }
    s_h[(c + 1) & 1][cg][0][lane] = nr;
    s_h[(c + 1) & 1][cg][1][lane] = ni;
    // ---- checkpoint: state at the end of every ck-step block and at the end of the sequence
    if (p.hck && dok && c < nchunks && ((c + 1) % ck_chunks == 0 || c == nchunks - 1)) {
      float* __restrict__ hp = p.hck + ((((size_t)b * p.nck + c / ck_chunks) * N + 4 * g) * 2) * D + dc;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (4 * g + k < N) { hp[(size_t)k * 2 * D] = nr[k]; hp[(size_t)k * 2 * D + D] = ni[k]; }
    }
    lds_barrier();
  };

  // ---- phase B of chunk c (interval i = c + 1): S = C.H + G.V, outputs; then the gather of chunk c + 2
  auto phase_b = [&](int c) {
    const int i = c + 1;
    // (behind the image loads it collects, the phase A before it issued the input loads and, now and then,
    // checkpoint stores: a wait that leaves only the input loads in flight is the safe side of both cases)
    img_store(i + 2, i + 1, std::integral_constant<int, N_IN>{});
    img_load(i + 3, i + 2);
    const u4* sb_ = s_b[c % 3];
    u4 hk[NP];
    {
      const float x[8] = {Hr[0], Hr[1], Hr[2], Hr[3], Hi[0], Hi[1], Hi[2], Hi[3]};
      split8<NP>(sk, x, hk);
    }
    u4 nVi[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) nVi[q] = neg_bf16x8(Vi[q]);
    f4 Sr[2], Si[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      u4 c_r[NP], c_i[NP], g_r[NP], g_i[NP];
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        c_r[q] = sb_[q * (XT * 4) + xrec(16 * tt + dl, g, XT)];
        g_r[q] = sb_[(NP + q) * (XT * 4) + xrec(16 * tt + dl, g, XT)];
        g_i[q] = sb_[(2 * NP + q) * (XT * 4) + xrec(16 * tt + dl, g, XT)];
      }
      cs_i_from_r<NP>(c_r, c_i);
      f4 a0 = {0, 0, 0, 0}, a1 = {0, 0, 0, 0}, a2 = {0, 0, 0, 0}, a3 = {0, 0, 0, 0};
#pragma unroll
      for (int s = NP - 1; s >= 0; --s)
#pragma unroll
        for (int k = 0; k <= s; ++k) {
          if (k < NPA) {
            a0 = xdl(c_r[k], hk[s - k], a0);
            a1 = xdl(c_i[k], hk[s - k], a1);
          }
          a2 = xdl(g_r[k], Vr[s - k], a2);
          a3 = xdl(g_r[k], Vi[s - k], a3);
          a0 = xdl(g_i[k], nVi[s - k], a0);
          a1 = xdl(g_i[k], Vr[s - k], a1);
        }
      Sr[tt] = a0 + a2;
      Si[tt] = a1 + a3;
    }
    // ---- outputs: rows 16 tt + 4 g + k of channel dl are this lane's own timesteps.  They are
    // stored at the start of this wavefront's next interval: a store issued here would still be
    // in flight at the wait that ends the interval (loads and stores share one counter).
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int e = 4 * tt + k;
        float v = cs[e] * Sr[tt][k] - sn[e] * Si[tt][k];
        v = fmaf(dsk, uu[e], v);
        if (GATED) v *= siluf_(zz[e]);
        yo[tt][k] = v;
        po[tt][k] = cs[e] * Si[tt][k] + sn[e] * Sr[tt][k];
      }
    }
    out_l0 = c * XT;
    // (younger than the inputs it collects: the image loads of this interval)
    gather(c + 2, std::integral_constant<int, N_IMG>{});
    lds_barrier();
  };
  // an interval in which this wavefront has no chunk: it still takes part in the image loads
  auto idle = [&](int i) {
    img_store(i + 2, i + 1, std::integral_constant<int, 0>{});
    flush_out();
    img_load(i + 3, i + 2);
    lds_barrier();
  };

  // Vector-memory operations of a wavefront are issued in this order.  Phase A: the stores of the
  // previous phase B, the image loads, the input loads of the wavefront's next chunk (and, now and then,
  // checkpoint stores at its end).  Phase B: the image loads.  Every load is collected one interval (images)
  // or two (inputs) after it was issued, and every wait is for the OLDEST loads in flight: the counter
  // retires in order, so a wait for a younger load would drain the input loads long before they are needed
  // (they used to be issued at the end of phase B, in front of the next image loads: 4 % slower).  The
  // loop body is straight-line code on purpose: a join of two paths would make the compiler move
  // live registers, loads in flight included.
  const int npairs = (nchunks + 1) / 2;               // chunks per wavefront (the last may be past the end)
  if (hf == 1) idle(0);
  for (int k = 0; k < npairs; ++k) {
    const int c = 2 * k + hf;
    phase_a(c);
    phase_b(c);
  }
  if (hf == 0) idle(2 * npairs);
  // The loads issued last (images and inputs of chunks past the end) are never used, but they are
  // still in flight: their destination registers must stay reserved until they have landed, or
  // whatever the code below keeps there - the addresses of the final stores - is overwritten.
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(ireg[0]), "+v"(ireg[1]), "+v"(ireg[2])::"memory");
  in_landed(in, std::integral_constant<int, 0>{});

  flush_out();
  if (p.aux && blockIdx.x == 0 && tid == 0) p.aux[(size_t)(p.B / p.ns) * D * p.ld] = __uint_as_float(p.auxtag);
  // (the pre-pass that wrote the images has finished: this kernel read them)
  if (note.dst && blockIdx.x == 0 && tid < 8) note.dst[tid] = note.stamp.w[tid];
  if (note.clear && blockIdx.x == 0 && tid == 0) *note.clear = 0.0f;
  if (p.hL && dok && hf == 0) {
    const f4 hr = s_h[0][cg][0][lane], hi = s_h[0][cg][1][lane];    // state after the last (possibly padding) chunk
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        const size_t o = (((size_t)b * D + d) * N + n) * 2;
        p.hL[o] = hr[i];
        p.hL[o + 1] = hi[i];
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// Backward scan on prepared operands, same organisation: eight wavefronts, partners w / w + 4 take
// the chunks in turn (in reverse order), intervals separated by one workgroup barrier.  With the
// notation of scan_bwd_xdl.h,
//   phase A of chunk c:  V, Q (split), Z = B^T V, W = conj(C)^T Q, then the carry
//                        J = conj(P_T) A',  H = conj(P_T) H_end - Z,  A = J + W   (H: state at the
//                        chunk start, recomputed backwards; A: its adjoint), then
//                        gV = conj(B) J + conj(G)^T Q and du / ddelta / dtheta
//   phase B of chunk c:  the sums over the channel behind dB, dC; then the rotations of the
//                        wavefront's next chunk.
// Every wavefront closes its own 16 channels' share of dB / dC (M conj(B), M^T conj(C)) and adds
// hands it over through LDS at the end of the interval.
// Im(P_t S_t) must have been left in p.aux by the forward call: a workgroup leaves at once when
// the buffer's tag says otherwise (p.tag_mode == 1; the launcher then lets the kernel of
// scan_bwd_xdl.h do the work, with tag_mode == 2).
//
// Memory operations.  All loads of a wavefront are issued at the start of its phase A: the images
// for two intervals ahead (straight into LDS), the inputs of its next chunk, the checkpoint that
// chunk may need, and Im(P S) for the phase B that follows.  They are collected by ONE wait in the
// middle of the next phase B, before that phase issues its first store or atomic: everything
// outstanding at that point is at least an interval old.  (A wait by count would have to know how
// many stores and atomics, which depend on masks, were issued after the loads.)
constexpr int PXB_TS = 33;                 // rows per channel group of the [t][d] scratch (32 + pad)
constexpr int PXB_TD = 4 * PXB_TS * 4;     // floats of one [t][d] array
constexpr int PXB_WS = 4 * PXB_TD;         // floats of a channel group's scratch: Q re, Q im, V re, V im
constexpr int PXB_NS = 17;                 // rows per channel group of the [n][d] arrays that later reuse it
constexpr int PXB_ND = 4 * PXB_NS * 4;
constexpr int PXB_RS = 68;                 // row stride of the dB / dC shares (64 floats + pad)
static_assert(4 * PXB_ND <= PXB_WS, "the scratch is reused");

template <int NPC, typename Tin = float>
__global__ __launch_bounds__(512) void unitary_bwd_px_kernel(const UniBwdArgs p, const u4* __restrict__ img) {
  constexpr int NP = PX_NP;
  constexpr int NPA = sizeof(Tin) == 2 ? 1 : NP, NPAC = sizeof(Tin) == 2 ? 1 : NPC;
  __shared__ u4 s_a[3][PXB_A];                     // bt, ct of chunk index r in slot r % 3 (phase A and the closing of phase B)
  __shared__ u4 s_b[2][PXB_B];                     // bs, g of chunk index r in slot r % 2 (phase A)
  __shared__ f4 s_x[4][4][64];                     // carry per channel group: H re, H im, A re, A im
  __shared__ __attribute__((aligned(16))) float s_ws[4][PXB_WS];   // per channel group: transposes
  // dC (rows 0..15) and dB (rows 16..31) of the chunk of one interval, one copy per channel group:
  // the wavefronts in phase B leave their shares here at the end of the interval, the wavefronts
  // that start the next interval add the four up and send the sums to global memory
  __shared__ __attribute__((aligned(16))) float s_tile[4][2 * XN * PXB_RS];

  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int b = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int cg = wave & 3, hf = wave >> 2;
  const int dl = lane & 15, g = lane >> 4;
  const int D = p.D, N = p.N, L = p.L;
  const int d = d0 + cg * 16 + dl;
  const bool dok = d < D;
  const int dc = dok ? d : D - 1;
  const int bb = b / p.ns;
  const size_t so = (size_t)(b - bb * p.ns) * L;
  const size_t row = ((size_t)bb * D + dc) * p.ld + so;
  const size_t tagpos = (size_t)(p.B / p.ns) * D * p.ld;
  if (p.tag_mode == 1 &&
      __builtin_amdgcn_readfirstlane(__float_as_uint(p.aux[tagpos])) != p.auxtag)
    return;
  // (the launcher only takes this kernel for tensors below 4 GiB: 32-bit byte offsets per lane)
  const uint32_t rowf = (uint32_t)(row * 4), rowt = (uint32_t)(row * sizeof(Tin));
  const float dsk = (p.Dskip && dok) ? p.Dskip[dc] : 0.0f;
  const int nchunks = (L + XT - 1) / XT;
  const int ck_chunks = p.ck / XT;
  const SplitK sk = make_splitk();
  float* __restrict__ ws = s_ws[cg];
  // images of this (batch element, segment); chunk index r counts from the END of the segment
  const u4* __restrict__ gimg = img + ((size_t)bb * ((p.ld + XT - 1) / XT) + so / XT) * PXB_REC;
  auto chunk_of = [&](int r) { const int c = nchunks - 1 - r; return c < 0 ? 0 : c; };   // clamped for the loads

  // Image loads, issued by the four wavefronts that start a phase B: parts of chunk indices ra (A
  // part) and rb (B part), 30 blocks of 64 records, up to eight per wavefront.
  auto img_load = [&](int ra, int rb) {
    const u4* __restrict__ ia = gimg + (size_t)chunk_of(ra) * PXB_REC;
    const u4* __restrict__ ib = gimg + (size_t)chunk_of(rb) * PXB_REC + PXB_A;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int j = cg + 4 * k;                                       // wave-uniform block index
      if (j < PXB_A / 64) px_load_block(ia + j * 64, &s_a[ra % 3][j * 64], lane);
      else if (j < PXB_REC / 64) px_load_block(ib + (j - PXB_A / 64) * 64, &s_b[rb & 1][(j - PXB_A / 64) * 64], lane);
    }
  };

  // ---- channel data of one chunk; issued at the start of a phase B, collected by the wait that ends it
  struct In { PxRaw4<Tin> u[2], de[2]; f4 th[2], dy[2]; };
  In in;
  f4 phi[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  const size_t ck_stride = (size_t)N * 2 * D;
  auto in_load = [&](int r) {
    const int c = chunk_of(r);
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int l = c * XT + 16 * st + 4 * g;
      const uint32_t lc = l < L ? l : 0;
      in.u[st].load(p.u, rowt + lc * (uint32_t)sizeof(Tin));
      in.de[st].load(p.delta, rowt + lc * (uint32_t)sizeof(Tin));
      px_ldg(in.th[st], p.theta, rowf + lc * 4);
      px_ldg(in.dy[st], p.dy, rowf + lc * 4);
      px_ldg(phi[st], p.aux, rowf + lc * 4);            // Im(P S) left by the forward call
    }
  };
  // everything the wavefront has loaded so far has landed
  auto all_landed = [&]() {
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(in.u[0].v), "+v"(in.u[1].v), "+v"(in.de[0].v), "+v"(in.de[1].v), "+v"(in.th[0]), "+v"(in.th[1]),
                   "+v"(in.dy[0]), "+v"(in.dy[1]), "+v"(phi[0]), "+v"(phi[1])
                 :
                 : "memory");
  };

  // ---- registers that pass between the phases of a wavefront
  float cs[8], sn[8], dy[8], uu[8], de[8];           // phase A -> phase B
  f4 Hr, Hi, Jr, Ji;                                 // state at the chunk start and J, lane (dl, g): n = 4 g + i
  float tq = 0.0f, accD = 0.0f;

  // What the phase-B wavefronts of interval i - 1 accumulated (the chunk of index i - 2) goes to
  // global memory: one wavefront per channel group takes eight of the 32 rows, one atomic
  // instruction per row (64 floats = the row's 32 timesteps x (re, im), two whole 128-byte lines).
  auto flush_acc = [&](int i) {
    const int rr = i - 2;
    if (rr < 0) return;
    const int c = nchunks - 1 - rr;
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int o = (8 * cg + k) * PXB_RS + lane;
      v[k] = (s_tile[0][o] + s_tile[1][o]) + (s_tile[2][o] + s_tile[3][o]);
    }
    if (c >= 0 && c * XT + (lane >> 1) < L) {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int rowi = 8 * cg + k, n = rowi & 15;
        if (n < N) {
          float* __restrict__ dst = (rowi < XN ? p.dC : p.dB) +
              (size_t)((uint32_t)((((size_t)bb * N + n) * p.ld + so) * 2) + (uint32_t)(c * XT) * 2 + lane);
          atomicAdd(dst, v[k]);
        }
      }
    }
  };

  // ---- gather of chunk index r (end of a phase B, prologue): the loaded inputs become masked
  // values, rotations and Im(P S) in the registers that phase A of the chunk starts from
  float ph_s[8];
  auto gather = [&](int r) {
    const int c = nchunks - 1 - r;                   // may be negative: a padding chunk (zero input, no stores)
    float th[2][4];
    bool big = false;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const bool ok = dok && c >= 0 && (c * XT + 16 * st + 4 * g < L);   // idle lanes must not feed the channel sums
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int e = 4 * st + k;
        th[st][k] = ok ? in.th[st][k] : 0.0f;
        big |= fabsf(th[st][k]) > 4.0f;
        uu[e] = ok ? in.u[st].get(k) : 0.0f;
        de[e] = ok ? in.de[st].get(k) : 0.0f;
        dy[e] = ok ? in.dy[st][k] : 0.0f;
        ph_s[e] = phi[st][k];
      }
    }
    if (__builtin_expect(__any(big), 0)) {
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int k = 0; k < 4; ++k) th[st][k] = (float)remainder((double)th[st][k], 6.283185307179586476925);
    }
#pragma unroll
    for (int st = 0; st < 2; ++st) { th[st][1] += th[st][0]; th[st][2] += th[st][1]; th[st][3] += th[st][2]; }
    float sa, sb, tot_a, tot_b_;
    rows_prefix(th[0][3], g, &sa, &tot_a);
    rows_prefix(th[1][3], g, &sb, &tot_b_);
    const float off_a = sa - th[0][3];
    const float off_b = tot_a + sb - th[1][3];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float ph = th[e >> 2][e & 3] + ((e >> 2) ? off_b : off_a);
      if (e == 7) sincos_small(ph, &sn[e], &cs[e]);       // (the chunk's rotation in lane group 3: see the forward kernel)
      else sincos_small_hw(ph, &sn[e], &cs[e]);
      accD = fmaf(dy[e], uu[e], accD);
    }
  };

  // ---- phase A of chunk index r
  auto phase_a = [&](int r) {
    const int c = nchunks - 1 - r;
    // A chunk that starts a checkpoint block hands the stored state on instead of the recomputed
    // one (this stops the drift of the backward recomputation).  Plain loads, once per block.
    const bool ck_here = c > 0 && c % ck_chunks == 0;     // (uniform)
    float ckv[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (ck_here) {
      const float* __restrict__ cp = p.hck + ((size_t)b * p.nck + (c / ck_chunks - 1)) * ck_stride + dc;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = 4 * g + i;
        if (n < N) { ckv[i] = cp[(size_t)n * 2 * D]; ckv[4 + i] = cp[(size_t)n * 2 * D + D]; }
      }
    }
    u4 Vr[NP], Vi[NP], Qr[NP], Qi[NP];
    float vr[8], vi[8];
    {
      float qr[8], qi[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float w = de[e] * uu[e];
        vr[e] = cs[e] * w;
        vi[e] = -sn[e] * w;
        qr[e] = cs[e] * dy[e];
        qi[e] = -sn[e] * dy[e];
      }
      split8<NP>(sk, vr, Vr); split8<NP>(sk, vi, Vi); split8<NP>(sk, qr, Qr); split8<NP>(sk, qi, Qi);
    }
    const float cT = rows_last(cs[7]), sT = rows_last(sn[7]);
    // ---- Z = B^T V, then W = conj(C)^T Q  (four independent accumulation chains each; one after
    // the other so that only one set of operand records is live at a time)
    f4 z0 = {0, 0, 0, 0}, z1 = z0, z2 = z0, z3 = z0, w0 = z0, w1 = z0, w2 = z0, w3 = z0;
    const u4* sa_ = s_a[r % 3];
    {
      u4 b_r[NP], b_i[NP], nVi[NP];
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        b_r[q] = sa_[q * (XN * 4) + xrec(dl, g, XN)];
        b_i[q] = sa_[(NP + q) * (XN * 4) + xrec(dl, g, XN)];
        nVi[q] = neg_bf16x8(Vi[q]);
      }
#pragma unroll
      for (int s = NP - 1; s >= 0; --s)
#pragma unroll
        for (int k = 0; k <= s; ++k)
          if (k < NPA) {
            z0 = xdl(b_r[k], Vr[s - k], z0);
            z1 = xdl(b_r[k], Vi[s - k], z1);
            z2 = xdl(b_i[k], nVi[s - k], z2);
            z3 = xdl(b_i[k], Vr[s - k], z3);
          }
    }
    __builtin_amdgcn_sched_barrier(0);
    {
      u4 c_r[NP], c_i[NP], nQr[NP];
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        c_r[q] = sa_[(2 * NP + q) * (XN * 4) + xrec(dl, g, XN)];
        c_i[q] = sa_[(3 * NP + q) * (XN * 4) + xrec(dl, g, XN)];
        nQr[q] = neg_bf16x8(Qr[q]);
      }
#pragma unroll
      for (int s = NP - 1; s >= 0; --s)
#pragma unroll
        for (int k = 0; k <= s; ++k)
          if (k < NPA) {
            w0 = xdl(c_r[k], Qr[s - k], w0);
            w1 = xdl(c_r[k], Qi[s - k], w1);
            w2 = xdl(c_i[k], Qi[s - k], w2);
            w3 = xdl(c_i[k], nQr[s - k], w3);
          }
    }
    __builtin_amdgcn_sched_barrier(0);
    // (here rather than at the start of the interval, where every wavefront of the workgroup has
    // memory operations to issue)
    flush_acc(r);
    // ---- carry
    const f4 er = s_x[cg][0][lane], ei = s_x[cg][1][lane], ar = s_x[cg][2][lane], ai = s_x[cg][3][lane];
    float t = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) t -= ar[i] * ei[i] - ai[i] * er[i];   // - sum_n Im(conj(A') H_end): phase gradient at the last step
    tq = rows_sum(t);
    f4 nAr, nAi;
    f4 pr, pi;                                            // what the next chunk takes as its end state
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      Hr[i] = cT * er[i] + sT * ei[i] - (z0[i] + z2[i]);
      Hi[i] = cT * ei[i] - sT * er[i] - (z1[i] + z3[i]);
      Jr[i] = cT * ar[i] + sT * ai[i];
      Ji[i] = cT * ai[i] - sT * ar[i];
      nAr[i] = Jr[i] + (w0[i] + w2[i]);
      nAi[i] = Ji[i] + (w1[i] + w3[i]);
      pr[i] = ck_here ? ckv[i] : Hr[i];
      pi[i] = ck_here ? ckv[4 + i] : Hi[i];
    }
    s_x[cg][0][lane] = pr;
    s_x[cg][1][lane] = pi;
    s_x[cg][2][lane] = nAr;
    s_x[cg][3][lane] = nAi;
    __builtin_amdgcn_sched_barrier(0);
    const u4* sb_ = s_b[r & 1];
    // ---- gV = sum_n conj(B_s[n]) J[n] + sum_{t>=s} conj(G[t,s]) Q_t   (one set of operand records live at a time)
    f4 gVr[2], gVi[2];
    {
      u4 jk[NP];
      const float x[8] = {Jr[0], Jr[1], Jr[2], Jr[3], Ji[0], Ji[1], Ji[2], Ji[3]};
      split8<NP>(sk, x, jk);
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        u4 a[NP], ac[NP];
#pragma unroll
        for (int q = 0; q < NP; ++q) a[q] = sb_[q * (XT * 4) + xrec(16 * st + dl, g, XT)];
        rot_i<NP>(a, ac);                                  // [-Bi, Br]
        gVr[st] = xmm_p<NP, NPA>(a, jk, f4{0, 0, 0, 0});
        gVi[st] = xmm_p<NP, NPA>(ac, jk, f4{0, 0, 0, 0});
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    {
      u4 nQr[NP];
#pragma unroll
      for (int q = 0; q < NP; ++q) nQr[q] = neg_bf16x8(Qr[q]);
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        u4 gr[NP], gi[NP];
#pragma unroll
        for (int q = 0; q < NP; ++q) {
          gr[q] = sb_[(NP + q) * (XT * 4) + xrec(16 * st + dl, g, XT)];
          gi[q] = sb_[(2 * NP + q) * (XT * 4) + xrec(16 * st + dl, g, XT)];
        }
        f4 a2 = {0, 0, 0, 0}, a3 = a2;
#pragma unroll
        for (int s = NP - 1; s >= 0; --s)
#pragma unroll
          for (int k = 0; k <= s; ++k) {
            a2 = xdl(gr[k], Qr[s - k], a2);
            a3 = xdl(gr[k], Qi[s - k], a3);
            gVr[st] = xdl(gi[k], Qi[s - k], gVr[st]);
            gVi[st] = xdl(gi[k], nQr[s - k], gVi[st]);
          }
        gVr[st] += a2;
        gVi[st] += a3;
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- per-element results
    {
      float dw[8], gth[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float gr = gVr[e >> 2][e & 3], gi = gVi[e >> 2][e & 3];
        dw[e] = gr * cs[e] - gi * sn[e];
        gth[e] = gr * vi[e] - gi * vr[e] - dy[e] * ph_s[e];
      }
      gth[7] += (g == 3) ? tq : 0.0f;
      // suffix sums over the chunk: runs (st 1: g 3..0) then (st 0: g 3..0) in reverse time
      gth[2] += gth[3]; gth[1] += gth[2]; gth[0] += gth[1];
      gth[6] += gth[7]; gth[5] += gth[6]; gth[4] += gth[5];
      float ra, rb, tot_a_, tot_b;
      rows_suffix(gth[0], g, &ra, &tot_a_);
      rows_suffix(gth[4], g, &rb, &tot_b);
      const float offb = rb - gth[4];
      const float offa = tot_b + ra - gth[0];
      if (dok && c >= 0) {
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const int l = c * XT + 16 * st + 4 * g;
          if (l < L) {
            f4 o_du, o_dd, o_dt;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int e = 4 * st + k;
              o_du[k] = fmaf(de[e], dw[e], dsk * dy[e]);
              o_dd[k] = uu[e] * dw[e];
              o_dt[k] = gth[e] + (st ? offb : offa);
            }
            const size_t ob = (size_t)(rowf + (uint32_t)l * 4);
            *reinterpret_cast<f4*>(reinterpret_cast<char*>(p.du) + ob) = o_du;
            *reinterpret_cast<f4*>(reinterpret_cast<char*>(p.ddelta) + ob) = o_dd;
            *reinterpret_cast<f4*>(reinterpret_cast<char*>(p.dtheta) + ob) = o_dt;
          }
        }
      }
    }
    lds_barrier();                 // (the shares of dB / dC of the interval before have been read)
    lds_barrier();
  };

  // ---- phase B of chunk index r
  auto phase_b = [&](int r) {
    const int c = nchunks - 1 - r;
    // ---- this wavefront's loads: the images of the next interval, the inputs of its next chunk
    img_load(r + 2, r + 2);
    const u4* sa_ = s_a[r % 3];
    f4 tr[4], ti[4];                                  // the four result tiles: dC 0, dC 1, dB 0, dB 1
    float vr[8], vi[8], qr[8], qi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float w = de[e] * uu[e];
      vr[e] = cs[e] * w;
      vi[e] = -sn[e] * w;
      qr[e] = cs[e] * dy[e];
      qi[e] = -sn[e] * dy[e];
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- sums over the channel: Q, V through the group's scratch with the channel in the K slots
    u4 Q0[NPC], Q1[NPC], V0[NPC], V1[NPC];
    {
      float* tqr = ws;
      float* tqi = ws + PXB_TD;
      float* tvr = ws + 2 * PXB_TD;
      float* tvi = ws + 3 * PXB_TD;
      const int dg = dl >> 2, dm = dl & 3;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int t = 16 * (e >> 2) + 4 * g + (e & 3);
        const int o = (dg * PXB_TS + t) * 4 + dm;
        tqr[o] = qr[e]; tqi[o] = qi[e]; tvr[o] = vr[e]; tvi[o] = vi[e];
      }
      __builtin_amdgcn_wave_barrier();
      auto rec_t = [&](const float* re, const float* im, int tile, u4 (&o)[NPC]) {
        const f4 a = *reinterpret_cast<const f4*>(re + (g * PXB_TS + 16 * tile + dl) * 4);
        const f4 bq = *reinterpret_cast<const f4*>(im + (g * PXB_TS + 16 * tile + dl) * 4);
        const float x[8] = {a[0], a[1], a[2], a[3], bq[0], bq[1], bq[2], bq[3]};
        split8<NPC>(sk, x, o);
      };
      rec_t(tqr, tqi, 0, Q0); rec_t(tqr, tqi, 1, Q1); rec_t(tvr, tvi, 0, V0); rec_t(tvr, tvi, 1, V1);
      __builtin_amdgcn_wave_barrier();
    }
    // M[t,s] = sum_d Q_t conj(V_s) in both orientations, as operands of the closing products:
    //   rows t, slots s (for dC): products with V as the row operand -> lane (col t = dl, rows s = 4 g + i)
    //   rows s, slots t (for dB): products with Q as the row operand -> lane (col s = dl, rows t = 4 g + i)
    const f4 z4 = {0, 0, 0, 0};
    // ---- X1[t,n] = sum_d Q_t conj(H[n]),  X2[s,n] = sum_d conj(V_s) J[n]: H, J through the scratch
    u4 Hc[NPC], Jc[NPC];
    {
      float* thr = ws;
      float* thi = ws + PXB_ND;
      float* tjr = ws + 2 * PXB_ND;
      float* tji = ws + 3 * PXB_ND;
      const int dg = dl >> 2, dm = dl & 3;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = (dg * PXB_NS + 4 * g + i) * 4 + dm;
        thr[o] = Hr[i]; thi[o] = Hi[i]; tjr[o] = Jr[i]; tji[o] = Ji[i];
      }
      __builtin_amdgcn_wave_barrier();
      auto rec_n = [&](const float* re, const float* im, u4 (&o)[NPC]) {
        const f4 a = *reinterpret_cast<const f4*>(re + (g * PXB_NS + dl) * 4);
        const f4 bq = *reinterpret_cast<const f4*>(im + (g * PXB_NS + dl) * 4);
        const float x[8] = {a[0], a[1], a[2], a[3], bq[0], bq[1], bq[2], bq[3]};
        split8<NPC>(sk, x, o);
      };
      rec_n(thr, thi, Hc); rec_n(tjr, tji, Jc);
      __builtin_amdgcn_wave_barrier();
    }
    __builtin_amdgcn_sched_barrier(0);
    in_load(r + 2);                // (not at the start of the interval, where every wavefront has loads to issue)
    // One output tile at a time: (dC, timesteps 16 tile ..), then (dB, ...).  The closing product
    // takes M with rows = the tile's timesteps and the other time index in the K slots: two 16 x 16
    // blocks of M side by side (the second one is zero above the block diagonal).
    auto close_tile = [&](bool isC, int tile) {
      // X term: lane (col n = dl, rows 4 g + i of the tile)
      const u4 (&R)[NPC] = tile ? (isC ? Q1 : V1) : (isC ? Q0 : V0);
      u4 Xi[NPC];                                           // [-Hi, Hr] or [Ji, -Jr]
      if (isC) rot_i<NPC>(Hc, Xi); else rot_mi<NPC>(Jc, Xi);
      f4 xr = isC ? xmm<NPC>(R, Hc, z4) : xmm<NPC>(R, Jc, z4);
      f4 xi = xmm<NPC>(R, Xi, z4);
      // M blocks with this tile's index in the rows (lane column = row index of the closing operand)
      f4 m0r, m0i, m1r, m1i;       // K-slot halves: other index 0..15, 16..31
      if (isC) {
        // rows t (tile), slots s: M[t][s] = sum_d Q_t conj(V_s), lane (col t = dl, rows s = 4 g + i)
        u4 Vx[NPC];                                         // [-Vi, Vr]
        rot_i<NPC>(V0, Vx);
        m0r = xmm<NPC>(V0, R, z4);  m0i = xmm<NPC>(Vx, R, z4);
        if (tile) { rot_i<NPC>(V1, Vx); m1r = xmm<NPC>(V1, R, z4); m1i = xmm<NPC>(Vx, R, z4); } else { m1r = z4; m1i = z4; }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // causal mask of the diagonal block: keep s = 4 g + i <= t = dl
          const bool keep = 4 * g + i <= dl;
          if (tile) { m1r[i] = keep ? m1r[i] : 0.0f; m1i[i] = keep ? m1i[i] : 0.0f; }
          else { m0r[i] = keep ? m0r[i] : 0.0f; m0i[i] = keep ? m0i[i] : 0.0f; }
        }
      } else {
        // rows s (tile), slots t: M[t][s], lane (col s = dl, rows t = 4 g + i)
        u4 Ri[NPC];                                         // [-Vi, Vr] of the tile
        rot_i<NPC>(R, Ri);
        if (tile) { m0r = z4; m0i = z4; } else { m0r = xmm<NPC>(Q0, R, z4); m0i = xmm<NPC>(Q0, Ri, z4); }
        m1r = xmm<NPC>(Q1, R, z4);  m1i = xmm<NPC>(Q1, Ri, z4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // keep t = 4 g + i >= s = dl in the diagonal block
          const bool keep = 4 * g + i >= dl;
          if (tile) { m1r[i] = keep ? m1r[i] : 0.0f; m1i[i] = keep ? m1i[i] : 0.0f; }
          else { m0r[i] = keep ? m0r[i] : 0.0f; m0i[i] = keep ? m0i[i] : 0.0f; }
        }
      }
      u4 mr[NPC], mi[NPC], nmr[NPC];
      {
        const float x[8] = {m0r[0], m0r[1], m0r[2], m0r[3], m1r[0], m1r[1], m1r[2], m1r[3]};
        const float y[8] = {m0i[0], m0i[1], m0i[2], m0i[3], m1i[0], m1i[1], m1i[2], m1i[3]};
        split8<NPC>(sk, x, mr);
        split8<NPC>(sk, y, mi);
        nega<NPC>(mr, nmr);
      }
      // dC = X1 + M conj(B);  dB = X2 + M^T conj(C): B or C of the chunk with the timestep in the K slots
      u4 er_[NPC], ei_[NPC];
#pragma unroll
      for (int q = 0; q < NPC; ++q) {
        er_[q] = sa_[((isC ? 0 : 2 * NP) + q) * (XN * 4) + xrec(dl, g, XN)];
        ei_[q] = sa_[((isC ? NP : 3 * NP) + q) * (XN * 4) + xrec(dl, g, XN)];
      }
      xr = xmm_q<NPC, NPAC>(mr, er_, xr);  xr = xmm_q<NPC, NPAC>(mi, ei_, xr);
      xi = xmm_q<NPC, NPAC>(mi, er_, xi);  xi = xmm_q<NPC, NPAC>(nmr, ei_, xi);
      tr[(isC ? 0 : 2) + tile] = xr;
      ti[(isC ? 0 : 2) + tile] = xi;
      __builtin_amdgcn_sched_barrier(0);
    };
    close_tile(true, 0);
    close_tile(true, 1);
    close_tile(false, 0);
    close_tile(false, 1);
    // ---- the one wait for this wavefront's loads: they were issued at the start of the phase, and
    // nothing else of it is in flight (the stores of the phase A before are an interval old)
    all_landed();
    gather(r + 2);
    lds_barrier();                 // the wavefronts in phase A have read the shares of the interval before
    // lane (row n = dl, timesteps 16 tile + 4 g + i) of each tile
    {
      float* __restrict__ tl = s_tile[cg];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float* __restrict__ at = tl + ((q >> 1) * XN + dl) * PXB_RS + (16 * (q & 1) + 4 * g) * 2;
        *reinterpret_cast<f4*>(at) = f4{tr[q][0], ti[q][0], tr[q][1], ti[q][1]};
        *reinterpret_cast<f4*>(at + 4) = f4{tr[q][2], ti[q][2], tr[q][3], ti[q][3]};
      }
    }
    lds_barrier();
  };
  // an interval in which this wavefront has no chunk
  auto idle = [&](int i) { flush_acc(i); lds_barrier(); lds_barrier(); };

  // ---- prologue: end state and its adjoint into the carry, first images, first inputs
  if (hf == 0) {
    f4 hr = {0, 0, 0, 0}, hi = hr, ar = hr, ai = hr;
    const float* __restrict__ cp = p.hck + ((size_t)b * p.nck + (p.nck - 1)) * ck_stride + dc;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        hr[i] = cp[(size_t)n * 2 * D];
        hi[i] = cp[(size_t)n * 2 * D + D];
        if (p.dhL && dok) {
          const size_t o = ((((size_t)b * p.hs + p.ho) * D + d) * N + n) * 2;
          ar[i] = p.dhL[o];
          ai[i] = p.dhL[o + 1];
        }
      }
    }
    s_x[cg][0][lane] = hr; s_x[cg][1][lane] = hi; s_x[cg][2][lane] = ar; s_x[cg][3][lane] = ai;
  }
  // images of chunk indices 0 and 1 (all eight wavefronts take part, here only)
  {
    const u4* __restrict__ i0 = gimg + (size_t)chunk_of(0) * PXB_REC;
    const u4* __restrict__ i1 = gimg + (size_t)chunk_of(1) * PXB_REC;
    for (int j = wave; j < PXB_REC / 64; j += 8) {
      if (j < PXB_A / 64) {
        px_load_block(i0 + j * 64, &s_a[0][j * 64], lane);
        px_load_block(i1 + j * 64, &s_a[1][j * 64], lane);
      } else {
        px_load_block(i0 + j * 64, &s_b[0][(j - PXB_A / 64) * 64], lane);
        px_load_block(i1 + j * 64, &s_b[1][(j - PXB_A / 64) * 64], lane);
      }
    }
  }
  in_load(hf);
  all_landed();
  gather(hf);
  __syncthreads();

  // Straight-line loop body (phase A, then phase B of the same chunk); the second half starts one
  // interval late and the first half idles through the last one.
  const int npairs = (nchunks + 1) / 2;
  if (hf == 1) idle(0);
  for (int k = 0; k < npairs; ++k) {
    const int r = 2 * k + hf;
    phase_a(r);
    phase_b(r);
  }
  if (hf == 0) {
    idle(2 * npairs);
    flush_acc(2 * npairs + 1);          // (what the second half accumulated in the last interval)
  }

  if (p.dh0 && dok && hf == 0) {
    const f4 ar = s_x[cg][2][lane], ai = s_x[cg][3][lane];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * g + i;
      if (n < N) {
        const size_t o = (((size_t)b * D + d) * N + n) * 2;
        p.dh0[o] = ar[i];
        p.dh0[o + 1] = ai[i];
      }
    }
  }
  if (p.dD && dok) {
    accD = rows_sum(accD);
    if (g == 0) atomicAdd(p.dD + d, accD);
  }
}

}  // namespace aussm
