// Reverse scan (gradients) of the complex and the real (S6) core scans.
//
// With |a_l| < 1 the recurrence cannot be run backwards (dividing by a_l amplifies rounding
// errors without bound), so the states are recomputed: the forward pass leaves a checkpoint
// every 16 timesteps, and for each 16-step tile, right to left, this kernel
//   1. re-runs the recurrence from the tile's checkpoint, keeping the 16 states in registers,
//   2. walks the tile backwards propagating the adjoint state g_l = dLoss/dh_l
//          g_l = conj(C_l) dy_l + conj(a_{l+1}) g_{l+1}
//      and emitting, with p_l = a_l h_{l-1} = h_l - B_l w_l and w = delta u,
//          dC_l[n] = sum_d dy_l conj(h_l)        dB_l[n] = sum_d w_l g_l
//          dw_l    = sum_n Re(conj(B_l) g_l)
//          complex: drho_l = sum_n Re(conj(g_l) p_l)     dtheta_l = -sum_n Im(conj(g_l) p_l)
//          real:    x = g_l h_{l-1} a_l;  dA[d,n] += x delta_l;  ddelta_l = sum_n x A[d,n] + dw_l u_l
// Gate: with z given the forward output was y = y_pre silu(z); dy is then scaled by silu(z) on the way in,
// y_pre = sum_n Re(C h) + D u is recomputed with the states (a fourth sum over the states), and
// dz = dy y_pre silu'(z) leaves with the other gradients.
// The work decomposition, LDS staging, wide scalar loads of B_t/C_t and the lane-transpose
// channel reduction are those of the unitary kernels.
// Reference semantics: extension-cpp/extension_cpp/ops.py:270-291 (complex), :349-356 (real),
// gradient structure of extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_complex.cu:358-660 and
// ssm_adaptive_real.cu:267-488, selective-scan call at ai-modules/wavesAI/model/aussm.py:791-802.
#pragma once
#include <type_traits>

#include "scan_bwd_unitary.h"
#include "scan_common.h"

namespace aussm {


constexpr int RT = 16;       // timesteps per tile == checkpoint interval of these kernels

// Eight consecutive records of a state row starting at timestep t0, safe at the ragged end of the
// sequence: in range -> one wide scalar load, otherwise element loads from clamped timesteps
// (the out-of-range timesteps carry zero weight in the scan, any finite value will do).
template <typename Tin>
__device__ __forceinline__ f32x16 ld_c8_safe(const Tin* p, size_t row, int t0, int L) {
  if (t0 + TG <= L) return ld_c8(p, row + t0);
  f32x16 r;
#pragma unroll
  for (int i = 0; i < TG; ++i) {
    const float2 v = ld_c(p, row + ((t0 + i < L) ? t0 + i : L - 1));
    r[2 * i] = v.x; r[2 * i + 1] = v.y;
  }
  return r;
}
template <typename Tin>
__device__ __forceinline__ f32x8 ld_r8_safe(const Tin* p, size_t row, int t0, int L) {
  const bool aligned = sizeof(Tin) == 4 || (((row + t0) & 1) == 0);
  if (t0 + TG <= L && aligned) return ld_r8(p, row + t0);
  f32x8 r;
#pragma unroll
  for (int i = 0; i < TG; ++i) r[i] = ld_r(p, row + ((t0 + i < L) ? t0 + i : L - 1));
  return r;
}

// FULL: the whole tile lies inside the sequence, wide loads are aligned and the wavefront owns NW
// existing states, known once per tile: no branch per load or state, so the compiler can issue the scalar loads of a tile ahead of their use.
template <bool FULL, typename Tin>
__device__ __forceinline__ f32x16 ld_c8_tile(const Tin* p, size_t row, int t0, int L) {
  if constexpr (FULL) return ld_c8(p, row + t0);
  else return ld_c8_safe(p, row, t0, L);
}
template <bool FULL, typename Tin>
__device__ __forceinline__ f32x8 ld_r8_tile(const Tin* p, size_t row, int t0, int L) {
  if constexpr (FULL) return ld_r8(p, row + t0);
  else return ld_r8_safe(p, row, t0, L);
}

// Column sums of 16 products per lane through LDS (the real scan's workgroups of eight wavefronts; the complex
// scan's use `lanes_sum16`).
// Lane (c = lane % 16, q = lane / 16) reads column c of the rows 16 (i / 4) + 4 q + i % 4, i = 0 .. 15: with a
// row stride of 20 floats the two q of a 32-lane half are 16 banks apart, and the 16-byte row writes of
// eight neighbouring lanes cover all banks.  finish() leaves the column's total in all four lanes.
constexpr int RED16_RS = 20;
struct LaneTranspose16 {
  float v[16];
  __device__ __forceinline__ void issue(const float (&vals)[16], float* red, int lane) {
    float4* row = reinterpret_cast<float4*>(red + lane * RED16_RS);
#pragma unroll
    for (int j = 0; j < 4; ++j) row[j] = make_float4(vals[4 * j], vals[4 * j + 1], vals[4 * j + 2], vals[4 * j + 3]);
    __builtin_amdgcn_wave_barrier();
    const float* colp = red + (4 * (lane >> 4)) * RED16_RS + (lane & 15);
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = colp[(16 * (i >> 2) + (i & 3)) * RED16_RS];
    sched_fence();
  }
  __device__ __forceinline__ float finish() {
#pragma unroll
    for (int s = 8; s >= 1; s >>= 1)
#pragma unroll
      for (int i = 0; i < s; ++i) v[i] += v[i + s];
    return rows_sum(v[0]);
  }
};

// Workgroups of four wavefronts (NT = 256) keep one slab of per-(timestep, channel) partial sums per
// wavefront and reduce 32 products per lane transpose.  Workgroups of eight wavefronts (NT = 512, two
// wavefronts per SIMD) fit with three planes of floats per wavefront instead of four-float records - complex:
// (dw, dtheta, drho), real: (dw, ddelta, y_pre), so the gated complex scan stays with four wavefronts - and with
// channel sums of 16 products at a time: through lane transposes in the real scan, on the vector ALU alone in the
// complex scan (`lanes_sum16`: row swaps and DPP; through LDS this reduction was two fifths of the complex kernel's
// time, while the real kernel, whose vector ALU is the busier, runs 4 % faster with the transposes).  The LDS the
// complex scan saves holds a fourth plane, the read-out before the gate, so the gated complex scan runs here too.  (Adding the partial sums of
// two wavefronts into one slab with LDS float atomics instead made the kernel 2.5 times slower: those run far below
// the rate of plain LDS writes.)
// PLANE4: the complex scan's workgroups of eight wavefronts with the fourth plane (calls that want dz).
template <int VAR, int NW, int NT, typename Tin, typename Tbc = Tin, bool PLANE4 = false>
__global__ __launch_bounds__(NT) void recompute_bwd_kernel(const RecBwdArgs p) {
  static_assert(VAR == VAR_COMPLEX || VAR == VAR_REAL, "unitary has its own kernel");
  constexpr int C = (VAR == VAR_REAL) ? 1 : 2;
  constexpr int NWV = NT / 64;
  constexpr int E = CH * RT / NT;
  constexpr int RSTEP = NT / RT;
  constexpr int NGRP = RT / TG;
  // rows reduced per lane transpose: a complex row fills the 32 columns, two real rows do
  constexpr int RPT = (VAR == VAR_REAL && NW % 2 == 0) ? 2 : 1;
  constexpr bool WIDE = NWV > 4;
  // real scan, two states per wavefront: the decay factors of the recomputed tile stay in registers for the
  // walk back (the exponential is a quarter-rate instruction; with more states per wavefront the registers are taken)
  constexpr bool KEEP_A = VAR == VAR_REAL && NW <= 2;
  constexpr int NRES = WIDE ? NGRP * NW * C : NGRP * NW / RPT;
  constexpr int PLANE = RT * TS;                           // floats of one plane of a slab
  static_assert(E >= 1, "tile too small for this workgroup size");

  __shared__ float4 s_in[RT * TS];                         // complex (Re a, Im a, w, dy); real (delta, w, dy, -)
  __shared__ float4 s_part[WIDE ? 1 : NWV * RT * TS];      // per wavefront partial (dw, dtheta|ddelta, drho, y_pre)
  constexpr int NPL = PLANE4 ? 4 : 3;                      // planes of a slab: gated complex (dw, dtheta, drho, y_pre)
  static_assert(!PLANE4 || (VAR == VAR_COMPLEX && NT == 512), "the fourth plane is the gated complex scan's");
  constexpr bool VALU_SUMS = WIDE && VAR == VAR_COMPLEX;   // channel sums without LDS
  constexpr int SLAB = NPL * PLANE;                        // floats of a wavefront's slab
  __shared__ float s_slab[WIDE ? NWV * SLAB : 1];   // WIDE: per wavefront, those sums as planes
  __shared__ __align__(16) float s_red[VALU_SUMS ? 4 : NWV * 64 * (WIDE ? RED16_RS : RED_RS)];  // lane-transpose scratch

  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  // vb: (batch, segment) pair of a launch that is split along the sequence, else the batch element
  const int vb = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int b = vb / p.ns, sg = vb - b * p.ns;
  const int lbeg = sg * p.L, ld = p.ld;
  const int tile0 = lbeg / RT;                              // index of the segment's first tile in the sequence
  const int N = p.N, D = p.D;
  const int L = (ld - lbeg < p.L) ? ld - lbeg : p.L;        // steps of this segment
  const int n0 = p.nbase + wave * NW;
  const bool active = n0 < N;
  const int d = d0 + lane;
  const bool dok = d < D;

  const Tin* __restrict__ gu = static_cast<const Tin*>(p.u);
  const Tin* __restrict__ gdl = static_cast<const Tin*>(p.delta);
  const Tbc* __restrict__ gB = static_cast<const Tbc*>(p.Bm);
  const Tbc* __restrict__ gC = static_cast<const Tbc*>(p.Cm);
  float* red = s_red + (VALU_SUMS ? 0 : wave * 64 * (WIDE ? RED16_RS : RED_RS));
  float4* part = s_part + (WIDE ? 0 : wave * RT * TS);
  float* slab = s_slab + (WIDE ? wave * SLAB : 0);
  const size_t row_base = ((size_t)b * N + n0) * ld + lbeg;

  // ---- per-lane constants and accumulators
  float a2[NW], an[NW], dAacc[NW], gr[NW], gi[NW];
#pragma unroll
  for (int k = 0; k < NW; ++k) {
    const int n = n0 + k;
    a2[k] = 0.f; an[k] = 0.f; dAacc[k] = 0.f; gr[k] = 0.f; gi[k] = 0.f;
    if (dok && n < N) {
      if (VAR == VAR_REAL) { an[k] = p.A[(size_t)d * N + n]; a2[k] = an[k] * LOG2E; }
      if (p.dhL) {
        const size_t o = (((size_t)vb * D + d) * N + n) * C;
        gr[k] = p.dhL[o];
        if (C == 2) gi[k] = p.dhL[o + 1];
      }
    }
  }

  // ---- start state of a tile: the checkpoint at the end of the previous 16-step block, or h0
  struct Start { float r[NW], i[NW]; };
  auto load_start = [&](Start& s, int it) {
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const int n = n0 + k;
      s.r[k] = 0.f; s.i[k] = 0.f;
      if (dok && n < N) {
        if (tile0 + it > 0) {
          const size_t o = ((((size_t)b * p.nck + (tile0 + it - 1)) * N + n) * C) * D + d;
          s.r[k] = p.hck[o];
          if (C == 2) s.i[k] = p.hck[o + D];
        } else if (p.h0) {
          const size_t o = (((size_t)b * D + d) * N + n) * C;
          s.r[k] = p.h0[o];
          if (C == 2) s.i[k] = p.h0[o + 1];
        }
      }
    }
  };
  auto collect_start = [&](Start& s) {
#pragma unroll
    for (int k = 0; k < NW; ++k) { touch_vgpr(s.r[k]); touch_vgpr(s.i[k]); }
  };

  // ---- staging-side mapping (lanes run along time) and the two raw register sets
  const int col = tid % RT, row0 = tid / RT;
  struct RawTile { Tin u[E], dl[E]; float th[E], rho[E], gy[E], zz[E]; };
  RawTile rdy, fly;
  float dsk[E], dbias[E], accD[E];
  size_t goff[E];
  bool rowok[E];
#pragma unroll
  for (int k = 0; k < E; ++k) {
    const int dd = d0 + row0 + k * RSTEP;
    rowok[k] = dd < D;
    goff[k] = ((size_t)b * D + (rowok[k] ? dd : 0)) * ld + lbeg;
    dsk[k] = (p.Dskip && rowok[k]) ? p.Dskip[dd] : 0.f;
    dbias[k] = (VAR == VAR_REAL && p.delta_bias && rowok[k]) ? p.delta_bias[dd] : 0.f;
    accD[k] = 0.f;
    rdy.u[k] = rdy.dl[k] = fly.u[k] = fly.dl[k] = Tin(0);
    rdy.th[k] = rdy.rho[k] = rdy.gy[k] = fly.th[k] = fly.rho[k] = fly.gy[k] = 0.f;
    rdy.zz[k] = fly.zz[k] = 0.f;
  }
  auto load_tile = [&](RawTile& r, int l0) {
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const int ll = (l0 + col < L) ? l0 + col : L - 1;
      const size_t o = goff[k] + ll;
      r.u[k] = gu[o];
      r.dl[k] = gdl[o];
      r.gy[k] = p.dy[o];
      if (p.z) r.zz[k] = p.z[o];
      if (VAR == VAR_COMPLEX) { r.th[k] = p.theta[o]; r.rho[k] = p.rho[o]; }
    }
  };
  auto collect_tile = [&](RawTile& r) {
#pragma unroll
    for (int k = 0; k < E; ++k) {
      touch_vgpr(r.u[k]); touch_vgpr(r.dl[k]); touch_vgpr(r.gy[k]); touch_vgpr(r.zz[k]);
      if (VAR == VAR_COMPLEX) { touch_vgpr(r.th[k]); touch_vgpr(r.rho[k]); }
    }
  };

  const int ntiles = (L + RT - 1) / RT;
  Start st_rdy, st_fly;
  load_tile(rdy, (ntiles - 1) * RT);
  load_start(st_rdy, ntiles - 1);
  collect_tile(rdy);
  collect_start(st_rdy);
  if (ntiles > 1) { load_tile(fly, (ntiles - 2) * RT); load_start(st_fly, ntiles - 2); }
  else { load_start(st_fly, 0); }

  // The walk consumes every B_t / C_t line of a tile through scalar loads that it waits for on the spot: the
  // lines of the tile that comes next are touched a tile ahead, during the staging maths, so that those loads
  // find them in the scalar cache.
  constexpr int RB = (int)sizeof(Tbc) * C;
  const bool full_group = active && n0 + NW <= N;          // wave-uniform
  TileWarm<NW, RB, RT> warm;
  if (full_group && ntiles * RT == L) {
    warm.issue(gB, gC, row_base + (size_t)(ntiles - 1) * RT, ld);
    warm.retire();
  }

  // a wavefront that owns no state never writes its slab: it clears it once, so that the epilogue can add the
  // slabs of all wavefronts without asking which of them exist (the first barrier of the loop orders the two)
  if (!active) {
    if constexpr (WIDE) {
      for (int i = lane; i < SLAB; i += 64) slab[i] = 0.f;
    } else {
      for (int i = lane; i < RT * TS; i += 64) part[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }

  for (int it = ntiles - 1; it >= 0; --it) {
    const int l0 = it * RT;
    const bool warm_next = full_group && it > 0;
    if (warm_next) warm.issue(gB, gC, row_base + l0 - RT, ld);

    // ---- stage
    float eu[E], edl[E], egy[E], eraw[E], egz[E];       // egz: dy silu'(z), for dz
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const bool ok = rowok[k] && l0 + col < L;
      eu[k] = ok ? to_f32(rdy.u[k]) : 0.f;
      egy[k] = ok ? rdy.gy[k] : 0.f;
      egz[k] = 0.f;
      if (p.z) {                                           // uniform
        egz[k] = egy[k] * dsiluf_(rdy.zz[k]);
        egy[k] *= siluf_(rdy.zz[k]);
      }
      float dl = ok ? to_f32(rdy.dl[k]) : 0.f;
      float4 rec;
      if (VAR == VAR_REAL) {
        dl += dbias[k];
        eraw[k] = dl;
        if (p.delta_softplus) dl = softplusf_(dl);
        if (!ok) dl = 0.f;                         // out-of-range steps: a = 1, w = 0
        rec = make_float4(dl, dl * eu[k], egy[k], 0.f);
      } else {
        eraw[k] = 0.f;
        float sn, cs;
        fast_sincosf(ok ? rdy.th[k] : 0.f, &sn, &cs);
        const float r = expf(ok ? rdy.rho[k] : 0.f);
        rec = make_float4(cs * r, sn * r, dl * eu[k], egy[k]);
      }
      edl[k] = dl;
      s_in[col * TS + row0 + k * RSTEP] = rec;
    }
    if (warm_next) warm.retire();
    __syncthreads();

    float rres[NRES > 0 ? NRES : 1];
    auto tile_body = [&](auto full_tag) {
      constexpr bool FULL = decltype(full_tag)::value;
      const size_t brow = row_base + l0;
      // ---- 1. recompute the tile's states from its start state
      float hsr[RT][NW], hsi[RT][NW];
      float cr_[NW], ci_[NW];
#pragma unroll
      for (int k = 0; k < NW; ++k) { cr_[k] = st_rdy.r[k]; ci_[k] = st_rdy.i[k]; }
#pragma unroll
      for (int g = 0; g < NGRP; ++g) {
        float rx[TG], ry[TG], rz[TG];
#pragma unroll
        for (int t = 0; t < TG; ++t) {
          const float4 v = s_in[(g * TG + t) * TS + lane];
          rx[t] = v.x; ry[t] = v.y; rz[t] = v.z;
        }
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          if (FULL || n0 + k < N) {                // wave-uniform; FULL: all NW states of the wavefront exist
            if constexpr (VAR == VAR_REAL) {
              const f32x8 bc = ld_r8_tile<FULL>(gB, brow + (size_t)k * ld - l0, l0 + g * TG, L);
#pragma unroll
              for (int t = 0; t < TG; ++t) {
                const float a = __builtin_amdgcn_exp2f(rx[t] * a2[k]);
                cr_[k] = fmaf(a, cr_[k], bc[t] * ry[t]);
                hsr[g * TG + t][k] = cr_[k];
                if constexpr (KEEP_A) hsi[g * TG + t][k] = a;        // (the real scan has no imaginary parts to keep there)
              }
            } else {
              const f32x16 bc = ld_c8_tile<FULL>(gB, brow + (size_t)k * ld - l0, l0 + g * TG, L);
#pragma unroll
              for (int t = 0; t < TG; ++t) {
                const float nr = fmaf(rx[t], cr_[k], fmaf(-ry[t], ci_[k], bc[2 * t] * rz[t]));
                const float ni = fmaf(rx[t], ci_[k], fmaf(ry[t], cr_[k], bc[2 * t + 1] * rz[t]));
                cr_[k] = nr; ci_[k] = ni;
                hsr[g * TG + t][k] = nr; hsi[g * TG + t][k] = ni;
              }
            }
          } else {
#pragma unroll
            for (int t = 0; t < TG; ++t) { hsr[g * TG + t][k] = 0.f; hsi[g * TG + t][k] = 0.f; }
          }
        }
      }

      // ---- 2. walk the tile backwards
#pragma unroll
      for (int g = NGRP - 1; g >= 0; --g) {
        float r0[TG], r1[TG], r2[TG], r3[TG];
#pragma unroll
        for (int t = 0; t < TG; ++t) {
          const float4 v = s_in[(g * TG + t) * TS + lane];
          r0[t] = v.x; r1[t] = v.y; r2[t] = v.z; r3[t] = v.w;
        }
        float kacc[TG], xacc[TG], zacc[TG], yacc[TG];
#pragma unroll
        for (int t = 0; t < TG; ++t) { kacc[t] = 0.f; xacc[t] = 0.f; zacc[t] = 0.f; yacc[t] = 0.f; }
        // products for the channel sums: [dB | dC] of TG steps; the narrow workgroups gather a complex row's 32
        // (or two real rows' 2 x 16) per transpose, the wide ones 16 at a time (vals, then vals + 16)
        float vals[RED_COLS];
#pragma unroll
        for (int j = 0; j < RED_COLS; ++j) vals[j] = 0.f;
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          if (FULL || n0 + k < N) {                // wave-uniform; FULL: all NW states of the wavefront exist
            if constexpr (VAR == VAR_REAL) {
              const f32x8 bc = ld_r8_tile<FULL>(gB, brow + (size_t)k * ld - l0, l0 + g * TG, L);
              const f32x8 cc = ld_r8_tile<FULL>(gC, brow + (size_t)k * ld - l0, l0 + g * TG, L);
              const int slot = (!WIDE && RPT == 2) ? (k & 1) : 0;
#pragma unroll
              for (int t = TG - 1; t >= 0; --t) {
                const int tt = g * TG + t;
                const float dlt = r0[t], w = r1[t], gy = r2[t];
                const float a = KEEP_A ? hsi[tt][k] : __builtin_amdgcn_exp2f(dlt * a2[k]);
                gr[k] = fmaf(cc[t], gy, gr[k]);
                vals[slot * 16 + t] = w * gr[k];
                vals[slot * 16 + 8 + t] = gy * hsr[tt][k];
                yacc[t] = fmaf(cc[t], hsr[tt][k], yacc[t]);
                kacc[t] = fmaf(bc[t], gr[k], kacc[t]);
                const float hprev = (tt > 0) ? hsr[tt > 0 ? tt - 1 : 0][k] : st_rdy.r[k];
                const float x = gr[k] * hprev * a;
                dAacc[k] = fmaf(x, dlt, dAacc[k]);
                xacc[t] = fmaf(x, an[k], xacc[t]);
                gr[k] *= a;
              }
            } else {
              const f32x16 bc = ld_c8_tile<FULL>(gB, brow + (size_t)k * ld - l0, l0 + g * TG, L);
              const f32x16 cc = ld_c8_tile<FULL>(gC, brow + (size_t)k * ld - l0, l0 + g * TG, L);
#pragma unroll
              for (int t = TG - 1; t >= 0; --t) {
                const int tt = g * TG + t;
                const float ar = r0[t], ai = r1[t], w = r2[t], gy = r3[t];
                const float br = bc[2 * t], bi = bc[2 * t + 1], cr = cc[2 * t], ci = cc[2 * t + 1];
                gr[k] = fmaf(cr, gy, gr[k]);
                gi[k] = fmaf(-ci, gy, gi[k]);
                vals[2 * t] = w * gr[k];
                vals[2 * t + 1] = w * gi[k];
                vals[2 * TG + 2 * t] = gy * hsr[tt][k];
                vals[2 * TG + 2 * t + 1] = -gy * hsi[tt][k];
                yacc[t] = fmaf(cr, hsr[tt][k], fmaf(-ci, hsi[tt][k], yacc[t]));
                kacc[t] = fmaf(br, gr[k], kacc[t]);
                kacc[t] = fmaf(bi, gi[k], kacc[t]);
                const float pr = fmaf(-br, w, hsr[tt][k]);
                const float pi = fmaf(-bi, w, hsi[tt][k]);
                zacc[t] = fmaf(gr[k], pr, zacc[t]);          // drho
                zacc[t] = fmaf(gi[k], pi, zacc[t]);
                xacc[t] = fmaf(gi[k], pr, xacc[t]);          // dtheta
                xacc[t] = fmaf(-gr[k], pi, xacc[t]);
                const float tg = fmaf(ar, gr[k], ai * gi[k]);
                gi[k] = fmaf(ar, gi[k], -ai * gr[k]);
                gr[k] = tg;
              }
            }
          }
          // channel reduction of this turn's (or row pair's) dB/dC products
          if constexpr (WIDE) {
            float half[16];
#pragma unroll
            for (int h = 0; h < C; ++h) {
#pragma unroll
              for (int j = 0; j < 16; ++j) half[j] = vals[16 * h + j];
              if constexpr (VALU_SUMS) {
                rres[(g * NW + k) * C + h] = lanes_sum16(half, lane);
              } else {
                LaneTranspose16 xs;
                xs.issue(half, red, lane);
                rres[(g * NW + k) * C + h] = xs.finish();
              }
            }
#pragma unroll
            for (int j = 0; j < RED_COLS; ++j) vals[j] = 0.f;
          } else if ((k % RPT) == RPT - 1) {
            LaneTranspose xs;
            xs.issue(vals, red, lane);
            rres[g * (NW / RPT) + k / RPT] = xs.finish();
#pragma unroll
            for (int j = 0; j < RED_COLS; ++j) vals[j] = 0.f;
          }
        }
        if constexpr (WIDE) {
#pragma unroll
          for (int t = 0; t < TG; ++t) {
            float* q = slab + (g * TG + t) * TS + lane;
            q[0] = kacc[t];
            q[PLANE] = xacc[t];
            q[2 * PLANE] = (VAR == VAR_COMPLEX) ? zacc[t] : yacc[t];
            if constexpr (PLANE4) q[3 * PLANE] = yacc[t];
          }
        } else {
#pragma unroll
          for (int t = 0; t < TG; ++t) part[(g * TG + t) * TS + lane] = make_float4(kacc[t], xacc[t], zacc[t], yacc[t]);
        }
      }
        };
    if (active) {
      // (bf16 rows start at even element offsets when L is even: wide loads stay 4-byte aligned)
      const bool full = (l0 + RT <= L) && (n0 + NW <= N) && (sizeof(Tbc) == 4 || (ld & 1) == 0);
      if (full) tile_body(std::true_type{});
      else tile_body(std::false_type{});
    }
    __syncthreads();

    // ---- the tile's vector-memory traffic in one burst: wait, new loads, atomics, stores
    if (it > 0) { collect_tile(fly); rdy = fly; }
    collect_start(st_fly);
    st_rdy = st_fly;
    sched_fence();
    if (it > 1) load_tile(fly, l0 - 2 * RT);
    if (it > 1) load_start(st_fly, it - 2);
    sched_fence();
    if (active) {
      if constexpr (WIDE) {
        // lane (g, c < 4) holds column 4 c + g of the 16: complex (dB | dC of a row: 8 steps x (re, im)), real (8 dB, 8 dC)
        // (lanes_sum16), or lanes 0 .. 15 one column each (LaneTranspose16)
        const int c = VALU_SUMS ? 4 * (lane & 3) + (lane >> 4) : (lane & 15);
        const bool mine = VALU_SUMS ? (lane & 12) == 0 : lane < 16;
#pragma unroll
        for (int g = 0; g < NGRP; ++g)
#pragma unroll
          for (int k = 0; k < NW; ++k)
#pragma unroll
            for (int h = 0; h < C; ++h) {
              const int t = l0 + g * TG;
              const float v = rres[(g * NW + k) * C + h];
              if (VAR == VAR_REAL) {
                float* dst = (c >> 3) ? p.dC : p.dB;
                if (mine && n0 + k < N && t + (c & 7) < L) atomicAdd(dst + row_base + (size_t)k * ld + t + (c & 7), v);
              } else {
                float* dst = h ? p.dC : p.dB;
                if (mine && n0 + k < N && t + (c >> 1) < L) atomicAdd(dst + 2 * (row_base + (size_t)k * ld + t) + c, v);
              }
            }
      } else {
#pragma unroll
      for (int g = 0; g < NGRP; ++g)
#pragma unroll
        for (int j = 0; j < NW / RPT; ++j) {
          const int c = lane & 31;
          const int t = l0 + g * TG;
          if (VAR == VAR_REAL) {
            // columns: [row slot 0: 8 dB, 8 dC][row slot 1: 8 dB, 8 dC]
            const int k = j * RPT + (c >> 4);
            const int tt = t + (c & 7);
            float* dst = ((c >> 3) & 1) ? p.dC : p.dB;
            if (n0 + k < N && (RPT == 2 || c < 16) && tt < L)
              atomicAdd(dst + row_base + (size_t)k * ld + tt, rres[g * (NW / RPT) + j]);
          } else {
            // columns: 16 floats of dB (re, im interleaved), then 16 of dC
            const int k = j;
            const int tt = t + ((c & 15) >> 1);
            float* dst = (c < 16) ? p.dB : p.dC;
            if (n0 + k < N && tt < L)
              atomicAdd(dst + 2 * (row_base + (size_t)k * ld + t) + (c & 15), rres[g * (NW / RPT) + j]);
          }
        }
      }
    }

    // ---- epilogue: channel-wise gradients, coalesced along time
    constexpr int NSLAB = NWV;
    float4 pv[E][NSLAB];
#pragma unroll
    for (int k = 0; k < E; ++k)
#pragma unroll
      for (int w = 0; w < NSLAB; ++w) {
        if constexpr (WIDE) {
          const float* q = s_slab + w * SLAB + col * TS + row0 + k * RSTEP;
          // (the slab of a wavefront without states holds zeros: it cleared it before the first tile)
          pv[k][w] = make_float4(q[0], q[PLANE], VAR == VAR_COMPLEX ? q[2 * PLANE] : 0.f,
                                 VAR == VAR_COMPLEX ? (PLANE4 ? q[3 * PLANE] : 0.f) : q[2 * PLANE]);
        } else {
          pv[k][w] = s_part[(w * RT + col) * TS + row0 + k * RSTEP];
        }
      }
    sched_fence();
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const int ll = l0 + col;
      float kk = 0.f, xx = 0.f, zz = 0.f, yy = 0.f;
#pragma unroll
      for (int w = 0; w < NSLAB; ++w) { kk += pv[k][w].x; xx += pv[k][w].y; zz += pv[k][w].z; yy += pv[k][w].w; }
      if (rowok[k] && ll < L) {
        const size_t o = goff[k] + ll;
        const bool acc = p.accum != 0;                   // uniform
        p.du[o] = acc ? fmaf(kk, edl[k], p.du[o]) : fmaf(kk, edl[k], dsk[k] * egy[k]);
        if (VAR == VAR_REAL) {
          float dd = fmaf(kk, eu[k], xx);
          if (p.delta_softplus) dd *= (eraw[k] > 20.0f) ? 1.0f : sigmoidf_(eraw[k]);
          p.ddelta[o] = acc ? p.ddelta[o] + dd : dd;
        } else {
          p.ddelta[o] = acc ? fmaf(kk, eu[k], p.ddelta[o]) : kk * eu[k];
          p.dtheta[o] = acc ? p.dtheta[o] + xx : xx;
          p.drho[o] = acc ? p.drho[o] + zz : zz;
        }
        if (p.dz) {                                        // y_pre = sum over the states + D u (the latter once)
          const float dzv = egz[k] * (acc ? yy : fmaf(dsk[k], eu[k], yy));
          p.dz[o] = acc ? p.dz[o] + dzv : dzv;
        }
        accD[k] = fmaf(egy[k], eu[k], accD[k]);
      }
    }
  }

  // ---- per-channel results
  if (active && dok) {
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const int n = n0 + k;
      if (n < N) {
        if (p.dh0) {
          const size_t o = (((size_t)vb * D + d) * N + n) * C;
          p.dh0[o] = gr[k];
          if (C == 2) p.dh0[o + 1] = gi[k];
        }
        if (VAR == VAR_REAL && p.dA) atomicAdd(p.dA + (size_t)d * N + n, dAacc[k]);
      }
    }
  }
  if (p.dD && !p.accum) {
#pragma unroll
    for (int k = 0; k < E; ++k) {
      float s = accD[k];
#pragma unroll
      for (int o = RT / 2; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
      if (col == 0 && rowok[k]) atomicAdd(p.dD + d0 + row0 + k * RSTEP, s);
    }
  }
}

}  // namespace aussm
