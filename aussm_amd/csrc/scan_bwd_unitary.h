// Reverse scan (gradients) of the adaptive-unitary core scan.
//
// The recurrence h_l = a_l h_{l-1} + B_l w_l with |a_l| = 1 is invertible without loss:
// h_{l-1} = conj(a_l) (h_l - B_l w_l).  The backward pass therefore walks the sequence right to
// left ONCE, regenerating the states from the final state (re-synchronised at every checkpoint
// written by the forward pass) while it propagates the adjoint state g_l = dLoss/dh_l:
//     g_l      = conj(C_l) dy_l + conj(a_{l+1}) g_{l+1}
//     dC_l[n]  = sum_d dy_l conj(h_l)            dB_l[n] = sum_d w_l g_l          (w = delta u, real)
//     dw_l     = sum_n Re(conj(B_l) g_l)         du = dw delta + D dy,  ddelta = dw u
//     dtheta_l = -sum_n Im(conj(g_l) a_l h_{l-1})
// Gradient formulas: the recurrence form of
// extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_backward.cu:154-403.
#pragma once
#include "scan_common.h"

namespace aussm {

struct UniBwdArgs {
  const float* dy;      // [B,D,L]
  const float* dhL;     // [B,D,N,2] or null
  const void* u;        // [B,D,L] Tin
  const void* delta;    // [B,D,L] Tin
  const float* theta;   // [B,D,L]
  const void* Bm;       // [B,N,L,2] Tin
  const void* Cm;       // [B,N,L,2] Tin
  const float* Dskip;   // [D] or null
  const float* hck;     // [B,nck,N,2,D]
  float *du, *ddelta, *dtheta;   // [B,D,L]
  float *dB, *dC;       // [B,N,L,2]  accumulated into with atomics (caller zero-fills)
  float* dD;            // [D] or null, accumulated into
  float* dh0;           // [B,D,N,2] or null
  int B, D, N, L, ck, nck, ncg;
};

// Sum NV per-lane values over the 64 lanes (channels) of a wavefront through an LDS transpose.
// After the call lane c (< NV) holds the total of value c.  `red` is this wavefront's private
// scratch of 64 * RS floats.
template <int NV>
__device__ __forceinline__ float lane_transpose_sum(const float (&vals)[NV], float* red, int lane) {
  constexpr int RS = NV + 4;            // row stride in floats (keeps 16-byte alignment)
  constexpr int PARTS = 64 / NV;        // lanes per column
  float4* row = reinterpret_cast<float4*>(red + lane * RS);
#pragma unroll
  for (int j = 0; j < NV / 4; ++j) row[j] = make_float4(vals[4 * j], vals[4 * j + 1], vals[4 * j + 2], vals[4 * j + 3]);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int c = lane % NV, part = lane / NV;
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) acc += red[(i * PARTS + part) * RS + c];
#pragma unroll
  for (int o = NV; o < 64; o <<= 1) acc += __shfl_xor(acc, o, 64);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  return acc;
}

template <int NW, int NT, typename Tin>
__global__ __launch_bounds__(NT) void unitary_bwd_kernel(const UniBwdArgs p) {
  constexpr int NWV = NT / 64;
  constexpr int E = CH * T / NT;
  constexpr int RSTEP = NT / T;
  constexpr int NG = (NW < 4) ? NW : 4;          // states reduced per transpose batch
  constexpr int NV = 4 * NG;                     // values per batch: (dB re, dB im, dC re, dC im) per state
  constexpr int NB = NW / NG;                    // batches per step
  constexpr int AS = 4 * NW + 1;                 // padded row stride of the tile accumulator

  __shared__ float4 s_in[T * TS];                // (Re a, Im a, delta*u, dy) per (t, channel)
  __shared__ float2 s_part[NWV * T * TS];        // per wavefront partial (dw, dtheta)
  __shared__ __align__(16) float s_red[NWV * 64 * (NV + 4)];   // transpose scratch
  __shared__ float s_acc[NWV * T * AS];          // per wavefront dB/dC of the current tile

  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int b = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int N = p.N, L = p.L, D = p.D;
  const int n0 = wave * NW;
  const bool active = n0 < N;
  const int nwa = (N + NW - 1) / NW;
  const int d = d0 + lane;
  const bool dok = d < D;

  const Tin* __restrict__ gu = static_cast<const Tin*>(p.u);
  const Tin* __restrict__ gdl = static_cast<const Tin*>(p.delta);
  const Tin* __restrict__ gB = static_cast<const Tin*>(p.Bm);
  const Tin* __restrict__ gC = static_cast<const Tin*>(p.Cm);
  float* red = s_red + wave * 64 * (NV + 4);
  float* acc = s_acc + wave * T * AS;

  auto load_ck = [&](int kb, float (&xr)[NW], float (&xi)[NW]) {
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const int n = n0 + k;
      xr[k] = 0.f; xi[k] = 0.f;
      if (dok && n < N) {
        const size_t o = ((((size_t)b * p.nck + kb) * N + n) * 2) * D + d;
        xr[k] = p.hck[o];
        xi[k] = p.hck[o + D];
      }
    }
  };

  // ---- state h_L and adjoint g_L
  float hr[NW], hi[NW], gr[NW], gi[NW];
  load_ck(p.nck - 1, hr, hi);
#pragma unroll
  for (int k = 0; k < NW; ++k) {
    const int n = n0 + k;
    gr[k] = 0.f; gi[k] = 0.f;
    if (p.dhL && dok && n < N) {
      const size_t o = (((size_t)b * D + d) * N + n) * 2;
      gr[k] = p.dhL[o]; gi[k] = p.dhL[o + 1];
    }
  }

  // ---- staging-side mapping
  const int col = tid % T, row0 = tid / T;
  float ru[E], rdl[E], rth[E], rgy[E], dsk[E], accD[E];
  size_t goff[E];
  bool rowok[E];
#pragma unroll
  for (int k = 0; k < E; ++k) {
    const int dd = d0 + row0 + k * RSTEP;
    rowok[k] = dd < D;
    goff[k] = ((size_t)b * D + (rowok[k] ? dd : 0)) * L;
    dsk[k] = (p.Dskip && rowok[k]) ? p.Dskip[dd] : 0.f;
    accD[k] = 0.f;
  }
  auto load_tile = [&](int l0) {
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const int ll = l0 + col;
      const bool ok = rowok[k] && ll < L;
      const size_t o = goff[k] + (ok ? ll : 0);
      ru[k] = ok ? to_f32(gu[o]) : 0.f;
      rdl[k] = ok ? to_f32(gdl[o]) : 0.f;
      rth[k] = ok ? p.theta[o] : 0.f;
      rgy[k] = ok ? p.dy[o] : 0.f;
    }
  };

  const int ntiles = (L + T - 1) / T;
  load_tile((ntiles - 1) * T);

  for (int it = ntiles - 1; it >= 0; --it) {
    const int l0 = it * T;
    float eu[E], edl[E], egy[E];
#pragma unroll
    for (int k = 0; k < E; ++k) {
      float sn, cs;
      sincosf(rth[k], &sn, &cs);
      s_in[col * TS + row0 + k * RSTEP] = make_float4(cs, sn, rdl[k] * ru[k], rgy[k]);
      eu[k] = ru[k]; edl[k] = rdl[k]; egy[k] = rgy[k];
    }
    __syncthreads();
    if (it > 0) load_tile(l0 - T);

    const int tmax = (L - l0 < T) ? (L - l0) : T;
    if (active) {
      const size_t brow = ((size_t)b * N + n0) * L + l0;
      for (int t = tmax - 1; t >= 0; --t) {
        const float4 v = s_in[t * TS + lane];
        const float cs = v.x, sn = v.y, w = v.z, gy = v.w;
        float kacc = 0.f, qacc = 0.f;
#pragma unroll
        for (int bt = 0; bt < NB; ++bt) {
          float vals[NV];
#pragma unroll
          for (int j = 0; j < NG; ++j) {
            const int k = bt * NG + j;
            float2 bv = make_float2(0.f, 0.f), cv = make_float2(0.f, 0.f);
            if (n0 + k < N) {
              const size_t bi = brow + (size_t)k * L + t;
              bv = ld_c(gB, bi); cv = ld_c(gC, bi);
            }
            // adjoint of the read-out
            gr[k] = fmaf(cv.x, gy, gr[k]);
            gi[k] = fmaf(-cv.y, gy, gi[k]);
            vals[4 * j + 0] = w * gr[k];
            vals[4 * j + 1] = w * gi[k];
            vals[4 * j + 2] = gy * hr[k];
            vals[4 * j + 3] = -gy * hi[k];
            kacc = fmaf(bv.x, gr[k], kacc);
            kacc = fmaf(bv.y, gi[k], kacc);
            // p = a_l h_{l-1} = h_l - B_l w_l
            const float pr = fmaf(-bv.x, w, hr[k]);
            const float pi = fmaf(-bv.y, w, hi[k]);
            qacc = fmaf(gi[k], pr, qacc);
            qacc = fmaf(-gr[k], pi, qacc);
            // h_{l-1} = conj(a) p ;  adjoint carried to l-1 = conj(a) g
            hr[k] = fmaf(cs, pr, sn * pi);
            hi[k] = fmaf(cs, pi, -sn * pr);
            const float tg = fmaf(cs, gr[k], sn * gi[k]);
            gi[k] = fmaf(cs, gi[k], -sn * gr[k]);
            gr[k] = tg;
          }
          const float tot = lane_transpose_sum<NV>(vals, red, lane);
          if (lane < NV) acc[t * AS + bt * NV + lane] = tot;
        }
        s_part[(wave * T + t) * TS + lane] = make_float2(kacc, qacc);
      }
      // ---- flush this wavefront's dB/dC tile: lane = (t, re/im) -> 256 contiguous bytes per state row
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int ft = lane >> 1, fc = lane & 1;
      if (ft < tmax) {
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          if (n0 + k < N) {
            const size_t o = ((brow + (size_t)k * L + ft) << 1) + fc;
            atomicAdd(p.dB + o, acc[ft * AS + 4 * k + fc]);
            atomicAdd(p.dC + o, acc[ft * AS + 4 * k + 2 + fc]);
          }
        }
      }
      // ---- re-synchronise the regenerated state with the forward pass's checkpoint
      if (l0 > 0 && (l0 % p.ck) == 0) load_ck(l0 / p.ck - 1, hr, hi);
    }
    __syncthreads();

    // ---- epilogue: channel-wise gradients, coalesced along time
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const int ll = l0 + col;
      if (rowok[k] && ll < L) {
        float kk = 0.f, qq = 0.f;
        for (int w = 0; w < nwa; ++w) {
          const float2 pv = s_part[(w * T + col) * TS + row0 + k * RSTEP];
          kk += pv.x; qq += pv.y;
        }
        const size_t o = goff[k] + ll;
        p.du[o] = fmaf(kk, edl[k], dsk[k] * egy[k]);
        p.ddelta[o] = kk * eu[k];
        p.dtheta[o] = qq;
        accD[k] = fmaf(egy[k], eu[k], accD[k]);
      }
    }
  }

  if (p.dh0 && active && dok) {
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const int n = n0 + k;
      if (n < N) {
        const size_t o = (((size_t)b * D + d) * N + n) * 2;
        p.dh0[o] = gr[k]; p.dh0[o + 1] = gi[k];
      }
    }
  }
  if (p.dD) {
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const float s = half_wave_sum(accD[k]);
      if (col == 0 && rowok[k]) atomicAdd(p.dD + d0 + row0 + k * RSTEP, s);
    }
  }
}

}  // namespace aussm
