// The reference's operator, extension_cpp::ssm_adaptive_unitary, as fused kernels.
//
// Semantics (extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_forward.cu:83-181), per batch
// b, channel i, state j, with ut = silu(u), Bt_j = B_r[j] e^{i B_theta[j]}, Ct_j likewise:
//     theta_l[b,i,j] = sum_r x[i,j,r] u_l[b,r] + x_bias[i,j]
//     h_l[b,i,j]     = exp(i theta_l) h_{l-1}[b,i,j] + Bt_j dt_l[b,i] ut_l[b,i]
//     y_l[b,i]       = silu(z_l[b,i]) ( sum_j Re(Ct_j h_l[b,i,j]) + D_i ut_l[b,i] )
//
// The phase tensor theta[b,i,j,l] (n times the size of every other tensor) never exists in memory.
// A wavefront owns one (batch, channel) pair - with more than 16 states per channel, one block of 16
// states of it - and walks the sequence in tiles of 16 timesteps:
//   * the tile's RUNNING phases G = prefix(theta), a (16 states) x (16 timesteps) block, are one small matrix
//     product x[i] (16 x d) . U (d x 16) on the bf16 matrix cores with both operands split exactly into
//     three bf16 pieces (scan_fwd_xdl.h), i.e. fp32-accurate, where U is the tile of u[b] prefix-summed along
//     the tile (sum_{l' <= l} x.u_{l'} = x.U_l), plus (l + 1) x_bias.  The wavefront keeps its rows of x in
//     registers for the whole launch; the tiles of U, which all wavefronts of a batch element share, are
//     prepared once per call by a pre-pass (dropin_uprep_kernel) and copied into LDS once per workgroup;
//   * the product lands with the timestep along the lanes of a 16-lane row (lane = (timestep l,
//     state group g), states 4 g .. 4 g + 3 in registers), so the rest of the recurrence is prefix sums
//     along the row (DPP row shifts, no LDS): E = e^{iG}, p = conj(E) Bt w, R = h_in + prefix(p), h = E R.
//     This is the cumulative-sum form the reference itself uses (:122-162), tile by tile, with the state h
//     handed from tile to tile - so G restarts at every tile and stays small;
//   * one sincos per (state, timestep), the sum over the states inside the wavefront, the gates
//     and the skip fused into the store.
#pragma once
#include "dropin_args.h"
#include "scan_fwd_xdl.h"

namespace aussm {


// sin and cos of any argument without a branch: reduction by 2 pi in two fused steps (the result is as exact
// as the fp32 argument itself), then the hardware sine and cosine of the reduced argument (sincos_small_hw).  A
// branch here would cut the four state groups of a lane into separate blocks that the scheduler cannot interleave.
__device__ __forceinline__ void sincos_any(float x, float* sn, float* cs) {
  sincos_small_hw(x, sn, cs);
}

// silu and its derivative with the hardware reciprocal (1 ulp) instead of an IEEE division (ten instructions)
__device__ __forceinline__ float sigm_fast(float v) { return __builtin_amdgcn_rcpf(1.0f + __expf(-v)); }
__device__ __forceinline__ float silu_fast(float v) { return v * sigm_fast(v); }
__device__ __forceinline__ float dsilu_fast(float v) { const float sg = sigm_fast(v); return sg * (1.0f + v * (1.0f - sg)); }

// ---- prefix / suffix sums along a row of 16 lanes
template <int CTRL>
__device__ __forceinline__ float dpp_mov0(float v) {   // lanes that have no source read 0
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row_prefix(float v) {   // inclusive, towards higher lanes
  v += dpp_mov0<0x111>(v);    // row_shr:1
  v += dpp_mov0<0x112>(v);
  v += dpp_mov0<0x114>(v);
  v += dpp_mov0<0x118>(v);
  return v;
}
__device__ __forceinline__ float row_suffix(float v) {   // inclusive, towards lower lanes
  v += dpp_mov0<0x101>(v);    // row_shl:1
  v += dpp_mov0<0x102>(v);
  v += dpp_mov0<0x104>(v);
  v += dpp_mov0<0x108>(v);
  return v;
}
// value of the row's last / first lane in every lane of the row (DPP row broadcast: one vector instruction, where a
// lane shuffle is an LDS round trip on the chain that hands the state from tile to tile)
__device__ __forceinline__ float row_last(float v, int) { return dpp_perm<0x15F>(v); }    // row_newbcast:15
__device__ __forceinline__ float row_first(float v, int) { return dpp_perm<0x150>(v); }   // row_newbcast:0


// x (d, n, d) -> operand records.  Record (v = i nb + sb, ks, piece, lane = (row = lane % 16, g = lane / 16))
// holds x[i, 16 sb + row, 32 ks + 8 g .. + 7] (zero past the ends).  One thread per (v, ks, lane).
__global__ __launch_bounds__(256) void dropin_xprep_kernel(const float* __restrict__ x, u4* __restrict__ xp, int d, int n, int ks, int nb) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)d * nb * ks * 64) return;
  const int lane = (int)(idx & 63);
  const int k = (int)((idx >> 6) % ks), vc = (int)((idx >> 6) / ks);
  const int i = vc / nb, j = 16 * (vc % nb) + (lane & 15), g = lane >> 4;
  const SplitK sk = make_splitk();
  float v[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const int r = 32 * k + 8 * g + q;
    v[q] = (j < n && r < d) ? x[((size_t)i * n + j) * d + r] : 0.0f;
  }
  u4 pc[3];
  split8<3>(sk, v, pc);
#pragma unroll
  for (int q = 0; q < 3; ++q) xp[(((size_t)vc * ks + k) * 3 + q) * 64 + lane] = pc[q];
}

// Tiles of u as the second operand of the phase product, prepared once per call (one workgroup of 256
// threads per (batch element, tile)): record (k, piece, lane = (column l = lane % 16, g)) holds
// U[32 k + 8 g .. + 7][l], U[r][l] = sum_{l' <= l} u[b, r, l0 + l'] - the prefix sum along the tile - so that
// the matrix product hands the scan kernels the running phase G = prefix(theta) directly
// (sum_{l' <= l} sum_r x[i,j,r] u[r,l'] = sum_r x[i,j,r] U[r,l]); timesteps past L count as zero.  All KS steps the
// kernels are compiled for are written, the ones past ceil(d / 32) as zeros.
__global__ __launch_bounds__(256) void dropin_uprep_kernel(const float* __restrict__ u, u4* __restrict__ up, int d, int L,
                                                           int KS, int b0, int t0, int nt) {
  const int zb = blockIdx.x / nt, t = t0 + blockIdx.x % nt;
  const float* __restrict__ ub = u + (size_t)(b0 + zb) * d * L;
  u4* __restrict__ dst = up + (size_t)blockIdx.x * KS * 3 * 64;
  const SplitK sk = make_splitk();
  for (int rec = threadIdx.x; rec < KS * 64; rec += 256) {        // (whole wavefronts: 64 records per k)
    const int lane = rec & 63, k = rec >> 6;
    const int l = t * DT + (lane & 15), g = lane >> 4;
    float v[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int r = 32 * k + 8 * g + q;
      v[q] = row_prefix((r < d && l < L) ? ub[(size_t)r * L + l] : 0.0f);
    }
    u4 pc[3];
    split8<3>(sk, v, pc);
#pragma unroll
    for (int q = 0; q < 3; ++q) dst[(k * 3 + q) * 64 + lane] = pc[q];
  }
}

// A tile's records, global memory -> registers -> LDS, in two steps so that the loads of the next tile fly
// while the current one is computed.
template <int NT, int NREC, int KS>
__device__ __forceinline__ void tile_load(const u4* __restrict__ src, u4 (&v)[NREC], int tid) {
#pragma unroll
  for (int e = 0; e < NREC; ++e) {
    const int rec = tid + e * NT;
    if (rec < KS * 3 * 64) v[e] = src[rec];
  }
}
template <int NT, int NREC, int KS>
__device__ __forceinline__ void tile_store(const u4 (&v)[NREC], u4* __restrict__ dst, int tid) {
#pragma unroll
  for (int e = 0; e < NREC; ++e) {
    const int rec = tid + e * NT;
    if (rec < KS * 3 * 64) dst[rec] = v[e];
  }
}

// Workgroup = (batch b, NW consecutive (channel, state block) pairs), one pair per wavefront; the nb
// wavefronts of a channel are neighbours (nb divides NW) and add their shares of y through LDS.
// KS: 32-wide steps of the contraction over r (d <= 32 KS).
template <int KS, int NW>
__global__ __launch_bounds__(NW * 64) void dropin_fwd_kernel(const DropinArgs p) {
  __shared__ u4 s_u[2][KS * 3 * 64];
  __shared__ float s_y[2][NW][DT];                     // shares of y of the tile, by tile parity (nb > 1)
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int nb = p.nb, ncg = (p.d * nb + NW - 1) / NW;
  const int b = p.b0 + blockIdx.x / ncg, v = (blockIdx.x % ncg) * NW + wave;
  const int i = v / nb, sb = v % nb, j0 = 16 * sb;
  const bool iok = i < p.d;
  const int ic = iok ? i : p.d - 1, vc = ic * nb + sb;
  const int l_ = lane & 15, g = lane >> 4;
  const int d = p.d, n = p.n, L = p.L;
  const size_t row = ((size_t)b * d + ic) * L;
  const u4* __restrict__ upb = p.up + ((size_t)(b - p.up_b0) * p.up_nt - p.up_t0) * (KS * 3 * 64);   // + tile * (KS 3 64)

  // this wavefront's rows of x, split, for the whole launch
  u4 xa[KS][3];
#pragma unroll
  for (int k = 0; k < KS; ++k)
#pragma unroll
    for (int q = 0; q < 3; ++q)
      xa[k][q] = (k < p.ks) ? p.xp[(((size_t)vc * p.ks + k) * 3 + q) * 64 + lane] : u4{0, 0, 0, 0};
  // per state j = j0 + 4 g + a: bias, Bt, Ct, carried state
  float xb[4], btr[4], bti[4], ctr[4], cti[4], hr[4], hi[4];
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int j = j0 + 4 * g + a;
    const bool ok = j < n;
    const int jc = ok ? j : 0;
    xb[a] = ok ? p.x_bias[(size_t)ic * n + jc] : 0.0f;
    float s, c;
    fast_sincosf(p.B_th[jc], &s, &c);
    btr[a] = ok ? p.B_r[jc] * c : 0.0f;
    bti[a] = ok ? p.B_r[jc] * s : 0.0f;
    fast_sincosf(p.C_th[jc], &s, &c);
    ctr[a] = ok ? p.C_r[jc] * c : 0.0f;
    cti[a] = ok ? p.C_r[jc] * s : 0.0f;
    hr[a] = ok ? p.h_re[((size_t)b * d + ic) * n + jc] : 0.0f;
    hi[a] = ok ? p.h_im[((size_t)b * d + ic) * n + jc] : 0.0f;
  }
  const float Di = p.Dp[ic];
  const int ntiles = p.t1;

  constexpr int NT = NW * 64, NREC = (KS * 3 * 64 + NT - 1) / NT;
  u4 sv[NREC];
  tile_load<NT, NREC, KS>(upb + (size_t)p.t0 * (KS * 3 * 64), sv, tid);
  tile_store<NT, NREC, KS>(sv, s_u[p.t0 & 1], tid);
  __syncthreads();
  // the wavefront's own inputs, requested one tile ahead
  const int lf = p.t0 * DT + l_;
  float un = lf < L ? p.u[row + lf] : 0.0f, dtn = lf < L ? p.dt[row + lf] : 0.0f, zn = lf < L ? p.z[row + lf] : 0.0f;
  for (int t = p.t0; t < ntiles; ++t) {
    const int l0 = t * DT, l = l0 + l_;
    const bool lok = l < L;
    const float uv = un, dtv = dtn, zv = zn;
    {
      const bool nok = l + DT < L;
      un = nok ? p.u[row + l + DT] : 0.0f;
      dtn = nok ? p.dt[row + l + DT] : 0.0f;
      zn = nok ? p.z[row + l + DT] : 0.0f;
    }
    if (t + 1 < ntiles) tile_load<NT, NREC, KS>(upb + (size_t)(t + 1) * (KS * 3 * 64), sv, tid);
    // ---- running phases of the tile, less the bias: lane (column l, rows j = 4 g + a)
    f4 th = {0, 0, 0, 0};
    const u4* su = s_u[t & 1];
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      u4 ubk[3];
#pragma unroll
      for (int q = 0; q < 3; ++q) ubk[q] = su[(k * 3 + q) * 64 + lane];
      th = xmm<3>(xa[k], ubk, th);
    }
    const float ut = silu_fast(uv), w = dtv * ut;
    const float cnt = (float)(min(l_ + 1, L - l0));      // timesteps of the tile up to this one that exist
    float ysum = 0.0f;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const float G = fmaf(xb[a], cnt, th[a]);
      float sn, cs;
      sincos_any(G, &sn, &cs);
      // p = conj(E) Bt w
      const float pr = (cs * btr[a] + sn * bti[a]) * w, pi = (cs * bti[a] - sn * btr[a]) * w;
      const float Rr = hr[a] + row_prefix(pr), Ri = hi[a] + row_prefix(pi);
      // h = E R
      const float her = cs * Rr - sn * Ri, hei = cs * Ri + sn * Rr;
      ysum += ctr[a] * her - cti[a] * hei;
      hr[a] = row_last(her, lane);
      hi[a] = row_last(hei, lane);
    }
    ysum = rows_sum(ysum);
    if (nb == 1) {
      if (p.y && iok && lok && g == 0) p.y[row + l] = silu_fast(zv) * (ysum + Di * ut);
    } else if (g == 0) {
      s_y[t & 1][wave][l_] = ysum;
    }
    if (t + 1 < ntiles) tile_store<NT, NREC, KS>(sv, s_u[(t + 1) & 1], tid);
    __syncthreads();
    if (nb > 1 && sb == 0 && g == 0 && p.y && iok && lok) {      // the channel's first wavefront adds the shares up
      float tot = ysum;
      for (int k = 1; k < nb; ++k) tot += s_y[t & 1][wave + k][l_];
      p.y[row + l] = silu_fast(zv) * (tot + Di * ut);
    }
  }
  if (p.nh_re && iok && l_ == 0) {
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int j = j0 + 4 * g + a;
      if (j < n) {
        p.nh_re[((size_t)b * d + i) * n + j] = hr[a];
        p.nh_im[((size_t)b * d + i) * n + j] = hi[a];
      }
    }
  }
}

// ---- backward ---------------------------------------------------------------------------------
//
// Reverse sweep of the same tiles (the reference's ssm_adaptive_unitary_backward.cu:90-330 computes the
// same gradients from the same twelve inputs).  With hats for adjoints (hat h = dL/dRe h + i dL/dIm h),
// a_l = grad_y_l silu(z_l), and inside a tile G, E, p, R, h as in the forward kernel:
//     hat R_l = conj(E_l) a_l conj(Ct)                      (+ conj(E_last) hat h_out at the tile's last step)
//     hat p_s = sum_{l >= s} hat R_l,      hat h_in = hat p_first
//     hat w_s = Re(E_s conj(Bt) hat p_s)   summed over the states
//     hat G_l = -Im(conj(a_l conj(Ct)) h_l) + Im(conj(hat p_l) p_l)   (- Im(conj(hat h_out) h_last) at the last step)
//     hat theta_s = sum_{l >= s} hat G_l                    (suffix sum inside the tile only: the state handed
//                                                            to the next tile carries the rotation)
//     hat Bt += E_s w_s hat p_s,   hat Ct += a_l conj(h_l),   hat D += a_l ut_l
// The state at the end of each tile is recovered backwards (the recurrence is unitary, so this is
// stable): R_last = conj(E_last) h_out, h_in = R_last - sum p.  h at the end of the sequence comes from
// one forward sweep without outputs.
//
// hat theta is what the two products with x and u need:
//     grad_x[i,j,r] = sum_{b,l} hat theta[b,i,j,l] u[b,r,l],   grad_u[b,r,l] += sum_{i,j} x[i,j,r] hat theta[b,i,j,l].
// The second one sums over every channel of a batch element, so hat theta has to leave the wavefront
// that made it: it goes to a workspace that holds it for a CHUNK of the sequence only (tens of MB,
// cache resident), and a matrix-core GEMM kernel consumes it before the next chunk overwrites it.
// A launch therefore covers the tiles t0 .. t1 - 1 of every (batch, channel) pair; the state and its
// adjoint pass from launch to launch through two small buffers.

__device__ __forceinline__ float row_sum(float v) {     // total of the row in its first lane (others: partial)
  return row_suffix(v);
}

#ifndef DROPIN_BWD_WAVES
#define DROPIN_BWD_WAVES 1
#endif
template <int KS, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(DROPIN_BWD_WAVES, DROPIN_BWD_WAVES))) void dropin_bwd_kernel(const DropinBwdArgs q) {
  __shared__ u4 s_u[2][KS * 3 * 64];
  __shared__ float2 s_yw[2][NW][DT];                   // shares of (sum_j Re(Ct h), sum_j hat w) of the tile (nb > 1)
  const DropinArgs& p = q.f;
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int nb = p.nb, ncg = (p.d * nb + NW - 1) / NW;
  const int zb = blockIdx.x / ncg, b = q.b0 + zb, v = (blockIdx.x % ncg) * NW + wave;
  const int i = v / nb, sb = v % nb, j0 = 16 * sb;
  const bool iok = i < p.d;
  const int ic = iok ? i : p.d - 1, vc = ic * nb + sb;
  const int l_ = lane & 15, g = lane >> 4;
  const int d = p.d, n = p.n, L = p.L;
  const size_t row = ((size_t)b * d + ic) * L;
  const u4* __restrict__ upb = p.up + ((size_t)(b - p.up_b0) * p.up_nt - p.up_t0) * (KS * 3 * 64);   // + tile * (KS 3 64)

  u4 xa[KS][3];
#pragma unroll
  for (int k = 0; k < KS; ++k)
#pragma unroll
    for (int c = 0; c < 3; ++c)
      xa[k][c] = (k < p.ks) ? p.xp[(((size_t)vc * p.ks + k) * 3 + c) * 64 + lane] : u4{0, 0, 0, 0};
  // per state: (Re Bt, Im Bt, Re Ct, Im Ct), shared by the workgroup, and the bias of this wavefront's channel.
  // They are read from LDS where they are used: in registers they would push the kernel over 256.
  __shared__ f4 s_par[D_MAXN];
  __shared__ float s_xb[NW][16];
  if (tid < D_MAXN) {
    const bool ok = tid < n;
    const int jc = ok ? tid : 0;
    float sb, cb, sc, cc;
    fast_sincosf(p.B_th[jc], &sb, &cb);
    fast_sincosf(p.C_th[jc], &sc, &cc);
    s_par[tid] = ok ? f4{p.B_r[jc] * cb, p.B_r[jc] * sb, p.C_r[jc] * cc, p.C_r[jc] * sc} : f4{0, 0, 0, 0};
  }
  if (lane < 16) s_xb[wave][lane] = j0 + lane < n ? p.x_bias[(size_t)ic * n + j0 + lane] : 0.0f;
  float hr[4], hi[4], ar[4], ai[4];
  float gBr[4], gBi[4], gCr[4], gCi[4], gxb[4];
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int j = j0 + 4 * g + a;
    const bool ok = j < n;
    const int jc = ok ? j : 0;
    const size_t sidx = ((size_t)b * d + ic) * n + jc;
    hr[a] = ok ? q.hc_re[sidx] : 0.0f;             // state at the end of the tile being processed
    hi[a] = ok ? q.hc_im[sidx] : 0.0f;
    ar[a] = ok ? q.dh_re[sidx] : 0.0f;             // its adjoint
    ai[a] = ok ? q.dh_im[sidx] : 0.0f;
    gBr[a] = gBi[a] = gCr[a] = gCi[a] = gxb[a] = 0.0f;
  }
  const float Di = p.Dp[ic];
  float gD = 0.0f;
  const int t_first = q.t0, t_last = q.t1 - 1;
  float* __restrict__ dth = q.dth + ((size_t)zb * d + ic) * n * q.lc - (size_t)t_first * DT;

  constexpr int NT = NW * 64, NREC = (KS * 3 * 64 + NT - 1) / NT;
  u4 sv[NREC];
  tile_load<NT, NREC, KS>(upb + (size_t)t_last * (KS * 3 * 64), sv, tid);
  tile_store<NT, NREC, KS>(sv, s_u[t_last & 1], tid);
  __syncthreads();
  // the wavefront's own inputs, requested one tile ahead
  float un, dtn, zn, gyn;
  {
    const int l = t_last * DT + l_;
    const bool ok = l < L;
    un = ok ? p.u[row + l] : 0.0f;
    dtn = ok ? p.dt[row + l] : 0.0f;
    zn = ok ? p.z[row + l] : 0.0f;
    gyn = ok ? q.gy[row + l] : 0.0f;
  }
  for (int t = t_last; t >= t_first; --t) {
    const int l0 = t * DT, l = l0 + l_;
    const bool lok = l < L;
    const float uv = un, dtv = dtn, zv = zn, gyv = gyn;
    if (t > t_first) {                 // l - DT < L holds
      un = p.u[row + l - DT];
      dtn = p.dt[row + l - DT];
      zn = p.z[row + l - DT];
      gyn = q.gy[row + l - DT];
    }
    if (t > t_first) tile_load<NT, NREC, KS>(upb + (size_t)(t - 1) * (KS * 3 * 64), sv, tid);
    f4 th = {0, 0, 0, 0};
    const u4* su = s_u[t & 1];
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      u4 ubk[3];
#pragma unroll
      for (int c = 0; c < 3; ++c) ubk[c] = su[(k * 3 + c) * 64 + lane];
      th = xmm<3>(xa[k], ubk, th);
    }
    const float ut = silu_fast(uv), w = dtv * ut, sz = silu_fast(zv), av = gyv * sz;
    const float cnt = (float)(min(l_ + 1, L - l0));      // timesteps of the tile up to this one that exist
    float ysum = 0.0f, wsum = 0.0f;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const f4 par = s_par[j0 + 4 * g + a];
      const float btr_ = par[0], bti_ = par[1], ctr_ = par[2], cti_ = par[3];
      const float G = fmaf(s_xb[wave][4 * g + a], cnt, th[a]);
      float sn, cs;
      sincos_any(G, &sn, &cs);
      const float csl = row_last(cs, lane), snl = row_last(sn, lane);
      // forward quantities of the tile from the state at its end
      const float pr = (cs * btr_ + sn * bti_) * w, pi = (cs * bti_ - sn * btr_) * w;
      const float Ppr = row_prefix(pr), Ppi = row_prefix(pi);
      const float Ptr = row_last(Ppr, lane), Pti = row_last(Ppi, lane);
      const float Rer = csl * hr[a] + snl * hi[a], Rei = csl * hi[a] - snl * hr[a];   // conj(E_last) h_out
      const float hinr = Rer - Ptr, hini = Rei - Pti;
      const float Rr = hinr + Ppr, Ri = hini + Ppi;
      const float her = cs * Rr - sn * Ri, hei = cs * Ri + sn * Rr;                  // h_l
      ysum += ctr_ * her - cti_ * hei;
      // adjoints
      const float hdr = av * ctr_, hdi = -av * cti_;                              // a conj(Ct)
      const float Rhr = cs * hdr + sn * hdi, Rhi = cs * hdi - sn * hdr;               // conj(E_l) (a conj(Ct))
      const float Kr = csl * ar[a] + snl * ai[a], Ki = csl * ai[a] - snl * ar[a];     // conj(E_last) hat h_out
      const float phr = row_suffix(Rhr) + Kr, phi = row_suffix(Rhi) + Ki;             // hat p_s
      // hat w: Re(E conj(Bt) hat p)
      const float ebr = cs * btr_ + sn * bti_, ebi = sn * btr_ - cs * bti_;   // E conj(Bt)
      wsum += ebr * phr - ebi * phi;
      // hat G
      float Gh = -(hdr * hei - hdi * her) + (phr * pi - phi * pr);
      if (l_ == 15) Gh -= ar[a] * hi[a] - ai[a] * hr[a];                              // h at the last step is h_out
      const float thh = row_suffix(Gh);
      if (lok && iok && j0 + 4 * g + a < n) dth[(size_t)(j0 + 4 * g + a) * q.lc + l] = thh;
      gxb[a] += lok ? thh : 0.0f;
      // hat Bt += E w hat p ; hat Ct += a conj(h)
      const float ewr = cs * w, ewi = sn * w;
      gBr[a] += ewr * phr - ewi * phi;
      gBi[a] += ewr * phi + ewi * phr;
      gCr[a] += av * her;
      gCi[a] -= av * hei;
      // hand over to the previous tile
      hr[a] = hinr;
      hi[a] = hini;
      ar[a] = row_first(phr, lane);
      ai[a] = row_first(phi, lane);
    }
    ysum = rows_sum(ysum);
    wsum = rows_sum(wsum);
    if (nb > 1 && g == 0) s_yw[t & 1][wave][l_] = make_float2(ysum, wsum);
    if (t > t_first) tile_store<NT, NREC, KS>(sv, s_u[(t - 1) & 1], tid);
    if (nb > 1) {                                      // the channel's first wavefront adds the shares up
      __syncthreads();
      for (int k = 1; k < nb; ++k) {
        const float2 o = s_yw[t & 1][(wave + k) & (NW - 1)][l_];
        ysum += o.x;
        wsum += o.y;
      }
    }
    if (iok && lok && g == 0 && sb == 0) {
      const float pre = ysum + Di * ut;
      q.dz[row + l] = gyv * pre * dsilu_fast(zv);
      q.ddt[row + l] = wsum * ut;
      q.du[row + l] = (wsum * dtv + av * Di) * dsilu_fast(uv);
      gD += av * ut;
    }
    if (nb == 1) __syncthreads();
  }
  // ---- reductions over the timesteps (lanes of a row) and hand-off.  The gradients of the 4 n shared
  // parameters are first summed over the workgroup's channels in LDS: every workgroup of the launch adds
  // to the same few addresses.
  __shared__ float s_red[4][D_MAXN];
  if (tid < 4 * D_MAXN) (&s_red[0][0])[tid] = 0.0f;
  __syncthreads();
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    gxb[a] = row_sum(gxb[a]);
    gBr[a] = row_sum(gBr[a]);
    gBi[a] = row_sum(gBi[a]);
    gCr[a] = row_sum(gCr[a]);
    gCi[a] = row_sum(gCi[a]);
  }
  gD = row_sum(gD);
  if (iok && l_ == 0) {
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int j = j0 + 4 * g + a;
      if (j < n) {
        const size_t sidx = ((size_t)b * d + i) * n + j;
        q.dh_re[sidx] = ar[a];
        q.dh_im[sidx] = ai[a];
        q.hc_re[sidx] = hr[a];
        q.hc_im[sidx] = hi[a];
        atomicAdd(q.dxb + (size_t)i * n + j, gxb[a]);
        // polar parameters: Bt = B_r e^{i B_theta}
        float ebr, ebi, ecr, eci;
        fast_sincosf(p.B_th[j], &ebi, &ebr);
        fast_sincosf(p.C_th[j], &eci, &ecr);
        const f4 par = s_par[j];
        atomicAdd(&s_red[0][j], gBr[a] * ebr + gBi[a] * ebi);
        atomicAdd(&s_red[1][j], gBi[a] * par[0] - gBr[a] * par[1]);
        atomicAdd(&s_red[2][j], gCr[a] * ecr + gCi[a] * eci);
        atomicAdd(&s_red[3][j], gCi[a] * par[2] - gCr[a] * par[3]);
      }
    }
    if (g == 0 && sb == 0) atomicAdd(q.dD + i, gD);
  }
  __syncthreads();
  if (tid < 4 * D_MAXN && (tid & (D_MAXN - 1)) < n) {
    constexpr int SH = 6;                              // log2(D_MAXN)
    float* dst = (tid >> SH) == 0 ? q.dB_r : (tid >> SH) == 1 ? q.dB_th : (tid >> SH) == 2 ? q.dC_r : q.dC_th;
    atomicAdd(dst + (tid & (D_MAXN - 1)), (&s_red[0][0])[tid]);
  }
}

// Several small buffers set in one launch (blockIdx.y picks the buffer): dst[i] = src ? src[i] : 0.
__global__ __launch_bounds__(256) void fill_kernel(const FillArgs a) {
  float* __restrict__ dst = a.dst[blockIdx.y];
  const float* __restrict__ src = a.src[blockIdx.y];
  const size_t n = a.n[blockIdx.y];
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = src ? src[i] : 0.0f;
}

// ---- fp32-accurate GEMM on the bf16 matrix cores ------------------------------------------------
//     C_z[m][n] (+)= sum_k A_z(m, k) B_z(k, n)           z = 0 .. Z-1
//     C[m][n]    += sum_z sum_k A_z(m, k) B_z(k, n)      (reduce_z)
// Workgroup tile 128 x (64 TNH), four wavefronts of 64 x (32 TNH) each, 32 of k per step, one workgroup per (tile,
// slice of z, slice of k): zper consecutive z per workgroup (1 unless reduce_z) and ksplit slices of k.  With more
// than one slice per element of C the results are summed into C with atomics (C holds the addend beforehand).
// A - the operand with the 128-row side of the tile - arrives split into three bf16 pieces in the order the
// kernel keeps it in LDS (a pre-pass, gemm_aprep_kernel: the callers' A is small and used by every workgroup of
// a column of tiles), so a step copies 24 KiB of records; B is fp32 with arbitrary strides and is split while
// it is staged.  The values of the next step are requested before the products of the current one.
// (Measured on the backward call of the fused operator, b = 32, d = 256, n = 16, L = 720.  Launches of 6.2 GFLOP in
// fp32 terms with 128 x 64 tiles: 54-58 us; without the stores of C - atomics, the launch is cut along k or z -
// 40-46 us; without the matrix instructions 41-43 us; with neither 30 us: operand traffic, LDS and the two barriers
// of a step set the floor, the rest adds up.  Launches twice that size: 99-102 us with 128 x 64 tiles, 84-97 us
// with 128 x 128 (TNH = 2).  Splitting A inside the loop, as B is, cost 5 % more.)
// K1: B is contiguous along k.  Then four neighbouring lanes fetch the 32 values of one row as 16-byte
// vectors (VEC; rows need not be 16-byte aligned) - a wavefront request covers 16 cache lines.  Otherwise it is
// contiguous along n and a 16-lane row of the wavefront fetches 16 neighbouring rows' values of one k.
// Rows of the B tile that lie past N are fetched from the last valid row instead (column n of B only reaches
// column n of C, which is not stored then), so only the last, partial step along k takes the bounds-checked loads.
// TR: the two operands change places in the matrix instruction, so that the lanes of a result register run
// along m: for a C that is contiguous along m (the stores and atomics of a wavefront then cover whole lines).

// Record slot of (row r of a 16-row tile, k group g = 8 values): 16 g + (r + 4 g) % 16.  The rotation keeps the
// 16-byte writes of the K1 mapping (four neighbouring lanes = the four g of one row) and the reads (16
// neighbouring lanes = 16 rows of one g) both free of bank conflicts.
__device__ __forceinline__ int gemm_slot(int r, int g) { return 16 * g + ((r + 4 * g) & 15); }

// A (fp32, strides sam / sak / saz) -> image: one thread per (z, 16-row tile, step, record)
__global__ __launch_bounds__(256) void gemm_aprep_kernel(const float* __restrict__ A, u4* __restrict__ img, long sam, long sak, long saz,
                                                         int M, int K, int m16, int nk, long total) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int slot = (int)(idx & 63);
  const long rest = idx >> 6;
  const int it = (int)(rest % nk), mt = (int)((rest / nk) % m16);
  const long z = rest / ((long)nk * m16);
  const int g = slot >> 4, r = ((slot & 15) - 4 * g) & 15;
  const int m = mt * 16 + r, k0 = it * 32 + 8 * g;
  const SplitK sk = make_splitk();
  float v[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) v[q] = (m < M && k0 + q < K) ? A[z * saz + (long)m * sam + (long)(k0 + q) * sak] : 0.0f;
  u4 pc[3];
  split8<3>(sk, v, pc);
#pragma unroll
  for (int c = 0; c < 3; ++c) img[(rest * 3 + c) * 64 + slot] = pc[c];
}

template <bool K1, bool VEC, bool TR, int TNH>
__global__ __launch_bounds__(256) void split_gemm_kernel(const GemmArgs p) {
  constexpr int NP = 3;                // bf16 pieces per operand: fp32-accurate products
  constexpr int AREC = 8 * NP * 64;    // records of the A tile of one step
  constexpr int AQ = AREC / 256;       // ... per thread
  constexpr int TN = 64 * TNH;         // columns of the workgroup tile
  constexpr int EN = 2 * TNH;          // 16-wide column tiles per wavefront
  __shared__ u4 s_a[AREC], s_b[4 * TNH * NP * 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int m0 = blockIdx.x * 128, n0 = blockIdx.y * TN;
  const int zs = blockIdx.z / p.ksplit, ksl = blockIdx.z % p.ksplit;
  const int z_lo = zs * p.zper, z_hi = z_lo + p.zper < p.Z ? z_lo + p.zper : p.Z;
  const int wm = (wave >> 1) * 4, wn = (wave & 1) * EN;      // this wavefront's first 16-wide tiles
  const SplitK sk = make_splitk();
  f4 acc[4][EN];
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int f = 0; f < EN; ++f) acc[e][f] = f4{0, 0, 0, 0};
  // the record of B this thread stages: row rb of the tile, k slots kq ..
  const int rb = K1 ? tid >> 2 : wave * 16 + (lane & 15);
  const int kq = 8 * (K1 ? tid & 3 : lane >> 4);
  const int slot = (rb >> 4) * (NP * 64) + gemm_slot(rb & 15, kq >> 3);
  const int rslot = gemm_slot(lane & 15, lane >> 4);       // the record of (row lane % 16, g lane / 16)
  // uniform bases, 32-bit per-thread offsets (a z-slice of B is below 2^31 elements)
  const unsigned sbk = (unsigned)p.sbk;
  unsigned ob[TNH];
#pragma unroll
  for (int h = 0; h < TNH; ++h) {
    const int n = n0 + rb + 64 * h;
    ob[h] = (unsigned)(n < p.N ? n : p.N - 1) * (unsigned)p.sbn + (unsigned)kq * sbk;
  }
  const int nk = (p.K + 31) / 32, per = (nk + p.ksplit - 1) / p.ksplit;
  const int it0 = ksl * per, it1 = it0 + per < nk ? it0 + per : nk;
  const int nit = it1 > it0 ? (it1 - it0) * (z_hi - z_lo) : 0;      // steps of this workgroup: (z, k step) pairs
  // this thread's records of the A tile: record tid + 256 q of the tile = record (tid + 256 q) % 192 of row tile
  // m0 / 16 + (tid + 256 q) / 192, whose steps lie nk * 192 records apart
  unsigned oa[AQ];
#pragma unroll
  for (int q = 0; q < AQ; ++q) {
    const int idx = tid + 256 * q, e = idx / (NP * 64);
    oa[q] = (unsigned)(((m0 >> 4) + e) * nk) * (unsigned)(NP * 64) + (unsigned)(idx - e * (NP * 64));
  }
  u4 ia[AQ];
  float vb[TNH][8];
  int fz = z_lo, fit = it0;                   // (z, k step) of the next fetch: steps are fetched in order
  auto fetch = [&]() {
    const int z = fz, it = fit;
    if (++fit == it1) { fit = it0; ++fz; }
    const u4* __restrict__ Az = p.Aimg + z * p.simz + (size_t)it * (NP * 64);
#pragma unroll
    for (int q = 0; q < AQ; ++q) ia[q] = Az[oa[q]];
    const float* __restrict__ Bz = p.Bm + z * p.sbz;
    const unsigned kb = (unsigned)(it * 32) * sbk;
    if (it * 32 + 32 <= p.K) {
      if constexpr (K1 && VEC) {
        // 16-byte loads that are only known to be 4-byte aligned (rows start anywhere when the row length is
        // not a multiple of four): the memory pipeline takes them, the type tells the compiler so
        typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
          for (int h = 0; h < TNH; ++h) {
            const f4u x = *reinterpret_cast<const f4u*>(Bz + (ob[h] + kb + 4 * q));
#pragma unroll
            for (int c = 0; c < 4; ++c) vb[h][4 * q + c] = x[c];
          }
      } else {
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
          for (int h = 0; h < TNH; ++h) vb[h][c] = Bz[ob[h] + kb + (unsigned)c * sbk];
      }
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c)
#pragma unroll
        for (int h = 0; h < TNH; ++h) vb[h][c] = (it * 32 + kq + c < p.K) ? Bz[ob[h] + kb + (unsigned)c * sbk] : 0.0f;
    }
  };
  if (nit > 0) fetch();
  for (int step = 0; step < nit; ++step) {
    u4 pb[TNH][NP];
#pragma unroll
    for (int h = 0; h < TNH; ++h) split8<NP>(sk, vb[h], pb[h]);
    __syncthreads();
#pragma unroll
    for (int q = 0; q < AQ; ++q) s_a[tid + 256 * q] = ia[q];
#pragma unroll
    for (int c = 0; c < NP; ++c)
#pragma unroll
      for (int h = 0; h < TNH; ++h) s_b[slot + 4 * h * (NP * 64) + c * 64] = pb[h][c];
    __syncthreads();
    if (step + 1 < nit) fetch();              // in flight during the products
    u4 rB[EN][NP];
#pragma unroll
    for (int f = 0; f < EN; ++f)
#pragma unroll
      for (int c = 0; c < NP; ++c) rB[f][c] = s_b[((wn + f) * NP + c) * 64 + rslot];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      u4 rA[NP];
#pragma unroll
      for (int c = 0; c < NP; ++c) rA[c] = s_a[((wm + e) * NP + c) * 64 + rslot];
#pragma unroll
      for (int f = 0; f < EN; ++f) acc[e][f] = TR ? xmm<NP>(rB[f], rA, acc[e][f]) : xmm<NP>(rA, rB[f], acc[e][f]);
    }
  }
  // result tile (e, f), register a: row 16 e + 4 (lane / 16) + a, column 16 f + lane % 16 of the wavefront's block
  // (TR: row 16 e + lane % 16, column 16 f + 4 (lane / 16) + a)
  float* __restrict__ C = p.C + (p.reduce_z ? 0 : z_lo * p.scz);
  const bool atomic = p.ksplit > 1 || (p.reduce_z && p.zper < p.Z);
  // element offsets inside a z-slice of C fit 32 bits (checked by the caller)
  const unsigned scm = (unsigned)p.scm, scn = (unsigned)p.scn;
  const int mr = m0 + wm * 16 + (TR ? (lane & 15) : 4 * (lane >> 4)), nc = n0 + wn * 16 + (TR ? 4 * (lane >> 4) : (lane & 15));
  const unsigned o0 = (unsigned)mr * scm + (unsigned)nc * scn;
  const unsigned sa = TR ? scn : scm;           // stride between the four registers of a result
  if (atomic && m0 + 128 <= p.M && n0 + TN <= p.N) {       // uniform: a whole tile, summed into C
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int f = 0; f < EN; ++f)
#pragma unroll
        for (int a = 0; a < 4; ++a) atomicAdd(C + (o0 + (unsigned)(16 * e) * scm + (unsigned)(16 * f) * scn + (unsigned)a * sa), acc[e][f][a]);
    return;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int f = 0; f < EN; ++f)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        if (mr + 16 * e + (TR ? 0 : a) < p.M && nc + 16 * f + (TR ? a : 0) < p.N) {
          float* c = C + (o0 + (unsigned)(16 * e) * scm + (unsigned)(16 * f) * scn + (unsigned)a * sa);
          if (atomic) atomicAdd(c, acc[e][f][a]);
          else *c = p.accumulate ? *c + acc[e][f][a] : acc[e][f][a];
        }
      }
}

}  // namespace aussm
