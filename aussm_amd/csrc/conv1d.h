// Depthwise causal 1-D convolution along the sequence, channels-last: the step the blocks apply
// to the scan's input,
//     y[b,l,d] = bias[d] + sum_{k<K} w[d,k] x[b, l - (K-1) + k, d]        (x = 0 before the sequence)
// = nn.Conv1d(D, D, K, groups=D, padding=K-1)(x^T)[:, :, :L]^T of
// ai-modules/wavesAI/model/aussm.py:762 and :863, computed where the data lies: the blocks hold
// x as (b, l, d) (a column slice of the in_proj output), so neighbouring lanes read neighbouring
// channels and no transposed copy is made.  K <= CONV_MAX_K.
#pragma once
#include <hip/hip_runtime.h>

#include "scan_args.h"

namespace aussm {



// grid: x = (b, l) row, y = block of 256 channels
__global__ __launch_bounds__(256) void causal_conv1d_fwd_kernel(const ConvArgs p) {
  const int d = blockIdx.y * 256 + threadIdx.x;
  if (d >= p.D) return;
  const unsigned r = blockIdx.x;
  const int b = (int)(r / (unsigned)p.L), l = (int)(r % (unsigned)p.L);
  const float* __restrict__ xr = p.x + (size_t)b * p.xs_b + d;
  float acc = p.bias ? p.bias[d] : 0.0f;
  for (int k = 0; k < p.K; ++k) {
    const int ls = l - (p.K - 1) + k;
    if (ls >= 0) acc = fmaf(p.w[(size_t)d * p.K + k], xr[(size_t)ls * p.xs_l], acc);
  }
  p.y[(size_t)r * p.D + d] = acc;
}

// dx[b,l,d] = sum_k w[d,k] dy[b, l + (K-1) - k, d]   (terms past the end of the sequence drop out)
__global__ __launch_bounds__(256) void causal_conv1d_bwd_data_kernel(const ConvArgs p) {
  const int d = blockIdx.y * 256 + threadIdx.x;
  if (d >= p.D) return;
  const unsigned r = blockIdx.x;
  const int l = (int)(r % (unsigned)p.L);
  const float* __restrict__ gr = p.dy + (size_t)r * p.D + d;      // row (b, l); later rows of b follow
  float acc = 0.0f;
  for (int k = 0; k < p.K; ++k) {
    const int lt = l + (p.K - 1) - k;
    if (lt < p.L) acc = fmaf(p.w[(size_t)d * p.K + k], gr[(size_t)(lt - l) * p.D], acc);
  }
  p.dx[(size_t)r * p.D + d] = acc;
}

// dw[d,k] += sum_{b,l} dy[b,l,d] x[b, l - (K-1) + k, d],  dbias[d] += sum_{b,l} dy[b,l,d].
// Workgroup = 64 channels x CONV_ROWS rows of (b, l); thread (channel tid % 64, row group tid / 64).
__global__ __launch_bounds__(256) void causal_conv1d_bwd_weight_kernel(const ConvArgs p) {
  __shared__ float s_red[4][CONV_MAX_K + 1][64];
  const int dl = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int d = blockIdx.x * 64 + dl;
  const bool dok = d < p.D;
  const size_t rows = (size_t)p.B * p.L;
  const size_t r0 = (size_t)blockIdx.y * CONV_ROWS;
  float acc[CONV_MAX_K + 1];
#pragma unroll
  for (int k = 0; k <= CONV_MAX_K; ++k) acc[k] = 0.0f;
  if (dok) {
    int b = (int)((unsigned)(r0 + rg) / (unsigned)p.L), l = (int)((unsigned)(r0 + rg) % (unsigned)p.L);
    for (int i = rg; i < CONV_ROWS; i += 4, l += 4) {
      const size_t r = r0 + i;
      if (r >= rows) break;
      while (l >= p.L) { l -= p.L; ++b; }
      const float g = p.dy[r * p.D + d];
      const float* __restrict__ xr = p.x + (size_t)b * p.xs_b + d;
#pragma unroll
      for (int k = 0; k < CONV_MAX_K; ++k) {
        const int ls = l - (p.K - 1) + k;
        if (k < p.K && ls >= 0) acc[k] = fmaf(g, xr[(size_t)ls * p.xs_l], acc[k]);
      }
      acc[CONV_MAX_K] += g;
    }
  }
#pragma unroll
  for (int k = 0; k <= CONV_MAX_K; ++k) s_red[rg][k][dl] = acc[k];
  __syncthreads();
  if (rg == 0 && dok) {
#pragma unroll
    for (int k = 0; k <= CONV_MAX_K; ++k) {
      const float v = s_red[0][k][dl] + s_red[1][k][dl] + s_red[2][k][dl] + s_red[3][k][dl];
      if (k < p.K) atomicAdd(p.dw + (size_t)d * p.K + k, v);
      else if (k == CONV_MAX_K && p.dbias) atomicAdd(p.dbias + d, v);
    }
  }
}

// ---- kernel length 4 (the blocks' default d_conv): each thread owns CONV_RUN consecutive steps of
// one channel and slides a register window over them, one load per step instead of four.

// grid: x = (b, run of CONV_RUN steps), y = block of 256 channels
__global__ __launch_bounds__(256) void causal_conv1d_k4_fwd_kernel(const ConvArgs p) {
  const int d = blockIdx.y * 256 + threadIdx.x;
  if (d >= p.D) return;
  const unsigned nrun = (unsigned)(p.L + CONV_RUN - 1) / CONV_RUN;
  const int b = (int)(blockIdx.x / nrun), l0 = (int)(blockIdx.x % nrun) * CONV_RUN;
  const float* __restrict__ xr = p.x + (size_t)b * p.xs_b + d;
  const float w0 = p.w[(size_t)d * 4], w1 = p.w[(size_t)d * 4 + 1], w2 = p.w[(size_t)d * 4 + 2], w3 = p.w[(size_t)d * 4 + 3];
  const float bias = p.bias ? p.bias[d] : 0.0f;
  float a = l0 >= 3 ? xr[(size_t)(l0 - 3) * p.xs_l] : 0.0f;
  float bq = l0 >= 2 ? xr[(size_t)(l0 - 2) * p.xs_l] : 0.0f;
  float c = l0 >= 1 ? xr[(size_t)(l0 - 1) * p.xs_l] : 0.0f;
  float* __restrict__ yr = p.y + ((size_t)b * p.L + l0) * p.D + d;
#pragma unroll
  for (int i = 0; i < CONV_RUN; ++i) {
    if (l0 + i < p.L) {
      const float e = xr[(size_t)(l0 + i) * p.xs_l];
      yr[(size_t)i * p.D] = fmaf(w0, a, fmaf(w1, bq, fmaf(w2, c, fmaf(w3, e, bias))));
      a = bq; bq = c; c = e;
    }
  }
}

// dx[l] = w3 dy[l] + w2 dy[l+1] + w1 dy[l+2] + w0 dy[l+3]
__global__ __launch_bounds__(256) void causal_conv1d_k4_bwd_data_kernel(const ConvArgs p) {
  const int d = blockIdx.y * 256 + threadIdx.x;
  if (d >= p.D) return;
  const unsigned nrun = (unsigned)(p.L + CONV_RUN - 1) / CONV_RUN;
  const int b = (int)(blockIdx.x / nrun), l0 = (int)(blockIdx.x % nrun) * CONV_RUN;
  const float* __restrict__ gr = p.dy + (size_t)b * p.L * p.D + d;
  const float w0 = p.w[(size_t)d * 4], w1 = p.w[(size_t)d * 4 + 1], w2 = p.w[(size_t)d * 4 + 2], w3 = p.w[(size_t)d * 4 + 3];
  float g[CONV_RUN + 3];
#pragma unroll
  for (int i = 0; i < CONV_RUN + 3; ++i) g[i] = (l0 + i < p.L) ? gr[(size_t)(l0 + i) * p.D] : 0.0f;
  float* __restrict__ dr = p.dx + ((size_t)b * p.L + l0) * p.D + d;
#pragma unroll
  for (int i = 0; i < CONV_RUN; ++i)
    if (l0 + i < p.L) dr[(size_t)i * p.D] = fmaf(w3, g[i], fmaf(w2, g[i + 1], fmaf(w1, g[i + 2], w0 * g[i + 3])));
}

// Weight and bias gradients: thread (channel tid % 64, quarter tid / 64) walks CONV_ROWS / 4 consecutive
// (b, l) rows with a window of the three previous inputs (cleared where a new batch element starts).
__global__ __launch_bounds__(256) void causal_conv1d_k4_bwd_weight_kernel(const ConvArgs p) {
  __shared__ float s_red[4][5][64];
  const int dl = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int d = blockIdx.x * 64 + dl;
  const bool dok = d < p.D;
  const size_t rows = (size_t)p.B * p.L;
  constexpr int RUN = CONV_ROWS / 4;
  const size_t r0 = (size_t)blockIdx.y * CONV_ROWS + (size_t)rg * RUN;
  float acc0 = 0.0f, acc1 = 0.0f, acc2 = 0.0f, acc3 = 0.0f, accb = 0.0f;
  if (dok && r0 < rows) {
    int b = (int)((unsigned)r0 / (unsigned)p.L), l = (int)((unsigned)r0 % (unsigned)p.L);
    const float* __restrict__ xr = p.x + (size_t)b * p.xs_b + d;
    float a = l >= 3 ? xr[(size_t)(l - 3) * p.xs_l] : 0.0f;
    float bq = l >= 2 ? xr[(size_t)(l - 2) * p.xs_l] : 0.0f;
    float c = l >= 1 ? xr[(size_t)(l - 1) * p.xs_l] : 0.0f;
    for (int i = 0; i < RUN; ++i) {
      const size_t r = r0 + i;
      if (r >= rows) break;
      if (l == p.L) { l = 0; ++b; xr = p.x + (size_t)b * p.xs_b + d; a = bq = c = 0.0f; }
      const float e = xr[(size_t)l * p.xs_l];
      const float g = p.dy[r * p.D + d];
      acc0 = fmaf(g, a, acc0); acc1 = fmaf(g, bq, acc1); acc2 = fmaf(g, c, acc2); acc3 = fmaf(g, e, acc3);
      accb += g;
      a = bq; bq = c; c = e;
      ++l;
    }
  }
  s_red[rg][0][dl] = acc0; s_red[rg][1][dl] = acc1; s_red[rg][2][dl] = acc2; s_red[rg][3][dl] = acc3; s_red[rg][4][dl] = accb;
  __syncthreads();
  if (rg == 0 && dok) {
#pragma unroll
    for (int k = 0; k < 5; ++k) {
      const float v = s_red[0][k][dl] + s_red[1][k][dl] + s_red[2][k][dl] + s_red[3][k][dl];
      if (k < 4) atomicAdd(p.dw + (size_t)d * 4 + k, v);
      else if (p.dbias) atomicAdd(p.dbias + d, v);
    }
  }
}

}  // namespace aussm
