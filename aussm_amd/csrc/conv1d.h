// Depthwise causal 1-D convolution along the sequence, channels-last: the step the blocks apply
// to the scan's input,
//     y[b,l,d] = bias[d] + sum_{k<K} w[d,k] x[b, l - (K-1) + k, d]        (x = 0 before the sequence)
// = nn.Conv1d(D, D, K, groups=D, padding=K-1)(x^T)[:, :, :L]^T of
// ai-modules/wavesAI/model/aussm.py:762 and :863, computed where the data lies: the blocks hold
// x as (b, l, d) (a column slice of the in_proj output), so neighbouring lanes read neighbouring
// channels and no transposed copy is made.  K <= CONV_MAX_K.
#pragma once
#include <hip/hip_runtime.h>

namespace aussm {

constexpr int CONV_MAX_K = 8;
constexpr int CONV_ROWS = 128;   // (b, l) rows per workgroup of the weight-gradient kernel

struct ConvArgs {
  const float* x;      // element (b, l, d) at x[b * xs_b + l * xs_l + d]
  const float* w;      // [D, K]
  const float* bias;   // [D] or null
  const float* dy;     // [B, L, D] contiguous (backward)
  float* y;            // [B, L, D] contiguous (forward)
  float* dx;           // [B, L, D] contiguous (backward)
  float* dw;           // [D, K], accumulated into
  float* dbias;        // [D] or null, accumulated into
  long long xs_b, xs_l;
  int B, L, D, K;
};

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

}  // namespace aussm
