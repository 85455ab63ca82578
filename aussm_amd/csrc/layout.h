// Swap of the last two dimensions of a batched matrix, y[b, c, r] = x[b, r, c]: the conversion
// between the blocks' channels-last activations (b, l, d) and the scans' (b, d, l) tensors
// (`rearrange(x, 'b l d -> b d l')` and back, ai-modules/wavesAI/model/aussm.py:760-803 and
// :861-900).  32 x 32 tiles through LDS, so both the reads and the writes are full lines; the
// input may be a column slice of a wider tensor (row stride xs_r >= C), the output is contiguous.
// Optionally the elementwise step the blocks apply on the way is done in the same pass: silu on the
// convolution output that feeds the S6 scan (aussm.py:787), softplus(dt + bias) in front of the
// adaptive-unitary operator (aussm.py:878-880), and their derivatives on the way back.
#pragma once
#include <hip/hip_runtime.h>

#include "scan_args.h"
#include "scan_common.h"

namespace aussm {

__device__ __forceinline__ float swap_act(int act, float v) { return act == 1 ? siluf_(v) : softplusf_(v); }
__device__ __forceinline__ float swap_dact(int act, float v) {
  return act == 1 ? dsiluf_(v) : (v > 20.0f ? 1.0f : sigmoidf_(v));
}

__global__ __launch_bounds__(256) void swap_last2_kernel(const SwapArgs p) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;      // 32 x 8 threads
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32, b = blockIdx.z;
  const float* __restrict__ xb = p.x + (size_t)b * p.xs_b;
  float* __restrict__ yb = p.y + (size_t)b * p.C * p.R;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = r0 + ty + 8 * j, c = c0 + tx;
    if (r < p.R && c < p.C) {
      float v = xb[(size_t)r * p.xs_r + c];
      if (p.act && !p.deriv) v = swap_act(p.act, v + (p.bias ? p.bias[c] : 0.0f));
      tile[ty + 8 * j][tx] = v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = c0 + ty + 8 * j, r = r0 + tx;
    if (c < p.C && r < p.R) {
      float v = tile[tx][ty + 8 * j];
      if (p.act && p.deriv)
        v *= swap_dact(p.act, p.pre[(size_t)b * p.ps_b + (size_t)c * p.ps_r + r] + (p.bias ? p.bias[r] : 0.0f));
      yb[(size_t)c * p.R + r] = v;
    }
  }
}

// The scans' output gate  y = y_pre silu(z)  (extension-cpp/extension_cpp/ops.py:226) and its two gradients
//     dy_pre = dy silu(z),   dz = dy y_pre silu'(z)
// as one pass each over contiguous tensors of n floats (vec: all of them 16-byte aligned), for the scan
// whose backward kernel takes the gradient of the ungated output.
__global__ __launch_bounds__(256) void gate_fwd_kernel(const float* __restrict__ ypre, const float* __restrict__ z,
                                                       float* __restrict__ y, size_t n, int vec) {
  const size_t stride = (size_t)gridDim.x * 256 * 4;
  for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4; i < n; i += stride) {
    if (vec && i + 4 <= n) {
      const float4 a = *reinterpret_cast<const float4*>(ypre + i), g = *reinterpret_cast<const float4*>(z + i);
      *reinterpret_cast<float4*>(y + i) = make_float4(a.x * siluf_(g.x), a.y * siluf_(g.y), a.z * siluf_(g.z), a.w * siluf_(g.w));
    } else {
      for (size_t j = i; j < n && j < i + 4; ++j) y[j] = ypre[j] * siluf_(z[j]);
    }
  }
}
__global__ __launch_bounds__(256) void gate_bwd_kernel(const float* __restrict__ dy, const float* __restrict__ ypre,
                                                       const float* __restrict__ z, float* __restrict__ dypre,
                                                       float* __restrict__ dz, size_t n, int vec) {
  const size_t stride = (size_t)gridDim.x * 256 * 4;
  for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4; i < n; i += stride) {
    if (vec && i + 4 <= n) {
      const float4 g = *reinterpret_cast<const float4*>(dy + i), a = *reinterpret_cast<const float4*>(ypre + i),
                   v = *reinterpret_cast<const float4*>(z + i);
      *reinterpret_cast<float4*>(dypre + i) = make_float4(g.x * siluf_(v.x), g.y * siluf_(v.y), g.z * siluf_(v.z), g.w * siluf_(v.w));
      *reinterpret_cast<float4*>(dz + i) = make_float4(g.x * a.x * dsiluf_(v.x), g.y * a.y * dsiluf_(v.y),
                                                       g.z * a.z * dsiluf_(v.z), g.w * a.w * dsiluf_(v.w));
    } else {
      for (size_t j = i; j < n && j < i + 4; ++j) {
        dypre[j] = dy[j] * siluf_(z[j]);
        dz[j] = dy[j] * ypre[j] * dsiluf_(z[j]);
      }
    }
  }
}

}  // namespace aussm
