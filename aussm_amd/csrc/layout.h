// Swap of the last two dimensions of a batched matrix, y[b, c, r] = x[b, r, c]: the conversion
// between the blocks' channels-last activations (b, l, d) and the scans' (b, d, l) tensors
// (`rearrange(x, 'b l d -> b d l')` and back, ai-modules/wavesAI/model/aussm.py:760-803 and
// :861-900).  32 x 32 tiles through LDS, so both the reads and the writes are full lines; the
// input may be a column slice of a wider tensor (row stride xs_r >= C), the output is contiguous.
#pragma once
#include <hip/hip_runtime.h>

#include "scan_args.h"

namespace aussm {


__global__ __launch_bounds__(256) void swap_last2_kernel(const SwapArgs p) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;      // 32 x 8 threads
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32, b = blockIdx.z;
  const float* __restrict__ xb = p.x + (size_t)b * p.xs_b;
  float* __restrict__ yb = p.y + (size_t)b * p.C * p.R;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = r0 + ty + 8 * j, c = c0 + tx;
    if (r < p.R && c < p.C) tile[ty + 8 * j][tx] = xb[(size_t)r * p.xs_r + c];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = c0 + ty + 8 * j, r = r0 + tx;
    if (c < p.C && r < p.R) yb[(size_t)c * p.R + r] = tile[tx][ty + 8 * j];
  }
}

}  // namespace aussm
