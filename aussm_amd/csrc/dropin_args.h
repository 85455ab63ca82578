// Argument blocks of the fused operator kernels (dropin.h), shared with the host side.
#pragma once
#include "scan_args.h"

namespace aussm {

constexpr int DT = 16;            // timesteps per tile
constexpr int D_MAXKS = 16;       // 32-wide steps of the contraction over r held in registers: d <= 512
constexpr int D_MAXN = 64;        // states per channel: up to four blocks of 16, one block per wavefront

struct DropinArgs {
  const float* u;        // [b, d, L]
  const float* dt;       // [b, d, L]
  const float* z;        // [b, d, L]
  const float* x_bias;   // [d, n]
  const float* B_r;      // [n]
  const float* B_th;
  const float* C_r;
  const float* C_th;
  const float* Dp;       // [d]
  const float* h_re;     // [b, d, n] state before tile t0
  const float* h_im;
  float* y;              // [b, d, L] or null (states only)
  float* nh_re;          // [b, d, n] or null: state after tile t1 - 1 (may be the same buffer as h_*)
  float* nh_im;
  const u4* xp;          // rows of x as matrix operands: [d nb][ks][piece][64 lanes]
  const u4* up;          // tiles of u, prefix-summed along the tile, as matrix operands: [b][tile - up_t0][KS][piece][64 lanes]
  int up_b0, up_t0, up_nt;   // up holds the batch elements from up_b0 on and the tiles up_t0 .. up_t0 + up_nt - 1
  int b, d, n, L, ks;    // b: batch elements of this launch; ks = ceil(d / 32)
  int nb;                // blocks of 16 states per channel: 1, 2 or 4 (>= ceil(n / 16))
  int b0;                // first batch element of this launch (tensors are indexed by b0 + ...)
  int t0, t1;            // tiles of 16 timesteps of this launch (forward kernel; the backward kernel has its own)
};

struct DropinBwdArgs {
  DropinArgs f;            // inputs (y, nh_* unused)
  const float* gy;         // [b, d, L]
  float* hc_re;            // [b, d, n] in: state after tile t1 - 1; out: state before tile t0
  float* hc_im;
  float* dth;              // workspace [bg][d n][lc]: phase adjoints of the launch
  float* du;               // [b, d, L] direct part (the product with x is added afterwards)
  float* ddt;
  float* dz;
  float* dxb;              // [d, n]   accumulated with atomics (zeroed by the host)
  float* dB_r;             // [n] each, accumulated with atomics
  float* dB_th;
  float* dC_r;
  float* dC_th;
  float* dD;               // [d]      (atomics)
  float* dh_re;            // [b, d, n] in: adjoint of the state after tile t1 - 1; out: of the state before tile t0
  float* dh_im;
  int b0, bg;              // batch elements b0 .. b0 + bg - 1 ...
  int t0, t1;              // ... and tiles of 16 timesteps t0 .. t1 - 1 (in reverse) are this launch's
  int lc;                  // row length of dth (>= 16 (t1 - t0))
};

// Up to 12 buffers set in one launch: dst[i] = src ? src[i] : 0 for i < n.
struct FillArgs {
  float* dst[12];
  const float* src[12];
  unsigned long long n[12];
  int count;
};

// A is a prepared image (gemm_aprep_kernel): [z][16-row tile][step of 32 along k][piece][64 records], the
// row tiles padded to whole workgroup tiles of 128 rows, zeros past M and K.
struct GemmArgs {
  const u4* Aimg; const float* Bm; float* C;
  long simz;              // records between the images of consecutive z (0: one image for all)
  long sbk, sbn, sbz;     // element strides of B over k, n, z
  long scm, scn, scz;
  int M, N, K, Z;
  int reduce_z, accumulate;
  int tr;                 // results leave with the lanes along m (for C contiguous along m) instead of along n
  int ksplit;             // slices of k per (tile, slice of z)
  int zper;               // z per workgroup (summed inside it; 1 unless reduce_z)
};

}  // namespace aussm
