// Translation unit of the matrix-core unitary kernels that build their operands in place
// (scan_fwd_xdl.h, scan_bwd_xdl.h) and of the split along L (scan_seg_xdl.h).
#include "launch.h"
#include "scan_bwd_xdl.h"
#include "scan_fwd_xdl.h"
#include "scan_seg_xdl.h"

namespace aussm {

int run_xdl_fwd(int mode, const FwdArgs& a, int in_dtype, hipStream_t s) {
  const dim3 grid((unsigned)(a.B * a.ncg));
  if (in_dtype == 1) {
    if (a.z) hipLaunchKernelGGL((unitary_fwd_xdl_kernel<3, true, bf16_t>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((unitary_fwd_xdl_kernel<3, false, bf16_t>), grid, dim3(256), 0, s, a);
  } else if (mode == 2) {
    if (a.z) hipLaunchKernelGGL((unitary_fwd_xdl_kernel<2, true>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((unitary_fwd_xdl_kernel<2, false>), grid, dim3(256), 0, s, a);
  } else {
    if (a.z) hipLaunchKernelGGL((unitary_fwd_xdl_kernel<3, true>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((unitary_fwd_xdl_kernel<3, false>), grid, dim3(256), 0, s, a);
  }
  return launch_status();
}

int run_xdl_bwd(int mode, const UniBwdArgs& a, int in_dtype, hipStream_t s) {
  const dim3 grid((unsigned)(a.B * a.ncg));
  if (in_dtype == 1) hipLaunchKernelGGL((unitary_bwd_xdl_kernel<3, 2, bf16_t>), grid, dim3(256), 0, s, a);
  else if (mode == 2) hipLaunchKernelGGL((unitary_bwd_xdl_kernel<2, 2>), grid, dim3(256), 0, s, a);
  else if (mode == 5) hipLaunchKernelGGL((unitary_bwd_xdl_kernel<3, 3>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((unitary_bwd_xdl_kernel<3, 2>), grid, dim3(256), 0, s, a);
  return launch_status();
}

int run_seg_state(bool adjoint, const SegArgs& a, int in_dtype, unsigned grid, hipStream_t s) {
  if (adjoint) {
    if (in_dtype == 1) hipLaunchKernelGGL((unitary_seg_state_kernel<3, true, bf16_t>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((unitary_seg_state_kernel<3, true>), dim3(grid), dim3(256), 0, s, a);
  } else {
    if (in_dtype == 1) hipLaunchKernelGGL((unitary_seg_state_kernel<3, false, bf16_t>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((unitary_seg_state_kernel<3, false>), dim3(grid), dim3(256), 0, s, a);
  }
  return launch_status();
}

int run_seg_carry_fwd(float* seg, const float* ptot, const float* h0, float* hL, int B, int D, int N, int nf, hipStream_t s) {
  const size_t nst = (size_t)B * D * N;
  if (nf > CARRY_SUBS * CARRY_RUN) return -2;
  hipLaunchKernelGGL(seg_carry_kernel<false>, dim3((unsigned)((nst + 31) / 32)), dim3(32 * CARRY_SUBS), 0, s, seg, ptot, h0, hL, B, D, N, nf);
  return launch_status();
}

int run_seg_carry_bwd(float* seg, const float* ptot, const float* dhL, float* dh0, int B, int D, int N, int nf, hipStream_t s) {
  const size_t nst = (size_t)B * D * N;
  if (nf > CARRY_SUBS * CARRY_RUN) return -2;
  hipLaunchKernelGGL(seg_carry_kernel<true>, dim3((unsigned)((nst + 31) / 32)), dim3(32 * CARRY_SUBS), 0, s, seg, ptot, dhL, dh0, B, D, N, nf);
  return launch_status();
}

}  // namespace aussm
