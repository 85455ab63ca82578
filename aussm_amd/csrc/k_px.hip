// Translation unit of the matrix-core unitary kernels that run on prepared operands (scan_px.h).
#include "launch.h"
#include "scan_px.h"

namespace aussm {

int run_px_prep(const PrepArgs& a, int B, int in_dtype, hipStream_t s) {
  const dim3 grid((unsigned)(B * a.nch));
  if (a.have) {
    if (in_dtype == 1) hipLaunchKernelGGL((unitary_px_prep_kernel<bf16_t, true>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((unitary_px_prep_kernel<float, true>), grid, dim3(256), 0, s, a);
  } else {
    if (in_dtype == 1) hipLaunchKernelGGL((unitary_px_prep_kernel<bf16_t, false>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((unitary_px_prep_kernel<float, false>), grid, dim3(256), 0, s, a);
  }
  return launch_status();
}

int run_px_fwd(const FwdArgs& a, const u4* img, const ImgNote& note, int in_dtype, hipStream_t s) {
  const dim3 grid((unsigned)(a.B * a.ncg));
  if (in_dtype == 1) {
    if (a.z) hipLaunchKernelGGL((unitary_fwd_px_kernel<true, bf16_t>), grid, dim3(512), 0, s, a, img, note);
    else hipLaunchKernelGGL((unitary_fwd_px_kernel<false, bf16_t>), grid, dim3(512), 0, s, a, img, note);
  } else {
    if (a.z) hipLaunchKernelGGL((unitary_fwd_px_kernel<true, float>), grid, dim3(512), 0, s, a, img, note);
    else hipLaunchKernelGGL((unitary_fwd_px_kernel<false, float>), grid, dim3(512), 0, s, a, img, note);
  }
  return launch_status();
}

int run_px_bwd(const UniBwdArgs& a, const u4* img, int in_dtype, hipStream_t s) {
  const dim3 grid((unsigned)(a.B * a.ncg));
  if (in_dtype == 1) hipLaunchKernelGGL((unitary_bwd_px_kernel<2, bf16_t>), grid, dim3(512), 0, s, a, img);
  else hipLaunchKernelGGL((unitary_bwd_px_kernel<2, float>), grid, dim3(512), 0, s, a, img);
  return launch_status();
}

}  // namespace aussm
