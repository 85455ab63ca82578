// Translation unit of the fused operator kernels (dropin.h).
#include "launch.h"
#include "dropin.h"

namespace aussm {

void run_dropin_xprep(const float* x, u4* xp, int d, int n, int ks, hipStream_t s) {
  const size_t total = (size_t)d * ks * 64;
  hipLaunchKernelGGL(dropin_xprep_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, x, xp, d, n, ks);
}

void run_fill_zero(float* p, size_t n, hipStream_t s) {
  if (n) hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n);
}

#ifndef DROPIN_NW_
#define DROPIN_NW_ 8
#endif
constexpr int DROPIN_NW = DROPIN_NW_;     // channels (wavefronts) per workgroup

template <int KS>
static void launch_fwd(const DropinArgs& a, hipStream_t s) {
  const unsigned grid = (unsigned)(a.b * ((a.d + DROPIN_NW - 1) / DROPIN_NW));
  hipLaunchKernelGGL((dropin_fwd_kernel<KS, DROPIN_NW>), dim3(grid), dim3(DROPIN_NW * 64), 0, s, a);
}
template <int KS>
static void launch_bwd(const DropinBwdArgs& a, hipStream_t s) {
  const unsigned grid = (unsigned)(a.bg * ((a.f.d + DROPIN_NW - 1) / DROPIN_NW));
  hipLaunchKernelGGL((dropin_bwd_kernel<KS, DROPIN_NW>), dim3(grid), dim3(DROPIN_NW * 64), 0, s, a);
}

int run_dropin_fwd(const DropinArgs& a, hipStream_t s) {
  if (a.ks <= 1) launch_fwd<1>(a, s);
  else if (a.ks <= 2) launch_fwd<2>(a, s);
  else if (a.ks <= 4) launch_fwd<4>(a, s);
  else if (a.ks <= 8) launch_fwd<8>(a, s);
  else launch_fwd<16>(a, s);
  return launch_status();
}

int run_dropin_bwd(const DropinBwdArgs& a, hipStream_t s) {
  if (a.f.ks <= 1) launch_bwd<1>(a, s);
  else if (a.f.ks <= 2) launch_bwd<2>(a, s);
  else if (a.f.ks <= 4) launch_bwd<4>(a, s);
  else if (a.f.ks <= 8) launch_bwd<8>(a, s);
  else launch_bwd<16>(a, s);
  return launch_status();
}

int run_split_gemm(const GemmArgs& a, hipStream_t s) {
  if (a.ksplit < 1 || (long)a.Z * a.ksplit > 65535) return -2;
  const dim3 grid((unsigned)((a.M + 127) / 128), (unsigned)((a.N + 63) / 64), (unsigned)(a.Z * a.ksplit));
  const bool k1 = a.sak == 1 && a.sbk == 1;
  const bool vec = k1 && a.sam % 4 == 0 && a.sbn % 4 == 0 && a.saz % 4 == 0 && a.sbz % 4 == 0 &&
                   (reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.Bm)) % 16 == 0;
  if (k1 && vec) hipLaunchKernelGGL((split_gemm_kernel<true, true>), grid, dim3(256), 0, s, a);
  else if (k1) hipLaunchKernelGGL((split_gemm_kernel<true, false>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((split_gemm_kernel<false, false>), grid, dim3(256), 0, s, a);
  return launch_status();
}

}  // namespace aussm
