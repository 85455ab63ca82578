// Translation unit of the fused operator kernels (dropin.h).
#include "launch.h"
#include "dropin.h"

namespace aussm {

void run_dropin_xprep(const float* x, u4* xp, int d, int n, int ks, int nb, hipStream_t s) {
  const size_t total = (size_t)d * nb * ks * 64;
  hipLaunchKernelGGL(dropin_xprep_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, x, xp, d, n, ks, nb);
}

void run_fill(const FillArgs& a, hipStream_t s) {
  size_t most = 0;
  for (int i = 0; i < a.count; ++i) most = a.n[i] > most ? a.n[i] : most;
  if (!a.count || !most) return;
  size_t blocks = (most + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks, (unsigned)a.count), dim3(256), 0, s, a);
}

#ifndef DROPIN_NW_
#define DROPIN_NW_ 8
#endif
constexpr int DROPIN_NW = DROPIN_NW_;     // channels (wavefronts) per workgroup

// (d > 256: the rows of x take 192 registers, which leaves room for one wavefront per SIMD only)
template <int KS>
static void launch_fwd(const DropinArgs& a, hipStream_t s) {
  constexpr int NW = KS > 8 ? 4 : DROPIN_NW;
  const unsigned grid = (unsigned)(a.b * ((a.d * a.nb + NW - 1) / NW));
  hipLaunchKernelGGL((dropin_fwd_kernel<KS, NW>), dim3(grid), dim3(NW * 64), 0, s, a);
}
template <int KS>
static void launch_bwd(const DropinBwdArgs& a, hipStream_t s) {
  constexpr int NW = KS > 8 ? 4 : DROPIN_NW;
  const unsigned grid = (unsigned)(a.bg * ((a.f.d * a.f.nb + NW - 1) / NW));
  hipLaunchKernelGGL((dropin_bwd_kernel<KS, NW>), dim3(grid), dim3(NW * 64), 0, s, a);
}

int dropin_channels_per_workgroup(int ks) { return ks > 8 ? 4 : DROPIN_NW; }

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
  if (a.ksplit < 1 || a.zper < 1 || (!a.reduce_z && a.zper != 1)) return -2;
  const long gz = (long)((a.Z + a.zper - 1) / a.zper) * a.ksplit;
  if (gz > 65535) return -2;
  const dim3 grid((unsigned)((a.M + 127) / 128), (unsigned)((a.N + 63) / 64), (unsigned)gz);
  const bool k1 = a.sak == 1 && a.sbk == 1;
  if (k1) hipLaunchKernelGGL((split_gemm_kernel<true, true>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((split_gemm_kernel<false, false>), grid, dim3(256), 0, s, a);
  return launch_status();
}

}  // namespace aussm
