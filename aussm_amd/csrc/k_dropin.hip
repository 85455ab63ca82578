// Translation unit of the fused operator kernels (dropin.h).
#include "launch.h"
#include "dropin.h"

namespace aussm {

int run_dropin_xprep(const float* x, u4* xp, int d, int n, int ks, int nb, hipStream_t s) {
  const size_t total = (size_t)d * nb * ks * 64;
  hipLaunchKernelGGL(dropin_xprep_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, x, xp, d, n, ks, nb);
  return launch_status();
}

int run_fill(const FillArgs& a, hipStream_t s) {
  size_t most = 0;
  for (int i = 0; i < a.count; ++i) most = a.n[i] > most ? a.n[i] : most;
  if (!a.count || !most) return 0;
  size_t blocks = (most + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks, (unsigned)a.count), dim3(256), 0, s, a);
  return launch_status();
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

// the compiled size of the contraction (steps of 32) that serves ceil(d / 32) = ks
int dropin_compiled_ks(int ks) { return ks <= 4 ? (ks < 1 ? 1 : ks) : ks <= 6 ? 6 : ks <= 8 ? 8 : ks <= 12 ? 12 : 16; }

int run_dropin_uprep(const float* u, u4* up, int d, int L, int ks, int b0, int bg, int t0, int nt, hipStream_t s) {
  hipLaunchKernelGGL(dropin_uprep_kernel, dim3((unsigned)(bg * nt)), dim3(256), 0, s, u, up, d, L, dropin_compiled_ks(ks), b0, t0, nt);
  return launch_status();
}

// compiled sizes of the contraction over r, in steps of 32: the smallest one >= ceil(d / 32) runs
#define DROPIN_KS_DISPATCH(LAUNCH, ks)          \
  if (ks <= 1) LAUNCH<1>(a, s);                 \
  else if (ks <= 2) LAUNCH<2>(a, s);            \
  else if (ks <= 3) LAUNCH<3>(a, s);            \
  else if (ks <= 4) LAUNCH<4>(a, s);            \
  else if (ks <= 6) LAUNCH<6>(a, s);            \
  else if (ks <= 8) LAUNCH<8>(a, s);            \
  else if (ks <= 12) LAUNCH<12>(a, s);          \
  else LAUNCH<16>(a, s);

int run_dropin_fwd(const DropinArgs& a, hipStream_t s) {
  DROPIN_KS_DISPATCH(launch_fwd, a.ks)
  return launch_status();
}

int run_dropin_bwd(const DropinBwdArgs& a, hipStream_t s) {
  DROPIN_KS_DISPATCH(launch_bwd, a.f.ks)
  return launch_status();
}

int run_split_gemm(const GemmArgs& a, hipStream_t s) {
  if (a.ksplit < 1 || a.zper < 1 || (!a.reduce_z && a.zper != 1) || !a.Aimg) return -2;
  const long gz = (long)((a.Z + a.zper - 1) / a.zper) * a.ksplit;
  if (gz > 65535) return -2;
  constexpr int TNH = GEMM_TILE_N / 64;
  const dim3 grid((unsigned)((a.M + 127) / 128), (unsigned)((a.N + 64 * TNH - 1) / (64 * TNH)), (unsigned)gz);
  const bool k1 = a.sbk == 1;
  if (k1 && a.tr) hipLaunchKernelGGL((split_gemm_kernel<true, true, true, TNH>), grid, dim3(256), 0, s, a);
  else if (k1) hipLaunchKernelGGL((split_gemm_kernel<true, true, false, TNH>), grid, dim3(256), 0, s, a);
  else if (a.tr) hipLaunchKernelGGL((split_gemm_kernel<false, false, true, TNH>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((split_gemm_kernel<false, false, false, TNH>), grid, dim3(256), 0, s, a);
  return launch_status();
}

// records of the image of an A with M rows and K columns (one z)
size_t gemm_image_records(int M, int K) { return (size_t)8 * ((M + 127) / 128) * ((K + 31) / 32) * 3 * 64; }

int run_gemm_aprep(const float* A, u4* img, long sam, long sak, long saz, int M, int K, int Z, hipStream_t s) {
  const int m16 = 8 * ((M + 127) / 128), nk = (K + 31) / 32;
  const long total = (long)Z * m16 * nk * 64;
  if (total <= 0 || (total + 255) / 256 > 0x7fffffffL) return -2;
  hipLaunchKernelGGL(gemm_aprep_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, A, img, sam, sak, saz, M, K, m16, nk, total);
  return launch_status();
}

}  // namespace aussm
