// Launch functions of the library's translation units (one unit per kernel family, so that they
// compile side by side).  Each enqueues on the given stream and returns AUSSM_OK or the launch's
// hipError_t; argument checking is done by the callers in scan_api.hip.
#pragma once
#include <hip/hip_runtime.h>

#include "scan_args.h"
#include "dropin_args.h"

namespace aussm {

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

// A workgroup of nt threads (nt / 64 wavefronts) of the vector-ALU kernels owns 64 channels; each
// wavefront owns nw states.
struct Cfg { int nw, nt; };

// ---- k_generic.hip: vector-ALU scans, convolution, layout swap
// in_dtype: 0 float, 1 bf16 (unitary only), 2 = u / delta bf16 and B_t / C_t float (complex and real only)
int run_core_fwd(int variant, const FwdArgs& a, int in_dtype, Cfg c, hipStream_t s);
int run_unitary_bwd_generic(const UniBwdArgs& a, int in_dtype, Cfg c, hipStream_t s);
int run_rec_bwd(int variant, const RecBwdArgs& a, int in_dtype, hipStream_t s);
int run_aux_invalidate(float* tag, bool fill_tag, bool images_tag, hipStream_t s);   // clears tag(s) in the buffer's pad
// split of the complex / real scans along L: adjoint entering every segment, chain of the real scan's segments
int run_adjoint_seg(int variant, const AdjSegArgs& a, int in_dtype, unsigned grid, hipStream_t s);
int run_bc_to_f32(const void* Bm, const void* Cm, float* oB, float* oC, size_t n, hipStream_t s);   // bf16 -> float
int run_seg_carry_real(bool adjoint, float* seg, const float* ptot, const float* A, const float* first, float* last,
                        int B, int D, int N, int ns, hipStream_t s);
int run_hbm_probe(const float* a, const float* b, const float* c, float* o1, float* o2, int rows, int L, int pattern,
                  int write, hipStream_t s);
int run_conv_fwd(const ConvArgs& a, hipStream_t s);
int run_conv_bwd(const ConvArgs& a, hipStream_t s);
int run_swap_last2(const SwapArgs& a, int B, hipStream_t s);
// dz null: out = ypre silu(z); else out = dy silu(z), dz = dy ypre silu'(z)
int run_gate(const float* dy, const float* ypre, const float* z, float* out, float* dz, size_t n, hipStream_t s);

// ---- k_xdl.hip: matrix-core unitary scans that prepare their operands themselves, and the
// kernels of the split along L.  mode: operand pieces (2, 3; backward also 5 = three everywhere).
int run_xdl_fwd(int mode, const FwdArgs& a, int in_dtype, hipStream_t s);
int run_xdl_bwd(int mode, const UniBwdArgs& a, int in_dtype, hipStream_t s);
int run_seg_state(bool adjoint, const SegArgs& a, int in_dtype, unsigned grid, hipStream_t s);
int run_seg_carry_fwd(float* seg, const float* ptot, const float* h0, float* hL, int B, int D, int N, int nf, hipStream_t s);
int run_seg_carry_bwd(float* seg, const float* ptot, const float* dhL, float* dh0, int B, int D, int N, int nf, hipStream_t s);

// ---- k_px.hip: matrix-core unitary scans on operands prepared by a pre-pass
int run_px_prep(const PrepArgs& a, int B, int in_dtype, hipStream_t s);
int run_px_fwd(const FwdArgs& a, const u4* img, const ImgNote& note, int in_dtype, hipStream_t s);
int run_px_bwd(const UniBwdArgs& a, const u4* img, int in_dtype, hipStream_t s);

// ---- k_dropin.hip: the reference's 12-input operator as fused kernels
int run_dropin_xprep(const float* x, u4* xp, int d, int n, int ks, int nb, hipStream_t s);
int dropin_channels_per_workgroup(int ks);
int dropin_compiled_ks(int ks);
int run_dropin_uprep(const float* u, u4* up, int d, int L, int ks, int b0, int bg, int t0, int nt, hipStream_t s);
int run_dropin_fwd(const DropinArgs& a, hipStream_t s);
int run_dropin_bwd(const DropinBwdArgs& a, hipStream_t s);
int run_fill(const FillArgs& a, hipStream_t s);   // several buffers set (zero or a copy) in one launch
constexpr int GEMM_TILE_M = 128, GEMM_TILE_N = 128;   // workgroup tile of run_split_gemm
int run_split_gemm(const GemmArgs& a, hipStream_t s);
size_t gemm_image_records(int M, int K);       // 16-byte records of the prepared image of an M x K operand
int run_gemm_aprep(const float* A, u4* img, long sam, long sak, long saz, int M, int K, int Z, hipStream_t s);

}  // namespace aussm
