// Translation unit of the vector-ALU kernels: the three forward scans, the unitary reverse scan,
// the recomputing reverse scans (complex, real), the causal convolution and the layout swap.
#include "conv1d.h"
#include "launch.h"
#include "layout.h"
#include "scan_bwd_recompute.h"
#include "scan_bwd_unitary.h"
#include "scan_fwd.h"
#include "scan_seg_generic.h"

namespace aussm {

#define AUSSM_FWD_CASE(NW_, NT_)                                                                     \
  if (c.nw == NW_ && c.nt == NT_) {                                                                  \
    hipLaunchKernelGGL((core_fwd_kernel<VAR, NW_, NT_, Tin, Tbc>), grid, dim3(NT_), 0, s, a);        \
    return launch_status();                                                                          \
  }

// in_dtype of the launch functions below: 0 float, 1 bf16, 2 (complex and real scans only, which take no
// bf16 B_t / C_t) u and delta bf16 with B_t / C_t already converted to float
constexpr int IN_BF16_BC32 = 2;

template <int VAR, typename Tin, typename Tbc>
static int core_fwd_t(const FwdArgs& a, Cfg c, hipStream_t s) {
  const dim3 grid((unsigned)(a.B * a.ncg));
  AUSSM_FWD_CASE(1, 256) AUSSM_FWD_CASE(2, 256) AUSSM_FWD_CASE(4, 256) AUSSM_FWD_CASE(8, 256)
  AUSSM_FWD_CASE(16, 256) AUSSM_FWD_CASE(1, 512) AUSSM_FWD_CASE(2, 512) AUSSM_FWD_CASE(4, 512)
  AUSSM_FWD_CASE(8, 512)
  return -2;
}

template <int VAR>
static int core_fwd_v(const FwdArgs& a, int in_dtype, Cfg c, hipStream_t s) {
  if (in_dtype == 0) return core_fwd_t<VAR, float, float>(a, c, s);
  if constexpr (VAR == VAR_UNITARY) {
    if (in_dtype == 1) return core_fwd_t<VAR, bf16_t, bf16_t>(a, c, s);
  } else {
    if (in_dtype == IN_BF16_BC32) return core_fwd_t<VAR, bf16_t, float>(a, c, s);
  }
  return -2;
}

int run_core_fwd(int variant, const FwdArgs& a, int in_dtype, Cfg c, hipStream_t s) {
  if (variant == VAR_UNITARY) return core_fwd_v<VAR_UNITARY>(a, in_dtype, c, s);
  if (variant == VAR_COMPLEX) return core_fwd_v<VAR_COMPLEX>(a, in_dtype, c, s);
  return core_fwd_v<VAR_REAL>(a, in_dtype, c, s);
}

// The backward workgroup keeps a (dw, dtheta) slab per wavefront in LDS: four wavefronts afford
// 32-step tiles, eight wavefronts 16-step tiles.
#define AUSSM_UBWD_CASE(NW_, NT_, TT_)                                                               \
  if (c.nw == NW_ && c.nt == NT_) {                                                                  \
    hipLaunchKernelGGL((unitary_bwd_kernel<NW_, NT_, TT_, Tin>), grid, dim3(NT_), 0, s, a);          \
    return launch_status();                                                                          \
  }

template <typename Tin>
static int unitary_bwd_t(const UniBwdArgs& a, Cfg c, hipStream_t s) {
  const dim3 grid((unsigned)(a.B * a.ncg));
  AUSSM_UBWD_CASE(1, 256, 32) AUSSM_UBWD_CASE(2, 256, 32) AUSSM_UBWD_CASE(4, 256, 32)
  AUSSM_UBWD_CASE(8, 256, 32) AUSSM_UBWD_CASE(16, 256, 32)
  AUSSM_UBWD_CASE(1, 512, 16) AUSSM_UBWD_CASE(2, 512, 16) AUSSM_UBWD_CASE(4, 512, 16)
  AUSSM_UBWD_CASE(8, 512, 16)
  return -2;
}

int run_unitary_bwd_generic(const UniBwdArgs& a, int in_dtype, Cfg c, hipStream_t s) {
  return in_dtype == 1 ? unitary_bwd_t<bf16_t>(a, c, s) : unitary_bwd_t<float>(a, c, s);
}

#define AUSSM_RBWD_CASE(NW_)                                                                         \
  if (nw == NW_) {                                                                                   \
    hipLaunchKernelGGL((recompute_bwd_kernel<VAR, NW_, 256, Tin, float>), grid, dim3(256), 0, s, a); \
    done = true;                                                                                     \
  }

template <int VAR, typename Tin>
static int rec_bwd_t(const RecBwdArgs& args, hipStream_t s) {
  const dim3 grid((unsigned)(args.B * args.ncg));
  // one launch per block of 16 states (stream order makes the later blocks' additions safe)
  for (int nbase = 0; nbase < args.N; nbase += 16) {
    RecBwdArgs a = args;
    a.nbase = nbase;
    a.accum = nbase > 0;
    const int left = args.N - nbase;
    const int nw = left <= 4 ? 1 : (left <= 8 ? 2 : 4);
    bool done = false;
#ifndef AUSSM_REC_NARROW
    // a full block of 16 states: eight wavefronts of two states, two wavefronts per SIMD (the complex scan with a
    // gate gradient to return keeps a fourth partial sum per wavefront)
    if (left > 8) {
      if constexpr (VAR == VAR_COMPLEX) {
        if (a.dz) hipLaunchKernelGGL((recompute_bwd_kernel<VAR, 2, 512, Tin, float, true>), grid, dim3(512), 0, s, a);
        else hipLaunchKernelGGL((recompute_bwd_kernel<VAR, 2, 512, Tin, float, false>), grid, dim3(512), 0, s, a);
      } else {
        hipLaunchKernelGGL((recompute_bwd_kernel<VAR, 2, 512, Tin, float>), grid, dim3(512), 0, s, a);
      }
      done = true;
    }
#endif
    if (!done) { AUSSM_RBWD_CASE(1) AUSSM_RBWD_CASE(2) AUSSM_RBWD_CASE(4) }
    if (!done) return -2;
    if (int e = launch_status()) return e;
  }
  return 0;
}

int run_rec_bwd(int variant, const RecBwdArgs& a, int in_dtype, hipStream_t s) {
  if (in_dtype != 0 && in_dtype != IN_BF16_BC32) return -2;      // B_t / C_t are float in every instance
  if (variant == VAR_COMPLEX)
    return in_dtype ? rec_bwd_t<VAR_COMPLEX, bf16_t>(a, s) : rec_bwd_t<VAR_COMPLEX, float>(a, s);
  return in_dtype ? rec_bwd_t<VAR_REAL, bf16_t>(a, s) : rec_bwd_t<VAR_REAL, float>(a, s);
}

int run_adjoint_seg(int variant, const AdjSegArgs& a, int in_dtype, unsigned grid, hipStream_t s) {
  // (B_t / C_t are float in every instance of the complex and real scans; the complex kernel reads no u / delta
  // at all.  The unitary scan runs the complex instance without rho, with C_t in the type of its inputs.)
  if (variant == VAR_UNITARY) {
    if (in_dtype == 1) hipLaunchKernelGGL((adjoint_seg_kernel<VAR_COMPLEX, float, bf16_t>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((adjoint_seg_kernel<VAR_COMPLEX, float, float>), dim3(grid), dim3(256), 0, s, a);
  } else if (variant == VAR_COMPLEX) {
    hipLaunchKernelGGL((adjoint_seg_kernel<VAR_COMPLEX, float, float>), dim3(grid), dim3(256), 0, s, a);
  } else {
    if (in_dtype) hipLaunchKernelGGL((adjoint_seg_kernel<VAR_REAL, bf16_t, float>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((adjoint_seg_kernel<VAR_REAL, float, float>), dim3(grid), dim3(256), 0, s, a);
  }
  return launch_status();
}

int run_bc_to_f32(const void* Bm, const void* Cm, float* oB, float* oC, size_t n, hipStream_t s) {
  const size_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(bc_to_f32_kernel, dim3((unsigned)(blocks < 2048 ? blocks : 2048)), dim3(256), 0, s,
                     static_cast<const bf16_t*>(Bm), static_cast<const bf16_t*>(Cm), oB, oC, n);
  return launch_status();
}

int run_seg_carry_real(bool adjoint, float* seg, const float* ptot, const float* A, const float* first, float* last,
                        int B, int D, int N, int ns, hipStream_t s) {
  const size_t n = (size_t)B * D * N;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (adjoint) hipLaunchKernelGGL(seg_carry_real_kernel<true>, grid, dim3(256), 0, s, seg, ptot, A, first, last, B, D, N, ns);
  else hipLaunchKernelGGL(seg_carry_real_kernel<false>, grid, dim3(256), 0, s, seg, ptot, A, first, last, B, D, N, ns);
  return launch_status();
}

// ---- what the memory system gives for the scans' access pattern (no arithmetic to speak of): o1 = a + b c,
// o2 = 2 o1 over [rows, L] tensors.  PATTERN 0: every thread streams consecutive 16-byte pieces (a plain
// elementwise kernel).  PATTERN 1: what the matrix-core scan kernels do - a workgroup owns 64 rows, its eight
// wavefronts are four groups of 16 rows times two halves that take the 32-step chunks in turn, and one load or
// store instruction of a wavefront covers 16 rows x 64 bytes (the two halves of a 128-byte line in two
// consecutive instructions), loads running two chunks ahead of their use.
template <int PATTERN, bool WRITE>
__global__ __launch_bounds__(512) void hbm_probe_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                        const float* __restrict__ c, float* __restrict__ o1,
                                                        float* __restrict__ o2, int rows, int L) {
  typedef float v4 __attribute__((ext_vector_type(4)));
  v4 acc = {0, 0, 0, 0};
  if (PATTERN == 0) {
    const size_t n4 = (size_t)rows * L / 4;
    for (size_t i = (size_t)blockIdx.x * 512 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 512) {
      const v4 x = reinterpret_cast<const v4*>(a)[i] + reinterpret_cast<const v4*>(b)[i] * reinterpret_cast<const v4*>(c)[i];
      if (WRITE) { reinterpret_cast<v4*>(o1)[i] = x; reinterpret_cast<v4*>(o2)[i] = x + x; } else acc += x;
    }
  } else {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, cg = w & 3, hf = w >> 2;
    const int dl = lane & 15, g = lane >> 4;
    const size_t row = (size_t)blockIdx.x * 64 + cg * 16 + dl;
    const int nch = L / 64;                       // chunks of this half (L is a multiple of 64)
    auto at = [&](int u, int st) -> size_t { return row * L + (size_t)(2 * u + hf) * 32 + 16 * st + 4 * g; };
    v4 buf[2][2][3];
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const size_t o = at(q < nch ? q : nch - 1, st);
        buf[q][st][0] = *reinterpret_cast<const v4*>(a + o);
        buf[q][st][1] = *reinterpret_cast<const v4*>(b + o);
        buf[q][st][2] = *reinterpret_cast<const v4*>(c + o);
      }
    for (int u = 0; u < nch; u += 2) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        if (u + q >= nch) break;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const v4 x = buf[q][st][0] + buf[q][st][1] * buf[q][st][2];
          const size_t o = at(u + q, st);
          if (WRITE) { *reinterpret_cast<v4*>(o1 + o) = x; *reinterpret_cast<v4*>(o2 + o) = x + x; } else acc += x;
        }
        const int un = u + q + 2 < nch ? u + q + 2 : u + q;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const size_t o = at(un, st);
          buf[q][st][0] = *reinterpret_cast<const v4*>(a + o);
          buf[q][st][1] = *reinterpret_cast<const v4*>(b + o);
          buf[q][st][2] = *reinterpret_cast<const v4*>(c + o);
        }
      }
    }
  }
  // (keeps the loads of the read-only form alive; never true for finite data)
  if (!WRITE && acc[0] + acc[1] + acc[2] + acc[3] == 1.2345678e38f) o1[0] = acc[0];
}
int run_hbm_probe(const float* a, const float* b, const float* c, float* o1, float* o2, int rows, int L, int pattern,
                  int write, hipStream_t s) {
  if (pattern == 0) {
    if (write) hipLaunchKernelGGL((hbm_probe_kernel<0, true>), dim3(2048), dim3(512), 0, s, a, b, c, o1, o2, rows, L);
    else hipLaunchKernelGGL((hbm_probe_kernel<0, false>), dim3(2048), dim3(512), 0, s, a, b, c, o1, o2, rows, L);
  } else {
    const dim3 grid((unsigned)(rows / 64));
    if (write) hipLaunchKernelGGL((hbm_probe_kernel<1, true>), grid, dim3(512), 0, s, a, b, c, o1, o2, rows, L);
    else hipLaunchKernelGGL((hbm_probe_kernel<1, false>), grid, dim3(512), 0, s, a, b, c, o1, o2, rows, L);
  }
  return launch_status();
}

// marks an auxiliary buffer as NOT filled (a forward kernel that does not fill it ran) and / or the
// operand images behind it as not belonging to the call's tensors
__global__ void aux_invalidate_kernel(float* tag, int first, int last) {
  if ((int)threadIdx.x >= first && (int)threadIdx.x <= last) tag[threadIdx.x] = 0.0f;
}
int run_aux_invalidate(float* tag, bool fill_tag, bool images_tag, hipStream_t s) {
  if (!fill_tag && !images_tag) return 0;
  hipLaunchKernelGGL(aux_invalidate_kernel, dim3(1), dim3(64), 0, s, tag, fill_tag ? 0 : AUX_IMG_FP,
                     images_tag ? AUX_IMG_FP + 7 : 0);
  return launch_status();
}

int run_conv_fwd(const ConvArgs& a, hipStream_t s) {
  const size_t rows = (size_t)a.B * a.L;
  const size_t runs = (size_t)a.B * ((a.L + CONV_RUN - 1) / CONV_RUN);
  if (a.K == 4)
    hipLaunchKernelGGL(causal_conv1d_k4_fwd_kernel, dim3((unsigned)runs, (unsigned)((a.D + 255) / 256)), dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL(causal_conv1d_fwd_kernel, dim3((unsigned)rows, (unsigned)((a.D + 255) / 256)), dim3(256), 0, s, a);
  return launch_status();
}

int run_conv_bwd(const ConvArgs& a, hipStream_t s) {
  const size_t rows = (size_t)a.B * a.L;
  const dim3 wgrid((unsigned)((a.D + 63) / 64), (unsigned)((rows + CONV_ROWS - 1) / CONV_ROWS));
  if (a.K == 4) {
    const size_t runs = (size_t)a.B * ((a.L + CONV_RUN - 1) / CONV_RUN);
    hipLaunchKernelGGL(causal_conv1d_k4_bwd_data_kernel, dim3((unsigned)runs, (unsigned)((a.D + 255) / 256)), dim3(256), 0, s, a);
    hipLaunchKernelGGL(causal_conv1d_k4_bwd_weight_kernel, wgrid, dim3(256), 0, s, a);
  } else {
    hipLaunchKernelGGL(causal_conv1d_bwd_data_kernel, dim3((unsigned)rows, (unsigned)((a.D + 255) / 256)), dim3(256), 0, s, a);
    hipLaunchKernelGGL(causal_conv1d_bwd_weight_kernel, wgrid, dim3(256), 0, s, a);
  }
  return launch_status();
}

int run_gate(const float* dy, const float* ypre, const float* z, float* out, float* dz, size_t n, hipStream_t s) {
  const size_t blocks = (n + 1023) / 1024;
  const dim3 grid((unsigned)(blocks < 8192 ? blocks : 8192));
  auto off16 = [](const void* q) { return q && (reinterpret_cast<uintptr_t>(q) & 15) != 0; };
  const int vec = !(off16(dy) || off16(ypre) || off16(z) || off16(out) || off16(dz));
  if (dz) hipLaunchKernelGGL(gate_bwd_kernel, grid, dim3(256), 0, s, dy, ypre, z, out, dz, n, vec);
  else hipLaunchKernelGGL(gate_fwd_kernel, grid, dim3(256), 0, s, ypre, z, out, n, vec);
  return launch_status();
}

int run_swap_last2(const SwapArgs& a, int B, hipStream_t s) {
  hipLaunchKernelGGL(swap_last2_kernel, dim3((unsigned)((a.C + 31) / 32), (unsigned)((a.R + 31) / 32), (unsigned)B), dim3(256), 0, s, a);
  return launch_status();
}

}  // namespace aussm
