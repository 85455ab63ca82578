// Splitting the complex and the real (S6) scans along the sequence.  With few (batch, channel group)
// pairs a launch of the scan kernels leaves most of the chip idle, so the sequence is cut into ns
// segments and the scan runs over (batch, segment) pairs:
//   forward   1. core_fwd_kernel over the pairs from a zero state, outputs off: end state Z_k of every
//                segment and the product q_k of its a_l (FwdArgs::ptot),
//             2. the chain  h <- q_k h + Z_k  over the segments of each (batch, channel, state)
//                (seg_carry_kernel for complex states, seg_carry_real_kernel here),
//             3. core_fwd_kernel over the pairs, each from the state that enters it;
//   backward  1. adjoint_seg_kernel: adjoint Y_k of the state entering every segment from a zero adjoint
//                at its end (the reverse recurrence alone - no states are needed for it), and q_k,
//             2. the chain  g <- conj(q_k) g + Y_k, last segment first,
//             3. recompute_bwd_kernel over the pairs, each from the adjoint that enters it at its end.
// The unitary scan on the vector-ALU kernels (more than 16 states, a length that is not a multiple of 4, ...)
// splits the same way: core_fwd_kernel<VAR_UNITARY> for 1. and 3., the complex instance of adjoint_seg_kernel
// without rho, the complex chains, and unitary_bwd_kernel over the pairs, which takes the state at the end of
// each segment from the forward pass's checkpoints.
// Reference semantics: the loops of extension-cpp/extension_cpp/ops.py:215-223 (unitary), :270-291 (complex)
// and :349-356 (real) are associative in exactly this way; the reference itself does not split.
#pragma once
#include "scan_bwd_recompute.h"
#include "scan_common.h"

namespace aussm {

constexpr int ADJ_NSW = 16;      // states per wavefront of adjoint_seg_kernel (4 wavefronts: N <= 64)

// grid: (batch, segment) pairs x channel groups; 256 threads.  Lane = channel in the scan part, wavefront
// w owns the states w, w + 4, ...; tiles of 16 steps are staged like in recompute_bwd_kernel (lanes
// along time), two LDS buffers so that one barrier per tile is enough.
template <int VAR, typename Tin, typename Tbc = Tin>
__global__ __launch_bounds__(256) void adjoint_seg_kernel(const AdjSegArgs p) {
  static_assert(VAR == VAR_COMPLEX || VAR == VAR_REAL, "the unitary scan runs the complex instance without rho");
  constexpr int C = (VAR == VAR_REAL) ? 1 : 2;
  constexpr int E = CH * RT / 256;
  constexpr int RSTEP = 256 / RT;
  __shared__ float4 s_in[2][RT * TS];          // complex (Re a, Im a, dy silu(z), -); real (delta, dy silu(z), -, -)

  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int vb = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int b = vb / p.ns, sg = vb - b * p.ns;
  const int lbeg = sg * p.L, ld = p.ld;
  const int N = p.N, D = p.D;
  const int L = (ld - lbeg < p.L) ? ld - lbeg : p.L;
  const int d = d0 + lane;
  const bool dok = d < D;
  const Tin* __restrict__ gdl = static_cast<const Tin*>(p.delta);
  const Tbc* __restrict__ gC = static_cast<const Tbc*>(p.Cm);

  float gr[ADJ_NSW], gi[ADJ_NSW], a2[ADJ_NSW];
#pragma unroll
  for (int k = 0; k < ADJ_NSW; ++k) {
    const int n = wave + 4 * k;
    gr[k] = 0.f; gi[k] = 0.f;
    a2[k] = (VAR == VAR_REAL && dok && n < N) ? p.A[(size_t)d * N + n] * LOG2E : 0.f;
  }
  float fr = (VAR == VAR_REAL) ? 0.f : 1.f, fi = 0.f;      // product of the a_l / sum of the step sizes (wavefront 0)

  const int col = tid % RT, row0 = tid / RT;
  size_t goff[E];
  bool rowok[E];
  float dbias[E];
#pragma unroll
  for (int k = 0; k < E; ++k) {
    const int dd = d0 + row0 + k * RSTEP;
    rowok[k] = dd < D;
    goff[k] = ((size_t)b * D + (rowok[k] ? dd : 0)) * ld + lbeg;
    dbias[k] = (VAR == VAR_REAL && p.delta_bias && rowok[k]) ? p.delta_bias[dd] : 0.f;
  }

  const int ntiles = (L + RT - 1) / RT;
  for (int it = ntiles - 1; it >= 0; --it) {
    const int l0 = it * RT;
    float4* buf = s_in[it & 1];
    // ---- stage: steps past the end of the segment get a = 1 and a zero gradient
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const bool ok = rowok[k] && l0 + col < L;
      const size_t o = goff[k] + ((l0 + col < L) ? l0 + col : L - 1);
      float gy = ok ? p.dy[o] : 0.f;
      if (p.z) gy *= siluf_(p.z[o]);
      float4 rec;
      if (VAR == VAR_REAL) {
        float dl = to_f32(gdl[o]) + dbias[k];
        if (p.delta_softplus) dl = softplusf_(dl);
        rec = make_float4(ok ? dl : 0.f, gy, 0.f, 0.f);
      } else {
        float sn, cs;
        fast_sincosf(ok ? p.theta[o] : 0.f, &sn, &cs);
        const float r = p.rho ? expf(ok ? p.rho[o] : 0.f) : 1.f;     // (no rho: the unitary scan, uniform)
        rec = make_float4(cs * r, sn * r, gy, 0.f);
      }
      buf[col * TS + row0 + k * RSTEP] = rec;
    }
    __syncthreads();

    // ---- reverse recurrence  g <- conj(a_l) (g + conj(C_l) dy_l)
#pragma unroll
    for (int g = RT / TG - 1; g >= 0; --g) {
      float r0[TG], r1[TG], r2[TG];
#pragma unroll
      for (int t = 0; t < TG; ++t) {
        const float4 v = buf[(g * TG + t) * TS + lane];
        r0[t] = v.x; r1[t] = v.y; r2[t] = v.z;
      }
      if (wave == 0) {
#pragma unroll
        for (int t = 0; t < TG; ++t) {
          if (VAR == VAR_REAL) {
            fr += r0[t];
          } else {
            const float nr = fmaf(fr, r0[t], -fi * r1[t]);
            fi = fmaf(fr, r1[t], fi * r0[t]);
            fr = nr;
          }
        }
      }
#pragma unroll
      for (int k = 0; k < ADJ_NSW; ++k) {
        const int n = wave + 4 * k;
        if (n < N) {                             // wave-uniform
          const size_t row = ((size_t)b * N + n) * ld + lbeg;
          if constexpr (VAR == VAR_REAL) {
            const f32x8 cc = ld_r8_safe(gC, row, l0 + g * TG, L);
#pragma unroll
            for (int t = TG - 1; t >= 0; --t)
              gr[k] = fmaf(cc[t], r1[t], gr[k]) * __builtin_amdgcn_exp2f(r0[t] * a2[k]);
          } else {
            const f32x16 cc = ld_c8_safe(gC, row, l0 + g * TG, L);
#pragma unroll
            for (int t = TG - 1; t >= 0; --t) {
              const float xr = fmaf(cc[2 * t], r2[t], gr[k]);
              const float xi = fmaf(-cc[2 * t + 1], r2[t], gi[k]);
              gr[k] = fmaf(r0[t], xr, r1[t] * xi);
              gi[k] = fmaf(r0[t], xi, -r1[t] * xr);
            }
          }
        }
      }
    }
    // (no second barrier: the next tile is staged into the other buffer, whose readers all passed
    // the barrier above)
  }

  if (dok) {
#pragma unroll
    for (int k = 0; k < ADJ_NSW; ++k) {
      const int n = wave + 4 * k;
      if (n < N) {
        const size_t o = (((size_t)vb * D + d) * N + n) * C;
        p.out[o] = gr[k];
        if (C == 2) p.out[o + 1] = gi[k];
      }
    }
    if (wave == 0) {
      p.ptot[((size_t)vb * D + d) * 2] = fr;
      p.ptot[((size_t)vb * D + d) * 2 + 1] = fi;
    }
  }
}

// Chain of the segments of one (batch, channel, state) of the real scan, q_k = exp(A[d,n] * sum of the
// segment's step sizes).  Forward (ADJ false): on entry seg[k] holds the end state of segment k from a
// zero start, on return the state that enters it; the state after the last segment goes to `last`.
// ADJ: on entry the adjoint at the start of segment k from a zero adjoint at its end, on return the
// adjoint that enters it at its end, walking from the last segment; the adjoint of the initial state
// goes to `last`.  `first`: state before the first segment / adjoint after the last one (or null).
// B_t and C_t of a call with bf16 inputs, converted once (n elements each)
__global__ void bc_to_f32_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ b,
                                 float* __restrict__ oa, float* __restrict__ ob, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    oa[i] = to_f32(a[i]);
    ob[i] = to_f32(b[i]);
  }
}

template <bool ADJ>
__global__ void seg_carry_real_kernel(float* __restrict__ seg, const float* __restrict__ ptot,
                                      const float* __restrict__ A, const float* __restrict__ first,
                                      float* __restrict__ last, int B, int D, int N, int ns) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (size_t)B * D * N) return;
  const int n = (int)(idx % N);
  const int d = (int)((idx / N) % D);
  const int b = (int)(idx / ((size_t)N * D));
  const float a2 = A[(size_t)d * N + n] * LOG2E;
  float h = first ? first[idx] : 0.0f;
  for (int j = 0; j < ns; ++j) {
    const int k = ADJ ? ns - 1 - j : j;
    const size_t v = ((size_t)b * ns + k) * D + d;
    const float z = seg[v * N + n];
    const float q = __builtin_amdgcn_exp2f(ptot[v * 2] * a2);
    seg[v * N + n] = h;
    h = fmaf(q, h, z);
  }
  if (last) last[idx] = h;
}

}  // namespace aussm
