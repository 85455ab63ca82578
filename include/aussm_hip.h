/*
 * aussm_hip.h — C ABI of libaussm_hip.so, the MI355X (gfx950) selective-scan library.
 *
 * Every pointer is a DEVICE pointer unless stated otherwise.  Tensors are dense,
 * row-major, in the shapes given per function.  Functions enqueue work on the HIP
 * stream passed as `stream` (a hipStream_t cast to void*; NULL = default stream),
 * never synchronise, never allocate, and return 0 on success, a negative
 * AUSSM_E_* code for a rejected argument, or a positive hipError_t from the launch.
 *
 * Layout conventions
 *   B, D, N, L        batch, channels, state size per channel, sequence length
 *   u, delta, theta, rho, z, y, dy and their gradients      [B, D, L]
 *   complex B_t / C_t (unitary, complex variants)           [B, N, L, 2]  (re, im interleaved,
 *                                                            i.e. a torch complex64 [B,N,L] tensor)
 *   real B_t / C_t (real variant)                            [B, N, L]
 *   h0, hL, dh0, dhL  start / final state and their cotangents
 *                                                            [B, D, N, 2] complex, [B, D, N] real
 *   hck               checkpointed states at the END of every `ck`-step block,
 *                     [B, nck, N, C, D] with nck = ceil(L / ck), C = 2 (complex state) or 1;
 *                     channel index fastest so that a wavefront stores it coalesced.
 *                     The last block holds the final state.
 *   in_dtype          element type of u, delta, B_t, C_t: AUSSM_F32 or AUSSM_BF16.
 *                     Everything else (phases, skip, gate, states, outputs, gradients) is fp32
 *                     and the recurrence always accumulates in fp32.
 *
 * Reference interfaces these entry points replace are cited per function as
 * path:line inside the reference tree (arjunkaruvally/AUSSM).
 */
#ifndef AUSSM_HIP_H
#define AUSSM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AUSSM_F32 0
#define AUSSM_BF16 1

#define AUSSM_OK 0
#define AUSSM_E_NULL (-1)      /* a required pointer is NULL                         */
#define AUSSM_E_SHAPE (-2)     /* a dimension is out of the supported range          */
#define AUSSM_E_CK (-3)        /* checkpoint interval not accepted by this function  */
#define AUSSM_E_DTYPE (-4)     /* unknown in_dtype                                   */
#define AUSSM_E_ALIGN (-5)     /* a pointer is not aligned to its element size       */
#define AUSSM_E_SCRATCH (-6)   /* the call needs more workspace than the static scratch holds */

#define AUSSM_TILE 32          /* timesteps per staged tile; ck is a multiple of it, */
                               /* or exactly AUSSM_TILE / 2                          */
#define AUSSM_MAX_STATE 64     /* largest N accepted                                  */

/* Library version (major*10000 + minor*100 + patch). No reference counterpart. */
int aussm_version(void);

/* Human-readable text for a return code of this library (host pointer, static storage). */
const char* aussm_error_string(int code);

/* Process-wide options, for comparisons and tuning; none is needed for normal use.  value < 0
 * restores "let the library decide".  They are read once per call (atomics), so setting one
 * while another thread launches is safe; which of two racing values a launch sees is unspecified.
 * No reference counterpart (the reference fixes its launch table at compile time,
 * extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_forward.cu:215-266).
 *   AUSSM_OPT_UNITARY_FWD  forward kernel of the unitary scan: 0 vector ALU, 2 / 3 matrix cores on
 *                          two- / three-piece operands built inside the scan kernel (3 = fp32-accurate,
 *                          the choice where the shape allows and the call has no auxiliary buffer),
 *                          6 matrix cores on three-piece operands prepared once per batch element by a
 *                          pre-pass (the default for calls with an auxiliary buffer)
 *   AUSSM_OPT_UNITARY_BWD  backward kernel: 0 vector ALU, 2 two-piece operands, 3 three pieces
 *                          along the sequence and two in the sums over the channel, 5 three
 *                          pieces everywhere, 6 prepared operands
 *   AUSSM_OPT_SPLIT_CAP    largest number of segments a launch may be split into along L
 *                          (0 or 1: never split)
 *   AUSSM_OPT_BLOCK_KFLOATS   budget, in units of 1024 floats, of the blocks in which the fused operator calls
 *                          (aussm_ssm_adaptive_unitary_fwd / _bwd) walk their problem (default and largest
 *                          value 25600 = 100 MiB; the option can only lower it)
 * Workspace and auxiliary-buffer sizes do not depend on any option: a buffer sized by the query
 * functions below holds what a call of that shape uses under every setting.
 *   AUSSM_OPT_GENERIC_NW / AUSSM_OPT_GENERIC_NT   states per wavefront / threads per workgroup of
 *                          the vector-ALU kernels (both must be set; one of the built pairs) */
#define AUSSM_OPT_UNITARY_FWD 0
#define AUSSM_OPT_UNITARY_BWD 1
#define AUSSM_OPT_SPLIT_CAP 2
#define AUSSM_OPT_GENERIC_NW 3
#define AUSSM_OPT_GENERIC_NT 4
#define AUSSM_OPT_BLOCK_KFLOATS 5
#define AUSSM_OPT_COUNT 6
int aussm_set_option(int key, int value);
int aussm_get_option(int key);   /* -1 = unset */

/* nck = ceil(L / ck): number of checkpoint blocks the hck buffer must hold. */
int aussm_num_checkpoints(int L, int ck);

/* The checkpoint interval the backward pass of a variant requires (0 = any multiple of
 * AUSSM_TILE).  variant: 0 unitary, 1 complex, 2 real. */
int aussm_bwd_checkpoint_interval(int variant);

/* ---------------------------------------------------------------------------------------
 * Core adaptive-unitary scan
 *     h_l[b,d,n] = exp(i*theta_l[b,d]) * h_{l-1}[b,d,n] + delta_l[b,d] * B_l[b,n] * u_l[b,d]
 *     y_l[b,d]   = Re sum_n C_l[b,n] * h_l[b,d,n] + Dskip[d] * u_l[b,d]      (* silu(z_l[b,d]))
 * Replaces the recurrence of extension-cpp/extension_cpp/ops.py:215-223 (sequential scan) and
 * the device scan of extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_forward.cu:113-181
 * for a phase that is given per (b,d,l).
 * Optional (NULL allowed): Dskip, z, h0, y (NULL = states only), hL, hck.
 * Kernel choice is internal: calls with 6 <= N <= 16, L a multiple of 4, 16-byte aligned
 * tensors and ck a multiple of AUSSM_TILE run on the matrix cores (fp32-accurate, see the
 * kernel headers); every other accepted call runs on the vector ALU.  Results agree to
 * rounding.  aussm_set_option(AUSSM_OPT_UNITARY_FWD / _BWD, ...) forces one for comparisons.
 * ------------------------------------------------------------------------------------- */
int aussm_unitary_fwd(const void* u, const void* delta, const float* theta,
                      const void* Bc, const void* Cc, const float* Dskip, const float* z,
                      const float* h0, float* y, float* hL, float* hck,
                      int B, int D, int N, int L, int ck, int in_dtype, void* stream);

/* Reverse scan for aussm_unitary_fwd called WITHOUT a gate (z == NULL).  Recomputes the states
 * by running the (norm-preserving, hence invertible) recurrence backwards from the checkpoints
 * in hck, which must come from aussm_unitary_fwd on the same inputs with the same ck.
 * Replaces extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_backward.cu:22-491.
 * dB, dC use the convention dRe + i*dIm (what torch returns for a complex leaf).
 * Required: dy, u, delta, theta, Bc, Cc, hck, du, ddelta, dtheta, dB, dC.
 * Optional: dhL, Dskip, h0 (unused, may be NULL), dD, dh0.
 * dB, dC and dD are ACCUMULATED into (several channel groups add into the same element with
 * float atomics): the caller zero-fills them for a plain gradient, as the reference's host
 * launcher does (ssm_adaptive_unitary_backward.cu:531-543).  All other outputs are overwritten. */
int aussm_unitary_bwd(const float* dy, const float* dhL,
                      const void* u, const void* delta, const float* theta,
                      const void* Bc, const void* Cc, const float* Dskip, const float* hck,
                      float* du, float* ddelta, float* dtheta, float* dB, float* dC,
                      float* dD, float* dh0,
                      int B, int D, int N, int L, int ck, int in_dtype, void* stream);

/* Variants of the two calls above with an optional auxiliary buffer (NULL allowed; then they are
 * the calls above).  `aux` holds aussm_unitary_aux_floats(B, D, N, L, ck) floats, 16-byte aligned,
 * sized with the arguments of the calls it is passed to.  Three uses, all internal:
 *  - the forward call may leave per-(b,d,l) intermediate results in it (Im(P_t S_t), the term of
 *    the phase gradient that needs the forward states) together with a tag formed from the call's
 *    tensor addresses (u, delta, theta, Bc, Cc), B, D, N, L and in_dtype; a backward call given the
 *    same buffer AND the same tensors skips recomputing them.  A forward kernel that does not fill
 *    the buffer clears the tag, and a backward call whose arguments give another tag recomputes,
 *    so handing over `aux` is safe and only ever a speed-up - as long as the tensors are not
 *    modified in place between the two calls (the tag knows addresses, not contents);
 *  - the matrix-core kernels run on operands prepared from Bc and Cc by a pre-pass (split into bf16
 *    pieces, in the record orders the products need); they live at the end of the buffer.  A forward
 *    call that is given hck (a backward call can follow) prepares the backward call's operands in
 *    the same pre-pass and notes, behind the validity tag, what they were made from: the addresses
 *    of Bc and Cc, B, N, L and in_dtype.  A backward call whose arguments match that note uses them;
 *    any other backward call prepares its own.  So the contract for reusing one buffer is the
 *    autograd one: between a forward call and the backward call that is handed its buffer, Bc and
 *    Cc must not be modified in place, and no other call may be given the buffer;
 *  - a launch with few (batch, channel) pairs and a long sequence is split along L over more
 *    workgroups (per-segment end states from a zero start, a short chain over the segments, then
 *    the scan of every segment from its true incoming state - the two-level scan of
 *    ssm_adaptive_unitary_forward.cu:122-162 one level up); the segment states live behind the
 *    per-(b,d,l) part of the buffer, during the call only.  Each call writes there: two calls
 *    that share one buffer must not overlap.  aussm_set_option(AUSSM_OPT_SPLIT_CAP, 0) switches the split off.
 *    The vector-ALU kernels (more than 16 states, L not a multiple of 4, shared inputs, ...) split
 *    the same way, with their own kernels for the segment states; the buffer of a shape that only
 *    they serve has no per-(b,d,l) part and no operand images.
 * urep (>= 1, divides B): u and delta are [B / urep, D, L] and shared by urep consecutive batch
 * elements (theta, z, y, dy and every gradient stay [B, D, L]).  This is how the drop-in operator
 * runs its n states per channel, each with its own phase, as n batch elements of one launch without
 * replicating its inputs (the reference loops over the state inside one thread block,
 * ssm_adaptive_unitary_forward.cu:57-181).  urep > 1 takes the vector-ALU kernels.
 * No counterpart in the reference (its backward kernel recomputes,
 * ssm_adaptive_unitary_backward.cu:113-181, and its launches cover at most 2048 steps). */
size_t aussm_unitary_aux_floats(int B, int D, int N, int L, int ck);
/* Which kernel family a unitary call of this shape runs (tensors 16-byte aligned, current options):
 * 0 vector-ALU kernels, 2 / 3 / 5 matrix-core kernels that build their operands themselves,
 * 6 matrix-core kernels on operands prepared by a pre-pass.  have_aux: the call gets an auxiliary
 * buffer.  A caller can skip allocating that buffer when both directions answer 0 (the vector-ALU
 * kernels use it for the segment states of a split call only) and aussm_unitary_split_segments() answers 1. */
int aussm_unitary_kernel_mode(int backward, int B, int D, int N, int L, int ck, int in_dtype, int urep, int have_aux);

/* Number of segments a call of this shape is split into along L when it is given an auxiliary
 * buffer (1 = not split); lets a caller choose ck (a segment is a whole number of checkpoint blocks). */
int aussm_unitary_split_segments(int B, int D, int N, int L, int ck);

int aussm_unitary_fwd_aux(const void* u, const void* delta, const float* theta,
                          const void* Bc, const void* Cc, const float* Dskip, const float* z,
                          const float* h0, float* y, float* hL, float* hck, float* aux,
                          int B, int D, int N, int L, int ck, int in_dtype, int urep, void* stream);

int aussm_unitary_bwd_aux(const float* dy, const float* dhL,
                          const void* u, const void* delta, const float* theta,
                          const void* Bc, const void* Cc, const float* Dskip, const float* hck,
                          float* aux,
                          float* du, float* ddelta, float* dtheta, float* dB, float* dC,
                          float* dD, float* dh0,
                          int B, int D, int N, int L, int ck, int in_dtype, int urep, void* stream);

/* Forward unitary scan that ALLOCATES NOTHING and takes no workspace argument: the variant of
 * aussm_unitary_fwd_aux (called with hck == NULL, i.e. outputs and final state only) for callers
 * that cannot allocate device memory - code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose launcher
 * allocates its outputs per call, ssm_adaptive_unitary_forward.cu:215-222).
 * The one workspace such a call uses - the segment states of a launch with few (batch, channel)
 * pairs that is split along L, see above - lives in a device array of AUSSM_STATIC_SCRATCH_BYTES
 * inside the library, which every GPU the library runs on holds from the first use to the end of
 * the process.  Same arguments and results (to rounding) as aussm_unitary_fwd_aux with a buffer
 * sized for (B, D, N, L, ck); it runs the kernels that build their operands themselves, since it
 * has no room for prepared ones.  A call whose segment states do not fit returns AUSSM_E_SCRATCH.
 * All calls on one GPU share that GPU's array: calls that overlap there (different streams,
 * different threads) race; calls in one stream are ordered and safe.  Nothing in the array has
 * to start at zero (every state read is written earlier in the same call).
 * aussm_static_init() looks the array up for the CURRENT device (once per device; the entry point
 * does the same on its first use there): call it before a graph capture starts. */
#define AUSSM_STATIC_SCRATCH_BYTES (4u << 20)
int aussm_static_init(void);
int aussm_unitary_fwd_static(const void* u, const void* delta, const float* theta,
                             const void* Bc, const void* Cc, const float* Dskip, const float* z,
                             const float* h0, float* y, float* hL,
                             int B, int D, int N, int L, int ck, int in_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * Complex scan:  a_l = exp(rho_l[b,d] + i*theta_l[b,d]), otherwise as the unitary scan.
 * Replaces extension-cpp/extension_cpp/ops.py:270-291 (loop) and the semantics of
 * extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_complex.cu:181-293 / :358-660.
 * The backward pass needs hck written with ck == aussm_bwd_checkpoint_interval(1).
 *
 * workspace (complex and real scans, forward and backward): aussm_scan_workspace_floats() floats of
 * device memory, 16-byte aligned, contents irrelevant on entry; may be NULL for float inputs, required
 * (AUSSM_E_NULL otherwise) for bf16 inputs, whose B_t / C_t rows the call first converts to float in it
 * (the scan consumes them as wave-uniform scalar operands; converting them there costs a scalar
 * instruction per value).  With it, a call with fewer
 * than 129 (batch, group of 64 channels) pairs is split along the sequence into up to 64 segments of
 * at least 128 steps that run side by side (end state / adjoint of every segment from zero, a chain
 * over the segments, then the scan proper from the true incoming states), so that short batches of
 * long sequences fill the chip; results equal the unsplit call's up to fp32 rounding.  The function
 * answers 0 when the call needs none (pass NULL then).  No counterpart in the reference: its
 * complex kernel walks the sequence chunk after chunk inside one thread block
 * (ssm_adaptive_complex.cu:228-292, chunk size :313-321).
 * ------------------------------------------------------------------------------------- */
size_t aussm_scan_workspace_floats(int variant, int B, int D, int N, int L, int ck, int in_dtype);

int aussm_complex_fwd(const void* u, const void* delta, const float* rho, const float* theta,
                      const void* Bc, const void* Cc, const float* Dskip, const float* z,
                      const float* h0, float* y, float* hL, float* hck, float* workspace,
                      int B, int D, int N, int L, int ck, int in_dtype, void* stream);

/* z / dz of the two backward calls below (both NULL, or both given): the forward call was gated with this z
 * (y = y_pre silu(z)); dy is then the gradient of the gated y, the kernel applies the gate's derivative
 * itself and writes dz = dy y_pre silu'(z).  N <= 64 (one launch per block of 16 states). */
int aussm_complex_bwd(const float* dy, const float* dhL,
                      const void* u, const void* delta, const float* rho, const float* theta,
                      const void* Bc, const void* Cc, const float* Dskip,
                      const float* h0, const float* hck,
                      float* du, float* ddelta, float* drho, float* dtheta, float* dB, float* dC,
                      float* dD, float* dh0, const float* z, float* dz, float* workspace,
                      int B, int D, int N, int L, int ck, int in_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * Real (Mamba S6) selective scan:
 *     dl = delta (+ delta_bias[d]) (softplus if delta_softplus)
 *     h_l[b,d,n] = exp(dl_l[b,d]*A[d,n]) * h_{l-1} + dl_l[b,d] * B_l[b,n] * u_l[b,d]
 *     y_l[b,d]   = sum_n C_l[b,n] h_l[b,d,n] + Dskip[d] u_l[b,d]              (* silu(z_l))
 * Replaces the third-party selective_scan_fn called at
 * ai-modules/wavesAI/model/aussm.py:791-802 (same argument meaning: u, delta, A, B, C, D, z,
 * delta_bias, delta_softplus) and the real-state loop of extension-cpp/extension_cpp/ops.py:349-356.
 * ddelta is the gradient w.r.t. the RAW delta input (before bias and softplus).
 * ------------------------------------------------------------------------------------- */
int aussm_real_fwd(const void* u, const void* delta, const float* A,
                   const void* Bm, const void* Cm, const float* Dskip, const float* z,
                   const float* delta_bias, int delta_softplus,
                   const float* h0, float* y, float* hL, float* hck, float* workspace,
                   int B, int D, int N, int L, int ck, int in_dtype, void* stream);

int aussm_real_bwd(const float* dy, const float* dhL,
                   const void* u, const void* delta, const float* A,
                   const void* Bm, const void* Cm, const float* Dskip,
                   const float* delta_bias, int delta_softplus,
                   const float* h0, const float* hck,
                   float* du, float* ddelta, float* dA, float* dB, float* dC,
                   float* dD, float* dh0, const float* z, float* dz, float* workspace,
                   int B, int D, int N, int L, int ck, int in_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * Depthwise causal convolution along the sequence, channels-last (the step both blocks apply to
 * the scan's input):
 *     y[b,l,d] = bias[d] + sum_{k<K} w[d,k] * x[b, l-(K-1)+k, d]          (x = 0 before l = 0)
 * Replaces `self.conv1d(x)[:, :, :l]` of ai-modules/wavesAI/model/aussm.py:762 (MambaBlock) and
 * :863 (SSMauBlock) - nn.Conv1d(D, D, K, groups=D, padding=K-1), weight (D, 1, K) - without the
 * two transposes around it: element (b,l,d) of x is x[b*xs_b + l*xs_l + d] (so a column slice of
 * a wider (b, l, 2D) tensor can be passed as it is), y, dy and dx are contiguous (B, L, D).
 * K <= 8.  dw (D, K) and dbias (D, may be NULL) are ACCUMULATED into: zero them for a plain gradient.
 * ------------------------------------------------------------------------------------- */
int aussm_causal_conv1d_fwd(const float* x, const float* w, const float* bias, float* y,
                            int B, int L, int D, int K, long long xs_b, long long xs_l, void* stream);

int aussm_causal_conv1d_bwd(const float* dy, const float* x, const float* w,
                            float* dx, float* dw, float* dbias,
                            int B, int L, int D, int K, long long xs_b, long long xs_l, void* stream);

/* y[b, c, r] = x[b, r, c]: the layout change between the blocks' channels-last activations
 * (b, l, d) and the scans' (b, d, l) tensors - `rearrange(x, 'b l d -> b d l')` and its inverse,
 * ai-modules/wavesAI/model/aussm.py:760-803 and :861-900.  Element (b, r, c) of x is
 * x[b*xs_b + r*xs_r + c] (a column slice of a wider tensor is fine), y is contiguous (B, C, R).
 * B <= 65535. */
int aussm_swap_last2(const float* x, float* y, int B, int R, int C,
                     long long xs_b, long long xs_r, void* stream);

/* The same layout change with the elementwise step the blocks apply on the way done in the same pass:
 * act 1 = silu (`x = F.silu(x)` on the convolution output that feeds the S6 scan, aussm.py:787),
 * act 2 = softplus with threshold 20 (`dt = F.softplus(dt + self.dt_proj.bias)`, aussm.py:878-880).
 *   deriv == 0:  y[b, c, r] = f(x[b, r, c] + bias[c])                 bias (C) may be NULL
 *   deriv != 0:  y[b, c, r] = x[b, r, c] * f'(pre[b, c, r] + bias[r])  bias (R) may be NULL
 * the second form is the gradient: x is the gradient w.r.t. the first form's output (in that output's
 * layout), pre the first form's input (element (b, c, r) at pre[b*ps_b + c*ps_r + r]), y the gradient
 * w.r.t. that input.  The gradient of bias is the sum of y over b and c (left to the caller). */
int aussm_swap_last2_act(const float* x, const float* bias, const float* pre, float* y, int B, int R, int C,
                         long long xs_b, long long xs_r, long long ps_b, long long ps_r, int act, int deriv,
                         void* stream);

/* The scans' output gate and its gradients as one pass each over contiguous tensors of n floats (16-byte
 * aligned ones take the wide path; `y = y * F.silu(z)`, extension-cpp/extension_cpp/ops.py:226, and what autograd derives from it):
 *   aussm_gate_fwd:  y = y_pre silu(z)
 *   aussm_gate_bwd:  dy_pre = dy silu(z),  dz = dy y_pre silu'(z)
 * The complex and real scans and the fused operator apply and differentiate their gate inside their kernels;
 * the unitary core scan's backward kernels take the gradient of the ungated output, and a gated call with
 * gradients runs these two around them (in place is allowed: y may be y_pre, dy_pre may be dy). */
int aussm_gate_fwd(const float* y_pre, const float* z, float* y, size_t n, void* stream);
int aussm_gate_bwd(const float* dy, const float* y_pre, const float* z, float* dy_pre, float* dz, size_t n, void* stream);

/* ---------------------------------------------------------------------------------------
 * The reference's custom operator itself, as two calls: what
 *   torch.ops.extension_cpp.ssm_adaptive_unitary           (12 tensors -> y, next_hid_real, next_hid_imag)
 *   torch.ops.extension_cpp.ssm_adaptive_backward_unitary  (3 + 12 tensors -> 12 gradients)
 * bind to - extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_forward.cu:184-286 and
 * ssm_adaptive_unitary_backward.cu:493-617, Python side extension-cpp/extension_cpp/ops.py:97-154.
 * Arguments in the operator's order; all tensors fp32 and contiguous:
 *   u, dt, z (b, d, L);  x (d, n, d);  x_bias (d, n);  B_r, B_theta, C_r, C_theta (n);  D (d);
 *   h_re, h_im (b, d, n) the state before the first step;  y (b, d, L);  nh_* (b, d, n).
 *     theta_l[b,i,j] = sum_r x[i,j,r] u_l[b,r] + x_bias[i,j]
 *     h_l[b,i,j]     = exp(i theta_l) h_{l-1}[b,i,j] + B_r[j] e^{i B_theta[j]} dt_l[b,i] silu(u_l[b,i])
 *     y_l[b,i]       = silu(z_l[b,i]) ( sum_j Re(C_r[j] e^{i C_theta[j]} h_l[b,i,j]) + D[i] silu(u_l[b,i]) )
 * The phase tensor theta (b, d, n, L) is never stored: the forward call forms it tile by tile on
 * the matrix cores inside the scan kernel.  The backward call recomputes from the twelve inputs,
 * as the reference does, and needs the phase adjoints of a few batch elements at a time (for the
 * product that sums over all channels); they live in the workspace, at most about 50 MiB.
 * Limits: n <= 64, d <= 512 (AUSSM_E_SHAPE beyond).  L is arbitrary (the reference needs a
 * multiple of 16 and pads).  `workspace` holds aussm_ssm_adaptive_unitary_workspace_floats(...)
 * floats, 16-byte aligned; nothing in it has to be initialised, nothing in it is kept between calls.
 * grad_nh_re / grad_nh_im may be NULL (zero).  Every gradient buffer is fully written.
 * nh_re / nh_im of the backward call: the state after the last step as the forward call returned it,
 * or NULL - then the backward call recomputes it with one forward sweep (the reference's backward
 * operator gets the twelve inputs only), which costs about one forward call more.
 * ------------------------------------------------------------------------------------- */
size_t aussm_ssm_adaptive_unitary_workspace_floats(int b, int d, int n, int L, int backward);

int aussm_ssm_adaptive_unitary_fwd(const float* u, const float* dt, const float* x, const float* x_bias,
                                   const float* B_r, const float* B_theta, const float* C_r, const float* C_theta,
                                   const float* D, const float* z, const float* h_re, const float* h_im,
                                   float* y, float* nh_re, float* nh_im, float* workspace,
                                   int b, int d, int n, int L, void* stream);

int aussm_ssm_adaptive_unitary_bwd(const float* grad_y, const float* grad_nh_re, const float* grad_nh_im,
                                   const float* u, const float* dt, const float* x, const float* x_bias,
                                   const float* B_r, const float* B_theta, const float* C_r, const float* C_theta,
                                   const float* D, const float* z, const float* h_re, const float* h_im,
                                   const float* nh_re, const float* nh_im,
                                   float* du, float* ddt, float* dx, float* dx_bias, float* dB_r, float* dB_theta,
                                   float* dC_r, float* dC_theta, float* dD, float* dz, float* dh_re, float* dh_im,
                                   float* workspace, int b, int d, int n, int L, void* stream);

/* ---------------------------------------------------------------------------------------
 * Measurement aid: what the memory system delivers for the scan kernels' access pattern, with
 * next to no arithmetic: o1 = a + b * c and o2 = 2 * o1 over [rows, L] float tensors (three
 * tensors read, two written when write != 0; read only, nothing but o1[0] possibly written,
 * when write == 0).  pattern 0: a plain streaming elementwise kernel; pattern 1: the matrix-core
 * scans' pattern (a workgroup owns 64 rows and walks them in 32-step chunks; one load or store
 * instruction of a wavefront covers 16 rows x 64 bytes; loads two chunks ahead).  rows and L are
 * multiples of 64.  `bench.py --hbm-probe` times both at the headline shape; the rates bound what
 * a scan kernel with this layout of work can reach.  No counterpart in the reference.
 * ------------------------------------------------------------------------------------- */
int aussm_hbm_probe(const float* a, const float* b, const float* c, float* o1, float* o2, int rows, int L,
                    int pattern, int write, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AUSSM_HIP_H */
