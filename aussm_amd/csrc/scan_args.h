// Argument blocks of the kernels and the constants the host side shares with them.  Plain data
// only: every translation unit of the library includes this header, the kernel headers are
// included by the one unit that instantiates their kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aussm {

constexpr int CH = 64;        // channels per workgroup == lanes per wavefront
constexpr int XT = 32;        // timesteps per chunk of the matrix-core kernels
constexpr int XN = 16;        // state rows of the matrix tiles (N is zero-padded up to it)

enum { VAR_UNITARY = 0, VAR_COMPLEX = 1, VAR_REAL = 2 };

// The optional auxiliary buffer of the unitary scan holds B*D*L floats followed by AUX_PAD floats;
// the first of those is the call's aux_tag() when a forward kernel has filled the buffer, anything
// else if not: a backward call consumes the contents only when its own arguments give the same tag.
// Words AUX_IMG_FP .. + 7 of the pad describe the operand images behind it (ImgStamp below): written
// by the forward kernel that ran on freshly prepared images, cleared by every other forward call.
constexpr uint32_t AUX_TAG = 0x4f484950u;
constexpr uint32_t IMG_TAG = 0x494d4147u;
constexpr int AUX_PAD = 64;
constexpr int AUX_IMG_FP = 8;

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// What the per-(b,d,l) part of an auxiliary buffer was computed from: the tensors (addresses), the shape
// and the input type.  Never zero (zero is what an invalidated buffer holds).
inline uint32_t aux_tag(const void* u, const void* delta, const void* theta, const void* Bm, const void* Cm,
                        int B, int D, int N, int L, int in_dtype) {
  uint64_t h = AUX_TAG;
  const uint64_t v[] = {(uint64_t)(uintptr_t)u, (uint64_t)(uintptr_t)delta, (uint64_t)(uintptr_t)theta,
                        (uint64_t)(uintptr_t)Bm, (uint64_t)(uintptr_t)Cm, (uint64_t)B, (uint64_t)D, (uint64_t)N,
                        (uint64_t)L, (uint64_t)in_dtype};
  for (uint64_t x : v) h = (h ^ x) * 0x9e3779b97f4a7c15ull + (h >> 29);
  return (uint32_t)(h >> 32) | 1u;
}

struct FwdArgs {
  const void* u;            // [B,D,L]  Tin
  const void* delta;        // [B,D,L]  Tin
  const float* theta;       // [B,D,L]  (unitary, complex)
  const float* rho;         // [B,D,L]  (complex)
  const float* A;           // [D,N]    (real)
  const void* Bm;           // [B,N,L(,2)] Tin
  const void* Cm;           // [B,N,L(,2)] Tin
  const float* Dskip;       // [D] or null
  const float* z;           // [B,D,L] or null
  const float* delta_bias;  // [D] or null (real)
  const float* h0;          // [B,D,N,C] or null
  float* y;                 // [B,D,L] or null
  float* hL;                // [B,D,N,C] or null
  float* hck;               // [B,nck,N,C,D] or null
  float* aux;               // unitary, optional: Im(P_t S_t) [B,D,L] followed by a validity tag
  float* ptot;              // vector-ALU kernels, optional: [B,D,2] product of the a_l of the call's L steps
                            // (complex: re, im; real: the sum of delta after bias / softplus, 0)
  int B, D, N, L, ck, nck, ncg, delta_softplus;
  int ld, ns;                // row stride of the [.., L] tensors and segments per sequence: B then counts
                             // (batch, segment) pairs and L is the segment length.  The vector-ALU kernels take a
                             // shorter last segment (ld not a multiple of L) and keep nck = checkpoints of a whole
                             // sequence; h0 / hL / ptot are indexed by the pair
  int hs, ho;                // matrix-core kernels: h0 of pair b is entry b * hs + ho of the state array
  int urep;                  // generic kernels: u and delta are [B / urep, D, L], shared by urep consecutive batch elements
  uint32_t auxtag;           // what a kernel that fills aux writes behind it (aux_tag of the call)
};

struct UniBwdArgs {
  const float* dy;      // [B,D,L]
  const float* dhL;     // [B,D,N,2] or null
  const void* u;        // [B,D,L] Tin
  const void* delta;    // [B,D,L] Tin
  const float* theta;   // [B,D,L]
  const void* Bm;       // [B,N,L,2] Tin
  const void* Cm;       // [B,N,L,2] Tin
  const float* Dskip;   // [D] or null
  const float* hck;     // [B,nck,N,2,D]
  const float* aux;     // optional: what the forward call left in its aux buffer
  float *du, *ddelta, *dtheta;   // [B,D,L]
  float *dB, *dC;       // [B,N,L,2]  accumulated into with atomics (caller zero-fills)
  float* dD;            // [D] or null, accumulated into
  float* dh0;           // [B,D,N,2] or null
  int B, D, N, L, ck, nck, ncg;
  int ld, ns;           // matrix-core kernel: row stride of the [.., L] tensors, segments per sequence
  int hs, ho;           // ... and dhL of (batch, segment) pair b is entry b * hs + ho of the adjoint array
  int urep;             // generic kernel: u and delta are [B / urep, D, L], shared by urep consecutive batch elements
  int tag_mode;         // matrix-core kernels: 0 use the auxiliary buffer if its tag is valid; 1 leave at once
                        // unless it is; 2 leave at once if it is
  uint32_t auxtag;      // the tag a forward call of the same arguments leaves behind aux (aux_tag)
};

struct RecBwdArgs {
  const float* dy;          // [B,D,L]
  const float* dhL;         // [B,D,N,C] or null
  const void* u;            // [B,D,L] Tin
  const void* delta;        // [B,D,L] Tin
  const float* theta;       // [B,D,L] (complex)
  const float* rho;         // [B,D,L] (complex)
  const float* A;           // [D,N]   (real)
  const void* Bm;           // [B,N,L(,2)] Tin
  const void* Cm;           // [B,N,L(,2)] Tin
  const float* Dskip;       // [D] or null
  const float* delta_bias;  // [D] or null (real)
  const float* h0;          // [B,D,N,C] or null
  const float* hck;         // [B,nck,N,C,D], ck == 16
  float *du, *ddelta;       // [B,D,L]
  float *dtheta, *drho;     // [B,D,L] (complex)
  float* dA;                // [D,N] (real), accumulated into
  float *dB, *dC;           // [B,N,L(,2)], accumulated into
  float* dD;                // [D] or null, accumulated into
  float* dh0;               // [B,D,N,C] or null
  const float* z;           // [B,D,L] or null: the output was gated, y = y_pre silu(z); dy is the gradient of y
  float* dz;                // [B,D,L] (with z)
  int B, D, N, L, nck, ncg, delta_softplus;
  // Split along the sequence: ld = row stride of the [.., L] tensors (the whole sequence), ns segments per
  // sequence, B counts (batch, segment) pairs, L is the segment length (a multiple of 16; the last segment may
  // be shorter), nck the checkpoints of a whole sequence; dhL / dh0 are indexed by the pair, h0 by the batch element.
  int ld, ns;
  // A launch handles the states nbase .. nbase + 15 (a workgroup's four wavefronts of up to four states);
  // larger N takes one launch per block of 16 states.  accum: a later block - the sums over the states
  // (du, ddelta, dtheta, drho) are added to what the earlier blocks wrote, and the terms that do not
  // depend on the state (the D skip, dD) are left out.
  int nbase, accum;
};

// Adjoint of the state entering a segment, from a zero adjoint at its end (complex and real scans)
struct AdjSegArgs {
  const float* dy;          // [B,D,ld]
  const float* z;           // [B,D,ld] or null
  const void* delta;        // [B,D,ld] Tin (real)
  const float* theta;       // [B,D,ld] (complex)
  const float* rho;         // [B,D,ld] (complex)
  const float* A;           // [D,N] (real)
  const void* Cm;           // [B,N,ld(,2)] Tin
  const float* delta_bias;  // [D] or null (real)
  float* out;               // [B*ns,D,N,C]
  float* ptot;              // [B*ns,D,2]  as FwdArgs::ptot
  int D, N, L, ld, ns, ncg, delta_softplus;   // L: segment length (the last one may be shorter)
};

struct SegArgs {
  const void* x1;       // forward: delta (Tin), adjoint: dy (float)   [B, D, ld]
  const void* x2;       // forward: u (Tin), adjoint: unused           [B, D, ld]
  const float* theta;   //                                    [B, D, ld]
  const void* M;        // forward: B_t, adjoint: C_t (Tin)            [B, N, ld, 2]
  float* out;           // Z or Y                             [B * ns, D, N, 2]
  float* ptot;          // rotation of the segment            [B * ns, D, 2]
  int D, N, L, ld, ns, ncg;   // L: segment length
};

// Prepared operands ("images") of the matrix-core kernels, in 16-byte records per (batch, chunk)
constexpr int PX_NP = 3;                                    // bf16 pieces held by the images
constexpr int PXF_A = 2 * PX_NP * XN * 4;                   // forward: bt_r, bt_i          (phase A)
constexpr int PXF_B = 3 * PX_NP * XT * 4;                   //          cs_r, g_re, g_im    (phase B)
constexpr int PXF_REC = PXF_A + PXF_B;                      // 1536 records = 24 KiB
constexpr int PXB_A = 4 * PX_NP * XN * 4;                   // backward: bt_r, bt_i, ct_r, ct_i
constexpr int PXB_B = 3 * PX_NP * XT * 4;                   //           bs, g_r, g_i
constexpr int PXB_REC = PXB_A + PXB_B;                      // 1920 records = 30 KiB

// What a set of images was made from.  A backward call recomputes its images unless the stamp in
// the auxiliary buffer equals the stamp of its own arguments: same tensors (addresses), same
// shape and input type, backward images present.
struct ImgStamp { uint32_t w[8]; };
inline ImgStamp img_stamp(const void* Bm, const void* Cm, int B, int N, int L, int in_dtype, bool with_bwd) {
  const uint64_t b = (uint64_t)(uintptr_t)Bm, c = (uint64_t)(uintptr_t)Cm;
  return ImgStamp{{IMG_TAG, (uint32_t)B, (uint32_t)N, (uint32_t)L, (uint32_t)in_dtype | (with_bwd ? 0x100u : 0u),
                   (uint32_t)b ^ (uint32_t)(b >> 32) * 0x9e3779b1u, (uint32_t)c ^ (uint32_t)(c >> 32) * 0x9e3779b1u,
                   (uint32_t)(b >> 4) + (uint32_t)(c >> 4) * 31u}};
}

struct PrepArgs {
  const void* Bm;       // [B, N, ld, 2] Tin
  const void* Cm;
  u4* fimg;             // [B, nch, PXF_REC] or null
  u4* bimg;             // [B, nch, PXB_REC] or null
  int N, ld, nch;       // nch = ceil(ld / 32) chunks per batch element
  const uint32_t* have; // or null: the launch has nothing to do if these eight words equal `want`
  ImgStamp want;
};

// Where a forward kernel that ran on freshly prepared images records what they were made from; clear: the
// buffer's fill tag, set to zero by a call that is given the buffer and does not fill it (or null)
struct ImgNote { uint32_t* dst; ImgStamp stamp; float* clear; };

constexpr int CONV_MAX_K = 8;
constexpr int CONV_ROWS = 128;   // (b, l) rows per workgroup of the weight-gradient kernel
constexpr int CONV_RUN = 8;      // steps per thread of the kernels for filter length 4

struct ConvArgs {
  const float* x;      // element (b, l, d) at x[b * xs_b + l * xs_l + d]
  const float* w;      // [D, K]
  const float* bias;   // [D] or null
  const float* dy;     // [B, L, D] contiguous (backward)
  float* y;            // [B, L, D] contiguous (forward)
  float* dx;           // [B, L, D] contiguous (backward)
  float* dw;           // [D, K], accumulated into
  float* dbias;        // [D] or null, accumulated into
  long long xs_b, xs_l;
  int B, L, D, K;
};

struct SwapArgs {
  const float* x;      // element (b, r, c) at x[b * xs_b + r * xs_r + c]
  float* y;            // [B, C, R] contiguous
  long long xs_b, xs_r;
  int R, C;
  // optional activation fused into the swap (act: 0 none, 1 silu, 2 softplus with torch's threshold 20)
  //   forward (deriv 0):  y[b, c, r] = f(x[b, r, c] + bias[c])
  //   gradient (deriv 1): y[b, c, r] = x[b, r, c] * f'(pre[b, c, r] + bias[r])   (x is the incoming gradient
  //                       in the forward output's layout, pre the forward input, y its gradient)
  const float* bias;   // per channel, or null
  const float* pre;    // deriv: element (b, c, r) at pre[b * ps_b + c * ps_r + r]
  long long ps_b, ps_r;
  int act, deriv;
};

}  // namespace aussm
