// C ABI of libaussm_hip.so: argument checks, kernel selection and launches.
// Declarations and tensor layouts: include/aussm_hip.h.
#include "../../include/aussm_hip.h"

#include <hip/hip_runtime.h>
#include <atomic>

#include "launch.h"
#include "scan_args.h"

using namespace aussm;

namespace {

// Process-wide options (aussm_set_option): kernel selection for comparisons and tuning.  They are
// plain atomics read once per call; -1 means "let the launcher decide".
std::atomic<int> g_opt[AUSSM_OPT_COUNT] = {{-1}, {-1}, {-1}, {-1}, {-1}, {-1}};
static_assert(AUSSM_OPT_COUNT == 6, "one initialiser per option");
inline int opt(int key) { return g_opt[key].load(std::memory_order_relaxed); }

// ---- configuration of the vector-ALU kernels --------------------------------------------------
// The scalar loads of B_t/C_t are issued one "turn" ahead; with two or more wavefronts per SIMD
// the turn of another wavefront doubles that distance, so for a given N the configuration with
// MORE wavefronts (smaller NW) is preferred as long as the launch still fits one workgroup.
inline Cfg pick_cfg(int N, int max_waves) {
  // test/tuning override (must be one of the compiled configurations)
  {
    const Cfg c{opt(AUSSM_OPT_GENERIC_NW), opt(AUSSM_OPT_GENERIC_NT)};
    if (c.nw > 0 && c.nt > 0 && c.nw * (c.nt / 64) >= N) return c;
  }
  const Cfg table[] = {{1, 256}, {1, 512}, {2, 512}, {4, 512}, {8, 512},
                       {2, 256}, {4, 256}, {8, 256}, {16, 256}};
  for (const Cfg& c : table)
    if (c.nw * (c.nt / 64) >= N && c.nt / 64 <= max_waves) return c;
  return Cfg{16, 256};
}

inline int check_common(int B, int D, int N, int L, int ck, int in_dtype) {
  if (B < 1 || D < 1 || N < 1 || L < 1) return AUSSM_E_SHAPE;
  if (N > AUSSM_MAX_STATE) return AUSSM_E_SHAPE;
  if ((long long)B * ((D + CH - 1) / CH) > 0x7fffffffLL) return AUSSM_E_SHAPE;
  if (ck != AUSSM_TILE / 2 && (ck < AUSSM_TILE || ck % AUSSM_TILE != 0)) return AUSSM_E_CK;
  if (in_dtype != AUSSM_F32 && in_dtype != AUSSM_BF16) return AUSSM_E_DTYPE;
  return AUSSM_OK;
}

// The recomputing backward kernels (complex, real) keep a tile of states in registers: four
// wavefronts of at most four states each.
constexpr int REC_CK = AUSSM_TILE / 2;

inline bool misaligned(const void* p, size_t a) { return p && (reinterpret_cast<uintptr_t>(p) % a) != 0; }

// The matrix-core kernels cover the common unitary case (fp32 or bf16 inputs, 6 <= N <= 16, L a multiple of 4,
// 16-byte aligned tensors, checkpoint interval a multiple of 32); everything else takes the
// vector-ALU kernels.  aussm_set_option(AUSSM_OPT_UNITARY_FWD, m) selects the forward kernel for
// comparisons: 0 vector ALU, 2 / 3 bf16 matrix instructions on two- / three-piece operands built
// inside the scan kernel, 6 three-piece operands prepared by a pre-pass, two wavefronts per SIMD
// (the default when the call brings the workspace for them, i.e. an auxiliary buffer).
// AUSSM_OPT_UNITARY_BWD: 0 vector ALU, 2 two pieces everywhere, 3 three pieces along the sequence
// and two in the sums over the channel (dB, dC), 5 three pieces everywhere, 6 prepared operands.
//
// The matrix-core kernels cost the same for every N <= 16 while the vector-ALU ones scale with N:
// measured, the crossover is between N = 4 (vector ALU 15 % faster) and N = 8 (matrix 30 % faster).
constexpr int MATRIX_MIN_STATE = 6;
constexpr int DEFAULT_FWD_MODE = 6, DEFAULT_BWD_MODE = 6;   // (6 falls back to 3 where the call brings no workspace)
inline int kernel_mode(int key, int dflt, int N) {
  const int e = opt(key);
  if (e >= 0) return e;                        // an explicit choice is honoured for every N <= 16
  return N >= MATRIX_MIN_STATE ? dflt : 0;
}
// Splitting the sequence (scan_seg_xdl.h): with few (batch, channel group) pairs the launch would
// leave most of the chip idle, so the sequence is cut into ns segments of whole checkpoint blocks
// until about one workgroup per compute unit exists.  Only the matrix-core kernels take part,
// and only the *_aux entry points (the segment states live behind the auxiliary buffer).
// aussm_set_option(AUSSM_OPT_SPLIT_CAP, c): 0 or 1 switches it off, a power of two caps ns.
constexpr int SPLIT_MIN_WGS = 129;     // launches of at least this many workgroups are left alone
constexpr int SPLIT_TARGET_WGS = 256;
constexpr int SPLIT_MAX = 32;
constexpr int SPLIT_MIN_LEN = 128;
inline bool matrix_shape(int N, int L, int ck) { return N <= XN && L % 4 == 0 && ck >= XT && ck % XT == 0; }
inline int seg_capacity(int B, int D, int N, int L, int ck) {
  if (N < MATRIX_MIN_STATE || !matrix_shape(N, L, ck) || L % ck != 0) return 1;
  const long long wgs = (long long)B * ((D + CH - 1) / CH);
  if (wgs >= SPLIT_MIN_WGS) return 1;
  const int nblk = L / ck, target = (int)(SPLIT_TARGET_WGS / wgs);
  int ns = 1;
  while (ns * 2 <= target && ns * 2 <= SPLIT_MAX && nblk % (ns * 2) == 0 && L / (ns * 2) >= SPLIT_MIN_LEN) ns *= 2;
  return ns;
}
inline int seg_count(int B, int D, int N, int L, int ck) {
  int ns = seg_capacity(B, D, N, L, ck);
  const int cap = opt(AUSSM_OPT_SPLIT_CAP);
  if (cap >= 0)
    while (ns > 1 && ns > cap) ns /= 2;
  return ns;
}
// The segment states are computed on finer segments than the scan proper uses (the kernel that
// forms them is light: several workgroups per compute unit hide its latencies); the scan takes
// every SPLIT_FINE-th of them.
inline int seg_fine(int L, int ns) {
  const int Ls = L / ns;
  for (int r = 4; r > 1; r /= 2)
    if (Ls % (r * XT) == 0 && Ls / r >= SPLIT_MIN_LEN) return r;
  return 1;
}
inline size_t round64(size_t n) { return (n + 63) & ~(size_t)63; }
inline size_t seg_floats(int B, int D, int N, int L, int ns) {
  return ns > 1 ? round64((size_t)B * ns * seg_fine(L, ns) * D * (2 * N + 2)) : 0;
}
// The complex and the real scan split the same way (scan_seg_generic.h) when the call brings a workspace:
// ns segments of ls steps (whole tiles and checkpoint blocks), the last one possibly shorter.
constexpr int GSPLIT_MAX = 64;
struct GSplit { int ns, ls; };
inline GSplit generic_split(int B, int D, int L, int ck, bool use_cap) {
  const long long wgs = (long long)B * ((D + CH - 1) / CH);
  const int cap = use_cap ? opt(AUSSM_OPT_SPLIT_CAP) : -1;
  if (wgs >= SPLIT_MIN_WGS || cap == 0 || cap == 1) return GSplit{1, L};
  int want = (int)((SPLIT_TARGET_WGS + wgs - 1) / wgs);
  if (want > GSPLIT_MAX) want = GSPLIT_MAX;
  if (cap > 1 && want > cap) want = cap;
  const int unit = ck > XT ? ck : XT;
  int ls = ((L + want - 1) / want + unit - 1) / unit * unit;
  if (ls < SPLIT_MIN_LEN) ls = (SPLIT_MIN_LEN + unit - 1) / unit * unit;
  const int ns = (L + ls - 1) / ls;
  return ns > 1 ? GSplit{ns, ls} : GSplit{1, L};
}
inline size_t generic_split_floats(int variant, int B, int D, int N, int L, int ck) {
  const GSplit sp = generic_split(B, D, L, ck, false);
  const int C = variant == VAR_REAL ? 1 : 2;
  return sp.ns > 1 ? round64((size_t)B * sp.ns * D * (N * C + 2)) : 0;
}
// ... and their kernels take B_t / C_t as float: bf16 rows are converted once per call, behind the segments
inline size_t generic_bc_floats(int variant, int B, int N, int L, int in_dtype) {
  return in_dtype == AUSSM_BF16 ? round64((size_t)B * N * L * (variant == VAR_REAL ? 1 : 2)) : 0;
}
struct BcF32 { const void* Bm; const void* Cm; int in_dtype; int err; };
inline BcF32 generic_bc(int variant, const void* Bm, const void* Cm, float* ws, int B, int D, int N, int L, int ck,
                        int in_dtype, hipStream_t s) {
  if (in_dtype != AUSSM_BF16) return BcF32{Bm, Cm, 0, 0};
  const size_t n = generic_bc_floats(variant, B, N, L, in_dtype);
  float* fB = ws + generic_split_floats(variant, B, D, N, L, ck);
  const int err = run_bc_to_f32(Bm, Cm, fB, fB + n, (size_t)B * N * L * (variant == VAR_REAL ? 1 : 2), s);
  return BcF32{fB, fB + n, 2, err};
}

// Workspace of the prepared operands: per (batch element, chunk) one backward image and, behind
// all of those, one forward image.  The forward call of a training step writes both (one pre-pass);
// a backward call whose auxiliary buffer does not hold the images of its own tensors writes its own.
// The size does not depend on the option table: a buffer sized under one set of options fits every other.
inline size_t img_chunks(int B, int L) { return (size_t)B * ((L + XT - 1) / XT); }
inline size_t img_floats(int B, int N, int L, int ck) {
  if (!matrix_shape(N, L, ck)) return 0;
  return img_chunks(B, L) * (PXB_REC + PXF_REC) * 4;
}
// Layout of the auxiliary buffer: [B*D*L floats Im(P S)] [AUX_PAD] [segment states] [backward images] [forward images].
// A shape that only the vector-ALU kernels serve (more than 16 states, a length that is not a multiple of 4, ...)
// has no Im(P S) part and no images.  The segment area holds what either way of splitting a call along L
// needs (the matrix-core kernels' fine segments or the vector-ALU kernels' segments), so a call of a shape
// that could run on the matrix cores but does not (shared inputs, misaligned tensors, an option) can still split.
inline size_t aux_im_floats(int B, int D, int N, int L, int ck) { return matrix_shape(N, L, ck) ? (size_t)B * D * L : 0; }
inline size_t aux_seg_floats(int B, int D, int N, int L, int ck) {
  const size_t m = seg_floats(B, D, N, L, seg_capacity(B, D, N, L, ck)), g = generic_split_floats(VAR_COMPLEX, B, D, N, L, ck);
  return m > g ? m : g;
}
struct AuxLayout { float* seg; u4* img; u4* fimg; uint32_t* stamp; float* pad; float* gseg; };
inline AuxLayout aux_layout(float* aux, int B, int D, int N, int L, int ck) {
  if (!aux) return AuxLayout{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  float* pad = aux + aux_im_floats(B, D, N, L, ck);
  float* seg = pad + AUX_PAD;
  u4* img = reinterpret_cast<u4*>(seg + aux_seg_floats(B, D, N, L, ck));
  if (!img_floats(B, N, L, ck)) return AuxLayout{seg, nullptr, nullptr, nullptr, pad, seg};
  return AuxLayout{seg, img, img + img_chunks(B, L) * PXB_REC, reinterpret_cast<uint32_t*>(pad) + AUX_IMG_FP, pad, seg};
}

// Kernel family of a call whose tensors are 16-byte aligned: 0 vector ALU, 2 / 3 / 5 matrix-core kernels
// that prepare their operands themselves, 6 prepared-operand kernels.
inline int fwd_mode_for(int N, int L, int ck, int in_dtype, int urep, bool have_img) {
  int mode = kernel_mode(AUSSM_OPT_UNITARY_FWD, DEFAULT_FWD_MODE, N);
  if (mode <= 0 || urep != 1 || !matrix_shape(N, L, ck)) return 0;
  if (mode == 6 && !have_img) mode = 3;
  if (in_dtype != AUSSM_F32 && mode != 6) mode = 3;       // bf16 inputs: three-piece kernels only
  return mode;
}
inline int bwd_mode_for(int B, int D, int N, int L, int ck, int urep, bool have_img) {
  int mode = kernel_mode(AUSSM_OPT_UNITARY_BWD, DEFAULT_BWD_MODE, N);   // matrix-core kernels for the common case
  if (mode <= 0 || urep != 1 || !matrix_shape(N, L, ck)) return 0;
  // (the prepared-operand kernel addresses its tensors with 32-bit byte offsets)
  if (mode == 6 && (!have_img || (unsigned long long)B * D * L * 4 >= (1ull << 32) ||
                    (unsigned long long)B * N * L * 8 >= (1ull << 32)))
    mode = 3;
  return mode;
}
inline int mfma_fwd_mode(const FwdArgs& a, int in_dtype, bool have_img) {
  const int mode = fwd_mode_for(a.N, a.L, a.ck, in_dtype, a.urep, have_img);
  if (misaligned(a.u, 16) || misaligned(a.delta, 16) || misaligned(a.theta, 16) || misaligned(a.z, 16) ||
      misaligned(a.y, 16) || misaligned(a.Bm, 16) || misaligned(a.Cm, 16))
    return 0;
  return mode;
}

// ws: workspace of the call (segment states for a launch that is split along L, images of the
// prepared operands); either part may be null.
int launch_unitary_fwd(FwdArgs a, int in_dtype, hipStream_t s, AuxLayout ws) {
  const int mode = mfma_fwd_mode(a, in_dtype, ws.img != nullptr);
  // Im(P S) is only worth writing when a backward call can follow (it needs the checkpoints too);
  // a call that does not fill the buffer marks it as not filled, and a call that does not prepare
  // images clears the note about the ones behind the buffer
  const bool fill = a.aux && a.hck && mode >= 2;
  // (the prepared-operand kernel clears the fill tag itself, at its end: one launch less for a forward-only call)
  const bool clear_in_kernel = a.aux && !fill && mode == 6;
  if (a.aux)
    if (int e = run_aux_invalidate(ws.pad, !fill && !clear_in_kernel, mode != 6 && ws.stamp, s)) return e;
  if (!fill) a.aux = nullptr;
  if (!mode) {
    // vector-ALU kernel; with a segment area and few (batch, channel group) pairs, split along the sequence
    const Cfg cfg = pick_cfg(a.N, 8);
    const GSplit sp = ws.gseg ? generic_split(a.B, a.D, a.L, a.ck, true) : GSplit{1, a.L};
    if (sp.ns > 1) {
      const int B = a.B;
      float* seg = ws.gseg;
      float* ptot = seg + (size_t)B * sp.ns * a.D * a.N * 2;
      // 1. end state of every segment from a zero state (no outputs) and the product of its a_l
      FwdArgs z = a;
      z.B = B * sp.ns; z.L = sp.ls; z.ns = sp.ns;
      z.y = nullptr; z.z = nullptr; z.Dskip = nullptr; z.h0 = nullptr; z.hL = seg; z.hck = nullptr; z.ptot = ptot;
      if (int e = run_core_fwd(VAR_UNITARY, z, in_dtype, cfg, s)) return e;
      // 2. the state that enters every segment; the state after the last one is the call's hL
      if (int e = run_seg_carry_fwd(seg, ptot, a.h0, a.hL, B, a.D, a.N, sp.ns, s)) return e;
      // 3. the scan proper over (batch, segment) pairs
      a.B = B * sp.ns; a.L = sp.ls; a.ns = sp.ns; a.h0 = seg; a.hL = nullptr;
    }
    return run_core_fwd(VAR_UNITARY, a, in_dtype, cfg, s);
  }
  const int B = a.B, L = a.L;
  if ((mode == 2 || mode == 3 || mode == 6) && ws.seg) {
    const int ns = seg_count(B, a.D, a.N, L, a.ck);
    if (ns > 1) {
      // 1. end state of every segment from a zero start and its rotation; 2. chain them;
      // 3. the scan proper over (batch, segment) pairs, each from its true incoming state
      const int Ls = L / ns, r = seg_fine(L, ns), nf = ns * r;
      float* seg = ws.seg;
      float* ptot = seg + (size_t)B * nf * a.D * a.N * 2;
      SegArgs sa{a.delta, a.u, a.theta, a.Bm, seg, ptot, a.D, a.N, Ls / r, L, nf, a.ncg};
      if (int e = run_seg_state(false, sa, in_dtype, (unsigned)(B * nf * a.ncg), s)) return e;
      if (int e = run_seg_carry_fwd(seg, ptot, a.h0, a.hL, B, a.D, a.N, nf, s)) return e;
      a.B = B * ns; a.L = Ls; a.ns = ns; a.nck = Ls / a.ck; a.h0 = seg; a.hL = nullptr; a.hs = r; a.ho = 0;
    }
  }
  if (mode == 6) {
    // one pre-pass for the step: the backward call that follows finds its images too (it needs the
    // checkpoints, so a call without them is not followed by one)
    const bool with_bwd = a.hck != nullptr;
    PrepArgs pa{a.Bm, a.Cm, ws.fimg, with_bwd ? ws.img : nullptr, a.N, L, (L + XT - 1) / XT, nullptr, ImgStamp{}};
    if (int e = run_px_prep(pa, B, in_dtype, s)) return e;
    const ImgNote note{ws.stamp, img_stamp(a.Bm, a.Cm, B, a.N, L, in_dtype, with_bwd), clear_in_kernel ? ws.pad : nullptr};
    return run_px_fwd(a, ws.fimg, note, in_dtype, s);
  }
  return run_xdl_fwd(mode, a, in_dtype, s);
}

// Complex and real scans: with a workspace and few (batch, channel group) pairs, split along the sequence.
int launch_generic_fwd(int variant, FwdArgs a, int in_dtype, float* ws, hipStream_t s) {
  if (in_dtype == AUSSM_BF16 && !ws) return AUSSM_E_NULL;
  if (misaligned(ws, 16)) return AUSSM_E_ALIGN;
  const BcF32 bc = generic_bc(variant, a.Bm, a.Cm, ws, a.B, a.D, a.N, a.L, a.ck, in_dtype, s);
  if (bc.err) return bc.err;
  a.Bm = bc.Bm; a.Cm = bc.Cm; in_dtype = bc.in_dtype;
  const Cfg cfg = pick_cfg(a.N, 8);
  const GSplit sp = ws ? generic_split(a.B, a.D, a.L, a.ck, true) : GSplit{1, a.L};
  if (sp.ns > 1) {
    const int B = a.B, C = variant == VAR_REAL ? 1 : 2;
    float* seg = ws;
    float* ptot = seg + (size_t)B * sp.ns * a.D * a.N * C;
    // 1. end state of every segment from a zero state (no outputs) and the product of its a_l
    FwdArgs z = a;
    z.B = B * sp.ns; z.L = sp.ls; z.ns = sp.ns;
    z.y = nullptr; z.z = nullptr; z.Dskip = nullptr; z.h0 = nullptr; z.hL = seg; z.hck = nullptr; z.ptot = ptot;
    if (int e = run_core_fwd(variant, z, in_dtype, cfg, s)) return e;
    // 2. the state that enters every segment; the state after the last one is the call's hL
    if (int e = variant == VAR_COMPLEX ? run_seg_carry_fwd(seg, ptot, a.h0, a.hL, B, a.D, a.N, sp.ns, s)
                                       : run_seg_carry_real(false, seg, ptot, a.A, a.h0, a.hL, B, a.D, a.N, sp.ns, s))
      return e;
    // 3. the scan proper over (batch, segment) pairs
    a.B = B * sp.ns; a.L = sp.ls; a.ns = sp.ns; a.h0 = seg; a.hL = nullptr;
  }
  return run_core_fwd(variant, a, in_dtype, cfg, s);
}

int launch_generic_bwd(int variant, RecBwdArgs a, int in_dtype, float* ws, hipStream_t s) {
  if (in_dtype == AUSSM_BF16 && !ws) return AUSSM_E_NULL;
  if (misaligned(ws, 16)) return AUSSM_E_ALIGN;
  const BcF32 bc = generic_bc(variant, a.Bm, a.Cm, ws, a.B, a.D, a.N, a.L, REC_CK, in_dtype, s);
  if (bc.err) return bc.err;
  a.Bm = bc.Bm; a.Cm = bc.Cm; in_dtype = bc.in_dtype;
  const GSplit sp = ws ? generic_split(a.B, a.D, a.L, REC_CK, true) : GSplit{1, a.L};
  if (sp.ns > 1) {
    const int B = a.B, C = variant == VAR_REAL ? 1 : 2;
    float* seg = ws;
    float* ptot = seg + (size_t)B * sp.ns * a.D * a.N * C;
    AdjSegArgs g{};
    g.dy = a.dy; g.z = a.z; g.delta = a.delta; g.theta = a.theta; g.rho = a.rho; g.A = a.A; g.Cm = a.Cm;
    g.delta_bias = a.delta_bias; g.out = seg; g.ptot = ptot;
    g.D = a.D; g.N = a.N; g.L = sp.ls; g.ld = a.L; g.ns = sp.ns; g.ncg = a.ncg; g.delta_softplus = a.delta_softplus;
    if (int e = run_adjoint_seg(variant, g, in_dtype, (unsigned)(B * sp.ns * a.ncg), s)) return e;
    if (int e = variant == VAR_COMPLEX ? run_seg_carry_bwd(seg, ptot, a.dhL, a.dh0, B, a.D, a.N, sp.ns, s)
                                       : run_seg_carry_real(true, seg, ptot, a.A, a.dhL, a.dh0, B, a.D, a.N, sp.ns, s))
      return e;
    a.B = B * sp.ns; a.L = sp.ls; a.ns = sp.ns; a.dhL = seg; a.dh0 = nullptr;
  }
  return run_rec_bwd(variant, a, in_dtype, s);
}

// ---- static workspace of aussm_unitary_fwd_static ---------------------------------------------
// A file-scope device array: every GPU the library runs on holds its own copy at its own address
// until the process ends.  In host code the array's NAME is only a handle for the runtime, not a
// device address: the address is looked up once per device (hipGetSymbolAddress) and that pointer
// is what the launches are given.
constexpr size_t STATIC_SCRATCH_FLOATS = AUSSM_STATIC_SCRATCH_BYTES / sizeof(float);
static __device__ __align__(256) float g_static_scratch[STATIC_SCRATCH_FLOATS];
constexpr int MAX_DEVICES = 64;
std::atomic<float*> g_static_scratch_ptr[MAX_DEVICES];

int static_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEVICES) return AUSSM_E_SHAPE;
  float* ptr = g_static_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(g_static_scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return AUSSM_E_NULL;
    g_static_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return AUSSM_OK;
}

}  // namespace

extern "C" {

int aussm_version(void) { return 100; }

const char* aussm_error_string(int code) {
  switch (code) {
    case AUSSM_OK: return "ok";
    case AUSSM_E_NULL: return "a required pointer is NULL";
    case AUSSM_E_SHAPE: return "dimension out of the supported range (B,D,N,L >= 1, N <= 64)";
    case AUSSM_E_CK: return "checkpoint interval must be a multiple of 32 accepted by this function";
    case AUSSM_E_DTYPE: return "in_dtype must be AUSSM_F32 or AUSSM_BF16";
    case AUSSM_E_ALIGN: return "pointer not aligned to its element size";
    case AUSSM_E_SCRATCH: return "the call needs more workspace than the static scratch holds (use the _aux entry point)";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown aussm error";
  }
}

int aussm_set_option(int key, int value) {
  if (key < 0 || key >= AUSSM_OPT_COUNT) return AUSSM_E_SHAPE;
  g_opt[key].store(value < 0 ? -1 : value, std::memory_order_relaxed);
  return AUSSM_OK;
}

int aussm_get_option(int key) {
  if (key < 0 || key >= AUSSM_OPT_COUNT) return AUSSM_E_SHAPE;
  return opt(key);
}

int aussm_num_checkpoints(int L, int ck) { return (L < 1 || ck < 1) ? 0 : (L + ck - 1) / ck; }

int aussm_bwd_checkpoint_interval(int variant) { return variant == VAR_UNITARY ? 0 : REC_CK; }

int aussm_unitary_split_segments(int B, int D, int N, int L, int ck) {
  if (B < 1 || D < 1 || N < 1 || L < 1 || ck < 1) return 0;
  int ns = seg_capacity(B, D, N, L, ck);
  // shapes that the vector-ALU kernels serve by default split their way
  if (!(matrix_shape(N, L, ck) && N >= MATRIX_MIN_STATE)) {
    const int g = generic_split(B, D, L, ck, false).ns;
    if (g > ns) ns = g;
  }
  return ns;
}

size_t aussm_unitary_aux_floats(int B, int D, int N, int L, int ck) {
  if (B < 1 || D < 1 || N < 1 || L < 1) return 0;
  return aux_im_floats(B, D, N, L, ck) + AUX_PAD + aux_seg_floats(B, D, N, L, ck) + img_floats(B, N, L, ck);
}

size_t aussm_scan_workspace_floats(int variant, int B, int D, int N, int L, int ck, int in_dtype) {
  if (B < 1 || D < 1 || N < 1 || L < 1 || (variant != VAR_COMPLEX && variant != VAR_REAL)) return 0;
  if (ck != AUSSM_TILE / 2 && (ck < AUSSM_TILE || ck % AUSSM_TILE != 0)) return 0;
  return generic_split_floats(variant, B, D, N, L, ck) + 2 * generic_bc_floats(variant, B, N, L, in_dtype);
}

int aussm_unitary_kernel_mode(int backward, int B, int D, int N, int L, int ck, int in_dtype, int urep, int have_aux) {
  if (check_common(B, D, N, L, ck, in_dtype) != AUSSM_OK || urep < 1) return 0;
  const bool have_img = have_aux && img_floats(B, N, L, ck) > 0;
  return backward ? bwd_mode_for(B, D, N, L, ck, urep, have_img) : fwd_mode_for(N, L, ck, in_dtype, urep, have_img);
}

int aussm_hbm_probe(const float* a, const float* b, const float* c, float* o1, float* o2, int rows, int L,
                    int pattern, int write, void* stream) {
  if (rows < 64 || rows % 64 != 0 || L < 64 || L % 64 != 0 || (pattern != 0 && pattern != 1)) return AUSSM_E_SHAPE;
  if (!a || !b || !c || !o1 || (write && !o2)) return AUSSM_E_NULL;
  if (misaligned(a, 16) || misaligned(b, 16) || misaligned(c, 16) || misaligned(o1, 16) || misaligned(o2, 16))
    return AUSSM_E_ALIGN;
  return run_hbm_probe(a, b, c, o1, o2, rows, L, pattern, write, (hipStream_t)stream);
}

int aussm_unitary_fwd(const void* u, const void* delta, const float* theta, const void* Bc, const void* Cc,
                      const float* Dskip, const float* z, const float* h0, float* y, float* hL, float* hck,
                      int B, int D, int N, int L, int ck, int in_dtype, void* stream) {
  return aussm_unitary_fwd_aux(u, delta, theta, Bc, Cc, Dskip, z, h0, y, hL, hck, nullptr, B, D, N, L, ck, in_dtype,
                               1, stream);
}

int aussm_unitary_fwd_aux(const void* u, const void* delta, const float* theta, const void* Bc, const void* Cc,
                          const float* Dskip, const float* z, const float* h0, float* y, float* hL, float* hck,
                          float* aux, int B, int D, int N, int L, int ck, int in_dtype, int urep, void* stream) {
  if (int e = check_common(B, D, N, L, ck, in_dtype)) return e;
  if (urep < 1 || B % urep != 0) return AUSSM_E_SHAPE;
  if (misaligned(aux, 16)) return AUSSM_E_ALIGN;
  if (!u || !delta || !theta || !Bc || !Cc) return AUSSM_E_NULL;
  const size_t ca = in_dtype == AUSSM_BF16 ? 4 : 8;
  if (misaligned(Bc, ca) || misaligned(Cc, ca)) return AUSSM_E_ALIGN;
  FwdArgs a{};
  a.u = u; a.delta = delta; a.theta = theta; a.Bm = Bc; a.Cm = Cc; a.Dskip = Dskip; a.z = z;
  a.h0 = h0; a.y = y; a.hL = hL; a.hck = hck; a.aux = aux;
  a.B = B; a.D = D; a.N = N; a.L = L; a.ck = ck; a.nck = (L + ck - 1) / ck; a.ncg = (D + CH - 1) / CH;
  a.ld = L; a.ns = 1; a.hs = 1; a.ho = 0; a.urep = urep;
  a.auxtag = aux_tag(u, delta, theta, Bc, Cc, B, D, N, L, in_dtype);
  return launch_unitary_fwd(a, in_dtype, (hipStream_t)stream, aux_layout(aux, B, D, N, L, ck));
}

int aussm_static_init(void) {
  float* ptr = nullptr;
  return static_scratch(&ptr);
}

int aussm_unitary_fwd_static(const void* u, const void* delta, const float* theta, const void* Bc, const void* Cc,
                             const float* Dskip, const float* z, const float* h0, float* y, float* hL,
                             int B, int D, int N, int L, int ck, int in_dtype, void* stream) {
  if (int e = check_common(B, D, N, L, ck, in_dtype)) return e;
  if (!u || !delta || !theta || !Bc || !Cc) return AUSSM_E_NULL;
  const size_t ca = in_dtype == AUSSM_BF16 ? 4 : 8;
  if (misaligned(Bc, ca) || misaligned(Cc, ca)) return AUSSM_E_ALIGN;
  // the only workspace a forward call without checkpoints uses: the segment states of a launch
  // that is split along L
  const size_t need = seg_floats(B, D, N, L, seg_capacity(B, D, N, L, ck));
  if (need > STATIC_SCRATCH_FLOATS) return AUSSM_E_SCRATCH;
  float* scratch = nullptr;
  if (need > 0)
    if (int e = static_scratch(&scratch)) return e;
  FwdArgs a{};
  a.u = u; a.delta = delta; a.theta = theta; a.Bm = Bc; a.Cm = Cc; a.Dskip = Dskip; a.z = z;
  a.h0 = h0; a.y = y; a.hL = hL; a.hck = nullptr; a.aux = nullptr;
  a.B = B; a.D = D; a.N = N; a.L = L; a.ck = ck; a.nck = (L + ck - 1) / ck; a.ncg = (D + CH - 1) / CH;
  a.ld = L; a.ns = 1; a.hs = 1; a.ho = 0; a.urep = 1;
  // (every segment state the scan reads is written earlier in the same call: nothing in the
  // scratch has to start at zero)
  // (the vector-ALU kernels do not split here: no gseg)
  return launch_unitary_fwd(a, in_dtype, (hipStream_t)stream, AuxLayout{scratch, nullptr, nullptr, nullptr, nullptr, nullptr});
}

int aussm_complex_fwd(const void* u, const void* delta, const float* rho, const float* theta, const void* Bc,
                      const void* Cc, const float* Dskip, const float* z, const float* h0, float* y, float* hL,
                      float* hck, float* workspace, int B, int D, int N, int L, int ck, int in_dtype, void* stream) {
  if (int e = check_common(B, D, N, L, ck, in_dtype)) return e;
  if (!u || !delta || !rho || !theta || !Bc || !Cc) return AUSSM_E_NULL;
  const size_t ca = in_dtype == AUSSM_BF16 ? 4 : 8;
  if (misaligned(Bc, ca) || misaligned(Cc, ca)) return AUSSM_E_ALIGN;
  FwdArgs a{};
  a.u = u; a.delta = delta; a.rho = rho; a.theta = theta; a.Bm = Bc; a.Cm = Cc; a.Dskip = Dskip; a.z = z;
  a.h0 = h0; a.y = y; a.hL = hL; a.hck = hck;
  a.B = B; a.D = D; a.N = N; a.L = L; a.ck = ck; a.nck = (L + ck - 1) / ck; a.ncg = (D + CH - 1) / CH;
  a.ld = L; a.ns = 1; a.hs = 1; a.ho = 0; a.urep = 1;
  return launch_generic_fwd(VAR_COMPLEX, a, in_dtype, workspace, (hipStream_t)stream);
}

int aussm_real_fwd(const void* u, const void* delta, const float* A, const void* Bm, const void* Cm,
                   const float* Dskip, const float* z, const float* delta_bias, int delta_softplus,
                   const float* h0, float* y, float* hL, float* hck, float* workspace,
                   int B, int D, int N, int L, int ck, int in_dtype, void* stream) {
  if (int e = check_common(B, D, N, L, ck, in_dtype)) return e;
  if (!u || !delta || !A || !Bm || !Cm) return AUSSM_E_NULL;
  FwdArgs a{};
  a.u = u; a.delta = delta; a.A = A; a.Bm = Bm; a.Cm = Cm; a.Dskip = Dskip; a.z = z;
  a.delta_bias = delta_bias; a.delta_softplus = delta_softplus;
  a.h0 = h0; a.y = y; a.hL = hL; a.hck = hck;
  a.B = B; a.D = D; a.N = N; a.L = L; a.ck = ck; a.nck = (L + ck - 1) / ck; a.ncg = (D + CH - 1) / CH;
  a.ld = L; a.ns = 1; a.hs = 1; a.ho = 0; a.urep = 1;
  return launch_generic_fwd(VAR_REAL, a, in_dtype, workspace, (hipStream_t)stream);
}

int aussm_unitary_bwd(const float* dy, const float* dhL, const void* u, const void* delta, const float* theta,
                      const void* Bc, const void* Cc, const float* Dskip, const float* hck,
                      float* du, float* ddelta, float* dtheta, float* dB, float* dC, float* dD, float* dh0,
                      int B, int D, int N, int L, int ck, int in_dtype, void* stream) {
  return aussm_unitary_bwd_aux(dy, dhL, u, delta, theta, Bc, Cc, Dskip, hck, nullptr, du, ddelta, dtheta, dB, dC, dD,
                               dh0, B, D, N, L, ck, in_dtype, 1, stream);
}

int aussm_unitary_bwd_aux(const float* dy, const float* dhL, const void* u, const void* delta, const float* theta,
                          const void* Bc, const void* Cc, const float* Dskip, const float* hck, float* aux,
                          float* du, float* ddelta, float* dtheta, float* dB, float* dC, float* dD, float* dh0,
                          int B, int D, int N, int L, int ck, int in_dtype, int urep, void* stream) {
  if (int e = check_common(B, D, N, L, ck, in_dtype)) return e;
  if (urep < 1 || B % urep != 0) return AUSSM_E_SHAPE;
  if (misaligned(aux, 16)) return AUSSM_E_ALIGN;
  if (!dy || !u || !delta || !theta || !Bc || !Cc || !hck || !du || !ddelta || !dtheta || !dB || !dC)
    return AUSSM_E_NULL;
  const size_t ca = in_dtype == AUSSM_BF16 ? 4 : 8;
  if (misaligned(Bc, ca) || misaligned(Cc, ca)) return AUSSM_E_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  UniBwdArgs a{};
  a.dy = dy; a.dhL = dhL; a.u = u; a.delta = delta; a.theta = theta; a.Bm = Bc; a.Cm = Cc; a.Dskip = Dskip;
  a.hck = hck; a.aux = aux; a.du = du; a.ddelta = ddelta; a.dtheta = dtheta; a.dB = dB; a.dC = dC; a.dD = dD; a.dh0 = dh0;
  a.B = B; a.D = D; a.N = N; a.L = L; a.ck = ck; a.nck = (L + ck - 1) / ck; a.ncg = (D + CH - 1) / CH;
  a.ld = L; a.ns = 1; a.hs = 1; a.ho = 0; a.urep = 1;
  a.urep = urep;
  a.auxtag = aux_tag(u, delta, theta, Bc, Cc, B, D, N, L, in_dtype);
  const AuxLayout ws = aux_layout(aux, B, D, N, L, ck);
  const int mode = bwd_mode_for(B, D, N, L, ck, urep, ws.img != nullptr);
  if (mode > 0 &&
      !(misaligned(dy, 16) || misaligned(u, 16) || misaligned(delta, 16) || misaligned(theta, 16) ||
        misaligned(du, 16) || misaligned(ddelta, 16) || misaligned(dtheta, 16) || misaligned(Bc, 16) ||
        misaligned(Cc, 16))) {
    const int ns = aux ? seg_count(B, D, N, L, ck) : 1;
    if (ns > 1) {
      // adjoint at the start of every segment from a zero adjoint at its end, chained last to first
      const int Ls = L / ns, r = seg_fine(L, ns), nf = ns * r;
      float* seg = ws.seg;
      float* ptot = seg + (size_t)B * nf * D * N * 2;
      SegArgs sa{dy, nullptr, theta, Cc, seg, ptot, D, N, Ls / r, L, nf, a.ncg};
      if (int e = run_seg_state(true, sa, in_dtype, (unsigned)(B * nf * a.ncg), s)) return e;
      if (int e = run_seg_carry_bwd(seg, ptot, dhL, dh0, B, D, N, nf, s)) return e;
      // a segment of the scan ends where its last fine segment ends
      a.B = B * ns; a.L = Ls; a.ns = ns; a.nck = Ls / ck; a.dhL = seg; a.dh0 = nullptr; a.hs = r; a.ho = r - 1;
    }
    if (mode == 6) {
      // The prepared-operand kernel needs Im(P S) from the forward call in the auxiliary buffer; its
      // workgroups leave at once if the buffer's tag says it is not there, and the kernel that
      // recomputes it (launched behind, leaving at once in the opposite case) does the work.
      // (the pre-pass leaves at once when the forward call of these tensors has left the images)
      PrepArgs pa{Bc, Cc, nullptr, ws.img, N, L, (L + XT - 1) / XT, ws.stamp, img_stamp(Bc, Cc, B, N, L, in_dtype, true)};
      if (int e = run_px_prep(pa, B, in_dtype, s)) return e;
      a.tag_mode = 1;
      if (int e = run_px_bwd(a, ws.img, in_dtype, s)) return e;
      a.tag_mode = 2;
      return run_xdl_bwd(3, a, in_dtype, s);
    }
    return run_xdl_bwd(mode, a, in_dtype, s);
  }
  // vector-ALU kernel; split along the sequence like the forward call
  const GSplit sp = ws.gseg ? generic_split(B, D, L, ck, true) : GSplit{1, L};
  if (sp.ns > 1) {
    float* seg = ws.gseg;
    float* ptot = seg + (size_t)B * sp.ns * D * N * 2;
    AdjSegArgs g{};
    g.dy = dy; g.theta = theta; g.Cm = Cc; g.out = seg; g.ptot = ptot;
    g.D = D; g.N = N; g.L = sp.ls; g.ld = L; g.ns = sp.ns; g.ncg = a.ncg;
    if (int e = run_adjoint_seg(VAR_UNITARY, g, in_dtype, (unsigned)(B * sp.ns * a.ncg), s)) return e;
    if (int e = run_seg_carry_bwd(seg, ptot, dhL, dh0, B, D, N, sp.ns, s)) return e;
    a.B = B * sp.ns; a.L = sp.ls; a.ns = sp.ns; a.dhL = seg; a.dh0 = nullptr;
  }
  return run_unitary_bwd_generic(a, in_dtype, pick_cfg(a.N, 8), s);
}

int aussm_complex_bwd(const float* dy, const float* dhL, const void* u, const void* delta, const float* rho,
                      const float* theta, const void* Bc, const void* Cc, const float* Dskip,
                      const float* h0, const float* hck,
                      float* du, float* ddelta, float* drho, float* dtheta, float* dB, float* dC,
                      float* dD, float* dh0, const float* z, float* dz, float* workspace,
                      int B, int D, int N, int L, int ck, int in_dtype, void* stream) {
  if (int e = check_common(B, D, N, L, ck, in_dtype)) return e;
  if (ck != REC_CK) return AUSSM_E_CK;
  if (!dy || !u || !delta || !rho || !theta || !Bc || !Cc || !hck || !du || !ddelta || !drho || !dtheta ||
      !dB || !dC)
    return AUSSM_E_NULL;
  const size_t ca = in_dtype == AUSSM_BF16 ? 4 : 8;
  if (misaligned(Bc, ca) || misaligned(Cc, ca)) return AUSSM_E_ALIGN;
  RecBwdArgs a{};
  a.dy = dy; a.dhL = dhL; a.u = u; a.delta = delta; a.theta = theta; a.rho = rho; a.Bm = Bc; a.Cm = Cc;
  a.Dskip = Dskip; a.h0 = h0; a.hck = hck;
  a.du = du; a.ddelta = ddelta; a.dtheta = dtheta; a.drho = drho; a.dB = dB; a.dC = dC; a.dD = dD; a.dh0 = dh0;
  if ((z == nullptr) != (dz == nullptr)) return AUSSM_E_NULL;
  a.z = z; a.dz = dz;
  a.B = B; a.D = D; a.N = N; a.L = L; a.nck = (L + ck - 1) / ck; a.ncg = (D + CH - 1) / CH;
  a.ld = L; a.ns = 1;
  return launch_generic_bwd(VAR_COMPLEX, a, in_dtype, workspace, (hipStream_t)stream);
}

int aussm_real_bwd(const float* dy, const float* dhL, const void* u, const void* delta, const float* A,
                   const void* Bm, const void* Cm, const float* Dskip, const float* delta_bias,
                   int delta_softplus, const float* h0, const float* hck,
                   float* du, float* ddelta, float* dA, float* dB, float* dC, float* dD, float* dh0,
                   const float* z, float* dz, float* workspace,
                   int B, int D, int N, int L, int ck, int in_dtype, void* stream) {
  if (int e = check_common(B, D, N, L, ck, in_dtype)) return e;
  if (ck != REC_CK) return AUSSM_E_CK;
  if (!dy || !u || !delta || !A || !Bm || !Cm || !hck || !du || !ddelta || !dB || !dC) return AUSSM_E_NULL;
  RecBwdArgs a{};
  a.dy = dy; a.dhL = dhL; a.u = u; a.delta = delta; a.A = A; a.Bm = Bm; a.Cm = Cm; a.Dskip = Dskip;
  a.delta_bias = delta_bias; a.delta_softplus = delta_softplus; a.h0 = h0; a.hck = hck;
  a.du = du; a.ddelta = ddelta; a.dA = dA; a.dB = dB; a.dC = dC; a.dD = dD; a.dh0 = dh0;
  if ((z == nullptr) != (dz == nullptr)) return AUSSM_E_NULL;
  a.z = z; a.dz = dz;
  a.B = B; a.D = D; a.N = N; a.L = L; a.nck = (L + ck - 1) / ck; a.ncg = (D + CH - 1) / CH;
  a.ld = L; a.ns = 1;
  return launch_generic_bwd(VAR_REAL, a, in_dtype, workspace, (hipStream_t)stream);
}

int aussm_causal_conv1d_fwd(const float* x, const float* w, const float* bias, float* y,
                            int B, int L, int D, int K, long long xs_b, long long xs_l, void* stream) {
  if (B < 1 || L < 1 || D < 1 || K < 1 || K > CONV_MAX_K || xs_l < D || xs_b < (long long)L * xs_l - (xs_l - D))
    return AUSSM_E_SHAPE;
  if (!x || !w || !y) return AUSSM_E_NULL;
  ConvArgs a{};
  a.x = x; a.w = w; a.bias = bias; a.y = y; a.xs_b = xs_b; a.xs_l = xs_l; a.B = B; a.L = L; a.D = D; a.K = K;
  const size_t rows = (size_t)B * L;
  if (rows > 0x7fffffffULL || (D + 255) / 256 > 65535) return AUSSM_E_SHAPE;
  return run_conv_fwd(a, (hipStream_t)stream);
}

int aussm_causal_conv1d_bwd(const float* dy, const float* x, const float* w, float* dx, float* dw, float* dbias,
                            int B, int L, int D, int K, long long xs_b, long long xs_l, void* stream) {
  if (B < 1 || L < 1 || D < 1 || K < 1 || K > CONV_MAX_K || xs_l < D || xs_b < (long long)L * xs_l - (xs_l - D))
    return AUSSM_E_SHAPE;
  if (!dy || !x || !w || !dx || !dw) return AUSSM_E_NULL;
  ConvArgs a{};
  a.x = x; a.w = w; a.dy = dy; a.dx = dx; a.dw = dw; a.dbias = dbias;
  a.xs_b = xs_b; a.xs_l = xs_l; a.B = B; a.L = L; a.D = D; a.K = K;
  const size_t rows = (size_t)B * L;
  if (rows > 0x7fffffffULL || (D + 255) / 256 > 65535 || (rows + CONV_ROWS - 1) / CONV_ROWS > 65535) return AUSSM_E_SHAPE;
  return run_conv_bwd(a, (hipStream_t)stream);
}

int aussm_swap_last2(const float* x, float* y, int B, int R, int C, long long xs_b, long long xs_r, void* stream) {
  if (B < 1 || R < 1 || C < 1 || B > 65535 || xs_r < C || xs_b < (long long)R * xs_r - (xs_r - C)) return AUSSM_E_SHAPE;
  if ((R + 31) / 32 > 65535) return AUSSM_E_SHAPE;
  if (!x || !y) return AUSSM_E_NULL;
  SwapArgs a{};
  a.x = x; a.y = y; a.xs_b = xs_b; a.xs_r = xs_r; a.R = R; a.C = C;
  return run_swap_last2(a, B, (hipStream_t)stream);
}

int aussm_swap_last2_act(const float* x, const float* bias, const float* pre, float* y, int B, int R, int C,
                         long long xs_b, long long xs_r, long long ps_b, long long ps_r, int act, int deriv,
                         void* stream) {
  if (B < 1 || R < 1 || C < 1 || B > 65535 || xs_r < C || xs_b < (long long)R * xs_r - (xs_r - C)) return AUSSM_E_SHAPE;
  if ((R + 31) / 32 > 65535 || act < 1 || act > 2) return AUSSM_E_SHAPE;
  if (!x || !y || (deriv && !pre)) return AUSSM_E_NULL;
  // pre has the output's shape (B, C, R): rows of R elements that do not overlap
  if (deriv && (ps_r < R || ps_b < (long long)C * ps_r - (ps_r - R))) return AUSSM_E_SHAPE;
  SwapArgs a{};
  a.x = x; a.y = y; a.xs_b = xs_b; a.xs_r = xs_r; a.R = R; a.C = C;
  a.bias = bias; a.pre = deriv ? pre : nullptr; a.ps_b = ps_b; a.ps_r = ps_r; a.act = act; a.deriv = deriv ? 1 : 0;
  return run_swap_last2(a, B, (hipStream_t)stream);
}

int aussm_gate_fwd(const float* y_pre, const float* z, float* y, size_t n, void* stream) {
  if (!y_pre || !z || !y) return AUSSM_E_NULL;
  if (n < 1) return AUSSM_E_SHAPE;
  if (misaligned(y_pre, 4) || misaligned(z, 4) || misaligned(y, 4)) return AUSSM_E_ALIGN;
  return run_gate(nullptr, y_pre, z, y, nullptr, n, (hipStream_t)stream);
}

int aussm_gate_bwd(const float* dy, const float* y_pre, const float* z, float* dy_pre, float* dz, size_t n, void* stream) {
  if (!dy || !y_pre || !z || !dy_pre || !dz) return AUSSM_E_NULL;
  if (n < 1) return AUSSM_E_SHAPE;
  if (misaligned(dy, 4) || misaligned(y_pre, 4) || misaligned(z, 4) || misaligned(dy_pre, 4) || misaligned(dz, 4))
    return AUSSM_E_ALIGN;
  return run_gate(dy, y_pre, z, dy_pre, dz, n, (hipStream_t)stream);
}

// ---- the reference's operator extension_cpp::ssm_adaptive_unitary as fused kernels (dropin.h)

// blocks of 16 states per channel, one per wavefront: 1, 2 or 4 (they have to divide the wavefronts of a workgroup)
static int dropin_state_blocks(int n) { const int k = (n + 15) / 16; return k == 3 ? 4 : k; }
static size_t dropin_xp_floats(int d, int n) { return (size_t)d * dropin_state_blocks(n) * ((d + 31) / 32) * 3 * 64 * 4; }
// The backward call works through the (batch, sequence) plane in blocks of bg batch elements x ct tiles
// of 16 timesteps: the workspace holds the phase adjoints of one block (about 100 MiB at most:
// at b = 32, d = 256, n = 16, L = 720 a block of 8 batch elements then spans the whole sequence, 1.39 ms per backward
// call against 1.64 ms with 50 MiB blocks).  bg is
// what fills the chip with one workgroup per compute unit (fewer would idle units, more would only
// shorten the blocks and repeat the per-launch set-up, the rows of x among it, more often).
// budget of a block (phase adjoints; prepared tiles of u), in floats
// (the option can only lower it: the workspace query sizes for the full budget, so a buffer obtained under
// one setting of the option holds what a call under any other setting uses)
constexpr int DROPIN_BLOCK_KFLOATS = 25600;
static size_t dropin_block_floats(bool largest) {
  const int o = opt(AUSSM_OPT_BLOCK_KFLOATS);
  return (size_t)(!largest && o > 0 && o < DROPIN_BLOCK_KFLOATS ? o : DROPIN_BLOCK_KFLOATS) << 10;
}
struct DropinBlocks { int bg, ct; };
static DropinBlocks dropin_blocks(int b, int d, int n, int L, bool largest = false) {
  const int nw = dropin_channels_per_workgroup((d + 31) / 32);
  const int wgs_per_b = (d * dropin_state_blocks(n) + nw - 1) / nw;
  int bg = (256 + wgs_per_b - 1) / wgs_per_b;
  if (bg > b) bg = b;
  const int ng = (b + bg - 1) / bg;
  bg = (b + ng - 1) / ng;
  const size_t per_tile = (size_t)bg * d * n * DT, cap = dropin_block_floats(largest);
  const int ntiles = (L + DT - 1) / DT;
  size_t tmax = cap / per_tile;
  if (tmax < 1) tmax = 1;
  const size_t nc = ((size_t)ntiles + tmax - 1) / tmax;
  return DropinBlocks{bg, (int)(((size_t)ntiles + nc - 1) / nc)};
}
// How a GEMM launch is cut: about three workgroups of 128 x 128 per two compute units.  Without reduce_z every z is a
// slice of its own and k is cut (at least four steps per slice); with reduce_z the z are dealt to the
// slices first and k is cut only when there are too few z.
constexpr long GEMM_TARGET = 384;     // workgroups per launch aimed at (measured: 256 and 512 +9 % of the backward call)
static void gemm_slices(GemmArgs& g) {
  const long tiles = (long)((g.M + GEMM_TILE_M - 1) / GEMM_TILE_M) * ((g.N + GEMM_TILE_N - 1) / GEMM_TILE_N);
  const long target = GEMM_TARGET;
  const int nk = (g.K + 31) / 32;
  long zs = 1;                                   // slices of z
  g.zper = 1;
  if (g.reduce_z) {
    zs = (target + tiles - 1) / tiles;
    if (zs > g.Z) zs = g.Z;
    if (zs < 1) zs = 1;
    g.zper = (int)((g.Z + zs - 1) / zs);
    zs = (g.Z + g.zper - 1) / g.zper;
  } else {
    zs = g.Z;
  }
  long s = (target + tiles * zs - 1) / (tiles * zs);
  if (s > nk / 4) s = nk / 4;
  if (s < 1) s = 1;
  while (s > 1 && zs * s > 65535) --s;
  g.ksplit = (int)s;
}
static size_t round4(size_t v) { return (v + 3) & ~(size_t)3; }
static int dropin_check(int b, int d, int n, int L) {
  if (b < 1 || d < 1 || n < 1 || L < 1) return AUSSM_E_SHAPE;
  if (n > D_MAXN || d > 32 * D_MAXKS) return AUSSM_E_SHAPE;
  if ((long long)b * d > 0x7fffffffLL || (long long)d * n * L > 0x7fffffffLL) return AUSSM_E_SHAPE;
  return AUSSM_OK;
}

// floats of one prepared tile of u (all compiled steps of the contraction, three pieces, 64 lanes of 16 bytes)
static size_t dropin_tile_floats(int d) { return (size_t)dropin_compiled_ks((d + 31) / 32) * 3 * 64 * 4; }
// tiles per launch of the forward call: its prepared tiles of u (all batch elements) stay within the block budget
static int dropin_fwd_chunk_tiles(int b, int d, int L, bool largest = false) {
  const int ntiles = (L + DT - 1) / DT;
  size_t tmax = dropin_block_floats(largest) / ((size_t)b * dropin_tile_floats(d));
  if (tmax < 1) tmax = 1;
  const size_t nc = ((size_t)ntiles + tmax - 1) / tmax;
  return (int)(((size_t)ntiles + nc - 1) / nc);
}

size_t aussm_ssm_adaptive_unitary_workspace_floats(int b, int d, int n, int L, int backward) {
  if (dropin_check(b, d, n, L) != AUSSM_OK) return 0;
  size_t f = dropin_xp_floats(d, n);
  if (backward) {
    const DropinBlocks k = dropin_blocks(b, d, n, L, true);
    f += 2 * round4((size_t)b * d * n) + (size_t)k.bg * k.ct * DT * d * n + (size_t)k.bg * k.ct * dropin_tile_floats(d);
    // prepared first operands of the two products with the phase adjoints: x transposed (once per call), u of a block
    f += 4 * (gemm_image_records(d, d * n) + (size_t)k.bg * gemm_image_records(d, k.ct * DT));
  } else {
    f += (size_t)b * dropin_fwd_chunk_tiles(b, d, L, true) * dropin_tile_floats(d);
  }
  return f;
}

int aussm_ssm_adaptive_unitary_fwd(const float* u, const float* dt, const float* x, const float* x_bias,
                                   const float* B_r, const float* B_theta, const float* C_r, const float* C_theta,
                                   const float* D, const float* z, const float* h_re, const float* h_im,
                                   float* y, float* nh_re, float* nh_im, float* workspace,
                                   int b, int d, int n, int L, void* stream) {
  if (int e = dropin_check(b, d, n, L)) return e;
  if (!u || !dt || !x || !x_bias || !B_r || !B_theta || !C_r || !C_theta || !D || !z || !h_re || !h_im || !y ||
      !nh_re || !nh_im || !workspace)
    return AUSSM_E_NULL;
  if (misaligned(workspace, 16)) return AUSSM_E_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  const int ks = (d + 31) / 32, nb = dropin_state_blocks(n), ntiles = (L + DT - 1) / DT;
  const int ct = dropin_fwd_chunk_tiles(b, d, L);
  u4* xp = (u4*)workspace;
  u4* up = (u4*)(workspace + dropin_xp_floats(d, n));
  if (int e = run_dropin_xprep(x, xp, d, n, ks, nb, s)) return e;
  // the sequence in chunks of ct tiles (one chunk unless it is long): prepared tiles of u for the chunk, then the
  // scan over it, the state handed from chunk to chunk in the output buffers
  for (int t0 = 0; t0 < ntiles; t0 += ct) {
    const int t1 = t0 + ct < ntiles ? t0 + ct : ntiles;
    if (int e = run_dropin_uprep(u, up, d, L, ks, 0, b, t0, t1 - t0, s)) return e;
    DropinArgs a{};
    a.u = u; a.dt = dt; a.z = z; a.x_bias = x_bias; a.B_r = B_r; a.B_th = B_theta; a.C_r = C_r; a.C_th = C_theta;
    a.Dp = D; a.h_re = t0 ? nh_re : h_re; a.h_im = t0 ? nh_im : h_im; a.y = y; a.nh_re = nh_re; a.nh_im = nh_im;
    a.xp = xp; a.up = up; a.up_b0 = 0; a.up_t0 = t0; a.up_nt = t1 - t0;
    a.b = b; a.d = d; a.n = n; a.L = L; a.ks = ks; a.nb = nb; a.b0 = 0; a.t0 = t0; a.t1 = t1;
    if (int e = run_dropin_fwd(a, s)) return e;
  }
  return AUSSM_OK;
}

int aussm_ssm_adaptive_unitary_bwd(const float* grad_y, const float* grad_nh_re, const float* grad_nh_im,
                                   const float* u, const float* dt, const float* x, const float* x_bias,
                                   const float* B_r, const float* B_theta, const float* C_r, const float* C_theta,
                                   const float* D, const float* z, const float* h_re, const float* h_im,
                                   const float* nh_re, const float* nh_im,
                                   float* du, float* ddt, float* dx, float* dx_bias, float* dB_r, float* dB_theta,
                                   float* dC_r, float* dC_theta, float* dD, float* dz, float* dh_re, float* dh_im,
                                   float* workspace, int b, int d, int n, int L, void* stream) {
  if (int e = dropin_check(b, d, n, L)) return e;
  if (!grad_y || !u || !dt || !x || !x_bias || !B_r || !B_theta || !C_r || !C_theta || !D || !z || !h_re || !h_im ||
      !du || !ddt || !dx || !dx_bias || !dB_r || !dB_theta || !dC_r || !dC_theta || !dD || !dz || !dh_re || !dh_im ||
      !workspace)
    return AUSSM_E_NULL;
  if (misaligned(workspace, 16)) return AUSSM_E_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  const DropinBlocks blk = dropin_blocks(b, d, n, L);
  const int ks = (d + 31) / 32, nb = dropin_state_blocks(n), ct = blk.ct, lc = ct * DT;
  const int ntiles = (L + DT - 1) / DT;
  const size_t nstate = (size_t)b * d * n;
  u4* xp = (u4*)workspace;
  float* hc_re = workspace + dropin_xp_floats(d, n);
  float* hc_im = hc_re + round4(nstate);
  float* dth = hc_im + round4(nstate);
  u4* up = (u4*)(dth + (size_t)blk.bg * ct * DT * d * n);
  u4* xt = up + (size_t)blk.bg * ct * (dropin_tile_floats(d) / 4);     // image of A(r, (i j)) = x[(i j), r]
  u4* ui = xt + gemm_image_records(d, d * n);                          // images of A_b(r, l) = u[b, r, l0 + l] of a block
  if (int e = run_dropin_xprep(x, xp, d, n, ks, nb, s)) return e;
  if (int e = run_gemm_aprep(x, xt, 1, d, 0, d, d * n, 1, s)) return e;
  DropinArgs f{};
  f.u = u; f.dt = dt; f.z = z; f.x_bias = x_bias; f.B_r = B_r; f.B_th = B_theta; f.C_r = C_r; f.C_th = C_theta;
  f.Dp = D; f.xp = xp; f.up = up; f.d = d; f.n = n; f.L = L; f.ks = ks; f.nb = nb;
  FillArgs fa{};
  auto fill = [&](float* dst, const float* src, size_t cnt) {
    fa.dst[fa.count] = dst; fa.src[fa.count] = src; fa.n[fa.count] = cnt; ++fa.count;
  };
  const bool have_end = nh_re && nh_im;
  if (have_end) {
    fill(hc_re, nh_re, nstate);
    fill(hc_im, nh_im, nstate);
  }
  fill(dh_re, grad_nh_re, nstate);                  // the adjoint of the state travels in the output buffers
  fill(dh_im, grad_nh_im, nstate);
  fill(dx, nullptr, (size_t)d * n * d);
  fill(dx_bias, nullptr, (size_t)d * n);
  fill(dB_r, nullptr, n);
  fill(dB_theta, nullptr, n);
  fill(dC_r, nullptr, n);
  fill(dC_theta, nullptr, n);
  fill(dD, nullptr, d);
  if (int e = run_fill(fa, s)) return e;
  const long dn = (long)d * n;
  for (int b0 = 0; b0 < b; b0 += blk.bg) {
    const int bg = b - b0 < blk.bg ? b - b0 : blk.bg;
    f.b = bg; f.b0 = b0; f.up_b0 = b0;
    if (!have_end) {
      // the state at the end of the sequence: a forward sweep without outputs over this group's chunks
      for (int t0 = 0; t0 < ntiles; t0 += ct) {
        const int t1 = t0 + ct < ntiles ? t0 + ct : ntiles;
        if (int e = run_dropin_uprep(u, up, d, L, ks, b0, bg, t0, t1 - t0, s)) return e;
        DropinArgs a = f;
        a.h_re = t0 ? hc_re : h_re; a.h_im = t0 ? hc_im : h_im; a.y = nullptr; a.nh_re = hc_re; a.nh_im = hc_im;
        a.up_t0 = t0; a.up_nt = t1 - t0; a.t0 = t0; a.t1 = t1;
        if (int e = run_dropin_fwd(a, s)) return e;
      }
    }
    // the chunks in reverse: chunk c covers the tiles c ct .. (same cuts as the forward sweep above)
    for (int t0 = ((ntiles - 1) / ct) * ct; t0 >= 0; t0 -= ct) {
      const int t1 = t0 + ct < ntiles ? t0 + ct : ntiles;
      const int l0 = t0 * DT, len = (t1 * DT < L ? t1 * DT : L) - l0;
      if (int e = run_dropin_uprep(u, up, d, L, ks, b0, bg, t0, t1 - t0, s)) return e;
      DropinBwdArgs q{};
      q.f = f;
      q.f.up_t0 = t0; q.f.up_nt = t1 - t0;
      q.gy = grad_y; q.hc_re = hc_re; q.hc_im = hc_im; q.dth = dth;
      q.du = du; q.ddt = ddt; q.dz = dz; q.dxb = dx_bias;
      q.dB_r = dB_r; q.dB_th = dB_theta; q.dC_r = dC_r; q.dC_th = dC_theta; q.dD = dD;
      q.dh_re = dh_re; q.dh_im = dh_im; q.b0 = b0; q.bg = bg; q.t0 = t0; q.t1 = t1; q.lc = lc;
      if (int e = run_dropin_bwd(q, s)) return e;
      // grad_u[b, r, l0 + l] += sum_(i j) x[(i j), r] hat theta[b, (i j), l]
      GemmArgs gu{};
      gu.Aimg = xt; gu.simz = 0;
      gu.Bm = dth; gu.sbk = lc; gu.sbn = 1; gu.sbz = dn * lc;
      gu.C = du + (size_t)b0 * d * L + l0; gu.scm = L; gu.scn = 1; gu.scz = (long)d * L;
      gu.M = d; gu.N = len; gu.K = (int)dn; gu.Z = bg; gu.reduce_z = 0; gu.accumulate = 1; gu.tr = 0;
      gemm_slices(gu);
      if (int e = run_split_gemm(gu, s)) return e;
      // grad_x[(i j), r] += sum_b sum_l u[b, r, l0 + l] hat theta[b, (i j), l]: rows r, columns (i j), C contiguous along r
      if (int e = run_gemm_aprep(u + (size_t)b0 * d * L + l0, ui, L, 1, (long)d * L, d, len, bg, s)) return e;
      GemmArgs gx{};
      gx.Aimg = ui; gx.simz = (long)gemm_image_records(d, len);
      gx.Bm = dth; gx.sbk = 1; gx.sbn = lc; gx.sbz = dn * lc;
      gx.C = dx; gx.scm = 1; gx.scn = d; gx.scz = 0;
      gx.M = d; gx.N = (int)dn; gx.K = len; gx.Z = bg; gx.reduce_z = 1; gx.accumulate = 1; gx.tr = 1;
      gemm_slices(gx);
      if (int e = run_split_gemm(gx, s)) return e;
    }
  }
  return AUSSM_OK;
}

}  // extern "C"
