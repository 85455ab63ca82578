// Shared device helpers for the gfx950 selective-scan kernels.
//
// Work decomposition used by every kernel in this library
//   * one workgroup owns (batch b, a group of CH = 64 consecutive channels);
//   * inside the scan phase lane i of every wavefront IS channel d0 + i, and wavefront w owns the
//     NW consecutive state indices n0 = w*NW ..; the state of (channel, n) lives in registers;
//   * B_t[b,n,l] / C_t[b,n,l] do not depend on the channel, so inside a wavefront they are
//     wave-uniform: they are fetched with scalar loads and used as SGPR operands of the FMAs;
//   * u / delta / theta / dy are [B,D,L] with L fastest.  A tile of CH channels x T timesteps is
//     loaded with lanes running along L (coalesced 128-byte row segments), converted
//     (sincos / exp / products) once per (channel, timestep), and transposed through LDS into
//     [t][channel] order so that the scan phase reads one 16-byte record per lane per timestep.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "scan_args.h"

namespace aussm {

constexpr int T = 32;         // timesteps per staged tile (AUSSM_TILE)
constexpr int TS = CH + 1;    // padded row stride of [t][channel] LDS tiles (bank-conflict free)
constexpr int NXCD = 8;       // accelerator complex dies, each with a private L2

constexpr float LOG2E = 1.4426950408889634f;

typedef uint16_t bf16_t;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// Workgroups are dealt round-robin to the XCDs (workgroup i runs on XCD i % 8).  Remap so that
// logically consecutive workgroups, which share the B_t/C_t rows of one batch element and
// accumulate into the same dB/dC rows, land on the same XCD and hit in its L2.
__device__ __forceinline__ int xcd_remap(int i, int G) {
  const int q = G / NXCD, r = G % NXCD;
  const int x = i % NXCD, k = i / NXCD;
  return x * q + (x < r ? x : r) + k;
}

__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + __expf(-v)); }
__device__ __forceinline__ float siluf_(float v) { return v * sigmoidf_(v); }
// d/dv silu(v) = s + v s (1 - s)
__device__ __forceinline__ float dsiluf_(float v) { float s = sigmoidf_(v); return s * (1.0f + v * (1.0f - s)); }
// softplus with torch's threshold of 20 (F.softplus default)
__device__ __forceinline__ float softplusf_(float v) { return v > 20.0f ? v : log1pf(__expf(v)); }

// sin and cos of one argument, about 25 VALU instructions and no branch on the common path.
// Cody-Waite reduction by pi/2 in three fused steps, then minimax polynomials on [-pi/4, pi/4]
// (max error ~1 ulp of 1.0 for |x| < 1e4, which covers accumulated phases of practical length).
// Larger arguments take the library routine.
__device__ __forceinline__ void fast_sincosf(float x, float* sn, float* cs) {
  if (__builtin_expect(fabsf(x) > 1.0e4f, 0)) { sincosf(x, sn, cs); return; }
  const float kf = rintf(x * 0.636619772367581343f);
  float r = fmaf(-kf, 1.57079637050628662109375f, x);
  r = fmaf(-kf, -4.37113900018624283e-8f, r);
  r = fmaf(-kf, -1.71512449782676e-15f, r);
  const float r2 = r * r;
  float ps = fmaf(-1.9515295891e-4f, r2, 8.3321608736e-3f);
  ps = fmaf(ps, r2, -1.6666654611e-1f);
  const float s = fmaf(r * r2, ps, r);
  float pc = fmaf(2.443315711809948e-5f, r2, -1.388731625493765e-3f);
  pc = fmaf(pc, r2, 4.166664568298827e-2f);
  const float c = fmaf(r2 * r2, pc, fmaf(-0.5f, r2, 1.0f));
  const int q = (int)kf;
  const float s1 = (q & 1) ? c : s;
  const float c1 = (q & 1) ? s : c;
  *sn = (q & 2) ? -s1 : s1;
  *cs = ((q + 1) & 2) ? -c1 : c1;
}

// wave-uniform loads of B_t / C_t.  idx is uniform across the wavefront.  The tensors are inputs
// that no kernel of this library writes, so they are read through the constant address space:
// that lets the compiler select scalar (SMEM) loads whose results sit in SGPRs and feed the FMAs
// directly.  Complex records are (re, im) pairs.
#define AUSSM_CONST_AS __attribute__((address_space(4)))
template <typename V>
__device__ __forceinline__ const AUSSM_CONST_AS V* const_as(const void* p) {
  return reinterpret_cast<const AUSSM_CONST_AS V*>(reinterpret_cast<uintptr_t>(p));
}
__device__ __forceinline__ float2 ld_c(const float* __restrict__ p, size_t idx) {
  const AUSSM_CONST_AS float* q = const_as<float>(p) + 2 * idx;
  return make_float2(q[0], q[1]);
}
__device__ __forceinline__ float2 ld_c(const bf16_t* __restrict__ p, size_t idx) {
  const uint32_t raw = const_as<uint32_t>(p)[idx];
  return make_float2(__uint_as_float(raw << 16), __uint_as_float(raw & 0xffff0000u));
}
__device__ __forceinline__ float ld_r(const float* __restrict__ p, size_t idx) { return const_as<float>(p)[idx]; }
__device__ __forceinline__ float ld_r(const bf16_t* __restrict__ p, size_t idx) {
  // 16-bit scalar loads do not exist: fetch the aligned 32-bit word and pick the half
  const uint32_t raw = const_as<uint32_t>(p)[idx >> 1];
  return __uint_as_float((idx & 1) ? (raw & 0xffff0000u) : (raw << 16));
}

// ---- eight consecutive timesteps of one state row in one scalar load (one 64-byte line for
// complex fp32).  TG is the number of timesteps the scan consumes per row "turn".
constexpr int TG = 8;
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((aligned(8))) f32x16_a8 { f32x16 v; };
struct __attribute__((aligned(4))) f32x8_a4 { f32x8 v; };
struct __attribute__((aligned(4))) u32x8_a4 { u32x8 v; };
struct __attribute__((aligned(4))) u32x4_a4 { u32x4 v; };

// complex rows: idx counts (re, im) records; result = re0, im0, re1, im1, ...
__device__ __forceinline__ f32x16 ld_c8(const float* __restrict__ p, size_t idx) {
  return const_as<f32x16_a8>(p + 2 * idx)->v;
}
__device__ __forceinline__ f32x16 ld_c8(const bf16_t* __restrict__ p, size_t idx) {
  const u32x8 raw = const_as<u32x8_a4>(p + 2 * idx)->v;
  f32x16 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    r[2 * i] = __uint_as_float(raw[i] << 16);
    r[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
  }
  return r;
}
// real rows.  For bf16 the caller guarantees an even idx (4-byte aligned address).
__device__ __forceinline__ f32x8 ld_r8(const float* __restrict__ p, size_t idx) {
  return const_as<f32x8_a4>(p + idx)->v;
}
__device__ __forceinline__ f32x8 ld_r8(const bf16_t* __restrict__ p, size_t idx) {
  const u32x4 raw = const_as<u32x4_a4>(p + idx)->v;
  f32x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[2 * i] = __uint_as_float(raw[i] << 16);
    r[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
  }
  return r;
}

// Orders the instruction stream at this point: nothing is scheduled across it.
__device__ __forceinline__ void sched_fence() { __builtin_amdgcn_sched_barrier(0); }
// A use of a wave-uniform value that emits no instruction: makes the compiler place its
// "scalar loads have landed" wait here rather than at the first arithmetic use.
__device__ __forceinline__ void touch_uniform(float v) { asm volatile("" ::"s"(v)); }
__device__ __forceinline__ void touch_uniform(uint32_t v) { asm volatile("" ::"s"(v)); }
// The same for a per-lane value.  Vector loads, stores and atomics share ONE in-order counter on
// this architecture, and the compiler waits for "everything" whenever control flow hides how many
// younger stores follow a load.  Touching prefetched values at a point where the count is known
// (or where nothing younger is in flight) keeps that wait from also draining recent stores.
__device__ __forceinline__ void touch_vgpr(float v) { asm volatile("" ::"v"(v)); }
__device__ __forceinline__ void touch_vgpr(bf16_t v) { asm volatile("" ::"v"((uint32_t)v)); }

// One dword of record `idx` of a row tensor (REC_BYTES per record) through the scalar cache.  Its
// only purpose is to pull the record's 64-byte line into the scalar cache well before the scan
// asks for it; the value itself is discarded (pass it to touch_uniform before the next barrier).
template <int REC_BYTES>
__device__ __forceinline__ uint32_t ld_touch(const void* p, size_t idx) {
  return *const_as<uint32_t>(static_cast<const char*>(p) + ((idx * REC_BYTES) & ~(size_t)3));
}

// Warm the scalar cache with the B_t/C_t lines of the NW state rows starting at record `row`
// (row stride L records) for one tile of TT timesteps: one dword per 64-byte line (rows of real fp32 records
// have 16 steps per line, of complex ones 8 = TG).
template <int NW, int REC_BYTES, int TT = T>
struct TileWarm {
  static constexpr int STEP = (64 / REC_BYTES > TG) ? 64 / REC_BYTES : TG;   // records between touches
  static constexpr int NTOUCH = (TT + STEP - 1) / STEP;                       // touches per row
  uint32_t v[2 * NW * NTOUCH];
  __device__ __forceinline__ void issue(const void* gB, const void* gC, size_t row, int L) {
#pragma unroll
    for (int k = 0; k < NW; ++k)
#pragma unroll
      for (int g = 0; g < NTOUCH; ++g) {
        v[(2 * k) * NTOUCH + g] = ld_touch<REC_BYTES>(gB, row + (size_t)k * L + g * STEP);
        v[(2 * k + 1) * NTOUCH + g] = ld_touch<REC_BYTES>(gC, row + (size_t)k * L + g * STEP);
      }
  }
  __device__ __forceinline__ void retire() {
#pragma unroll
    for (int i = 0; i < 2 * NW * NTOUCH; ++i) touch_uniform(v[i]);
  }
};

// ---- sums and moves across the four 16-lane rows of a wavefront (lane = 16 g + c) on the vector ALU.  gfx950 swaps
// rows between two registers in one instruction (v_permlane16_swap: rows 1 and 3 of the first with rows 0 and 2 of
// the second; v_permlane32_swap: the upper half of the first with the lower half of the second), so none of these
// takes the LDS round trip of a lane shuffle (ds_bpermute), and the scans take two dependent steps instead of three.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void rows_swap16(float& a, float& b) {
  const u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void rows_swap32(float& a, float& b) {
  const u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}
// x = [x0 x1 x2 x3] by rows.  incl: row g gets x0 + .. + xg; tot: every row gets x0 + x1 + x2 + x3.
__device__ __forceinline__ void rows_prefix(float x, int g, float* incl, float* tot) {
  float a = x, b = x;
  rows_swap16(a, b);                              // a = [x0 x0 x2 x2], b = [x1 x1 x3 x3]
  const float pair = a + b;                       // [x0+x1, x0+x1, x2+x3, x2+x3]
  float c = pair, d = pair;
  rows_swap32(c, d);                              // c = x0+x1 in every row, d = x2+x3
  float y = (g & 1) ? pair : x;
  if (g >= 2) y += c;
  *incl = y; *tot = c + d;
}
// incl: row g gets xg + .. + x3
__device__ __forceinline__ void rows_suffix(float x, int g, float* incl, float* tot) {
  float a = x, b = x;
  rows_swap16(a, b);
  const float pair = a + b;
  float c = pair, d = pair;
  rows_swap32(c, d);
  float y = (g & 1) ? x : pair;
  if (g < 2) y += d;
  *incl = y; *tot = c + d;
}
__device__ __forceinline__ float rows_sum(float x) {
  float a = x, b = x;
  rows_swap16(a, b);
  float c = a + b, d = c;
  rows_swap32(c, d);
  return c + d;
}
// the value of row 3 (row 0) of the same column, in every row
__device__ __forceinline__ float rows_last(float x) {
  float c = x, d = x;
  rows_swap32(c, d);                              // d = [x2 x3 x2 x3]
  float a = d, b = d;
  rows_swap16(a, b);                              // b = [x3 x3 x3 x3]
  return b;
}
__device__ __forceinline__ float rows_first(float x) {
  float c = x, d = x;
  rows_swap32(c, d);                              // c = [x0 x1 x0 x1]
  float a = c, b = c;
  rows_swap16(a, b);                              // a = [x0 x0 x0 x0]
  return a;
}

// DPP moves inside a row of 16 lanes (every lane has a source for the patterns used here)
template <int CTRL>
__device__ __forceinline__ float dpp_perm(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// Sums over the 64 lanes of 16 values per lane on the vector ALU alone (35 instructions, no LDS): lane (g, c) returns
// the total of value 4 (c % 4) + g.  Two rounds of row swaps fold the four rows - 16 values, 8, 4: row g of q[j]
// holds value 4 j + g summed over the rows -; two transposing steps inside the quads leave q[lane % 4]'s quad sums,
// and two rotations by 4 and 8 lanes add the four quads of the row.
__device__ __forceinline__ float lanes_sum16(const float (&v)[16], int lane) {
  float q[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float a0 = v[4 * j], b0 = v[4 * j + 1], a1 = v[4 * j + 2], b1 = v[4 * j + 3];
    rows_swap16(a0, b0);
    rows_swap16(a1, b1);
    float c = a0 + b0, d = a1 + b1;
    rows_swap32(c, d);
    q[j] = c + d;
  }
  const bool b0 = lane & 1, b1 = lane & 2;
  const float r01 = (b0 ? q[1] : q[0]) + dpp_perm<0xB1>(b0 ? q[0] : q[1]);   // quad_perm:[1,0,3,2]
  const float r23 = (b0 ? q[3] : q[2]) + dpp_perm<0xB1>(b0 ? q[2] : q[3]);
  float r = (b1 ? r23 : r01) + dpp_perm<0x4E>(b1 ? r01 : r23);               // quad_perm:[2,3,0,1]
  r += dpp_perm<0x124>(r);                                                    // row_ror:4
  r += dpp_perm<0x128>(r);                                                    // row_ror:8
  return r;
}

// ---- staging geometry: a thread owns runs of FOUR consecutive timesteps of one channel row, so a
// tile row of TT timesteps is covered by TT/4 neighbouring lanes with 16-byte accesses.
template <int NT, int TT>
struct StageGeom {
  static constexpr int TPR = TT / 4;                        // threads per channel row
  static constexpr int RW = 64 / TPR;                       // channel rows covered by one wavefront
  static constexpr int RP = NT / TPR;                       // channel rows covered per pass
  static constexpr int PASS = (CH + RP - 1) / RP;           // passes over the tile (1 if RP >= CH)
};

// Four consecutive raw input elements, kept exactly as loaded (no arithmetic may touch a loaded
// register before the tile is collected, or the wait for the load moves up to the load).
template <typename Tin> struct Quad;
template <> struct Quad<float> {
  float4 v;
  __device__ __forceinline__ float get(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
  __device__ __forceinline__ void touch() const { touch_vgpr(v.x); touch_vgpr(v.y); touch_vgpr(v.z); touch_vgpr(v.w); }
  __device__ __forceinline__ void zero() { v = make_float4(0.f, 0.f, 0.f, 0.f); }
  // vec: one 16-byte load at element offset o (caller guarantees alignment and range);
  // otherwise four element loads at o + idx[i].
  __device__ __forceinline__ void load(const float* __restrict__ p, size_t o, bool vec, const int (&idx)[4]) {
    if (vec) v = *reinterpret_cast<const float4*>(p + o);
    else v = make_float4(p[o + idx[0]], p[o + idx[1]], p[o + idx[2]], p[o + idx[3]]);
  }
};
template <> struct Quad<bf16_t> {
  uint2 v;
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = (i < 2) ? v.x : v.y;
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  __device__ __forceinline__ void touch() const { touch_vgpr(__uint_as_float(v.x)); touch_vgpr(__uint_as_float(v.y)); }
  __device__ __forceinline__ void zero() { v = make_uint2(0u, 0u); }
  __device__ __forceinline__ void load(const bf16_t* __restrict__ p, size_t o, bool vec, const int (&idx)[4]) {
    if (vec) v = *reinterpret_cast<const uint2*>(p + o);
    else v = make_uint2((uint32_t)p[o + idx[0]] | ((uint32_t)p[o + idx[1]] << 16),
                        (uint32_t)p[o + idx[2]] | ((uint32_t)p[o + idx[3]] << 16));
  }
};

// Four consecutive float32 outputs at element offset o: one 16-byte store when `vec`, else
// element stores for the timesteps < nvalid.
__device__ __forceinline__ void store4(float* __restrict__ p, size_t o, const float (&x)[4], bool vec, int nvalid) {
  if (vec && nvalid >= 4) {
    *reinterpret_cast<float4*>(p + o) = make_float4(x[0], x[1], x[2], x[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nvalid) p[o + i] = x[i];
  }
}

typedef float f4 __attribute__((ext_vector_type(4)));

// sin and cos without the large-argument branch: the caller keeps |x| below ~150.
__device__ __forceinline__ void sincos_small(float x, float* sn, float* cs) {
  const float kf = rintf(x * 0.636619772367581343f);
  float r = fmaf(-kf, 1.57079637050628662109375f, x);
  r = fmaf(-kf, -4.37113900018624283e-8f, r);
  const float r2 = r * r;
  float ps = fmaf(-1.9515295891e-4f, r2, 8.3321608736e-3f);
  ps = fmaf(ps, r2, -1.6666654611e-1f);
  const float s = fmaf(r * r2, ps, r);
  float pc = fmaf(2.443315711809948e-5f, r2, -1.388731625493765e-3f);
  pc = fmaf(pc, r2, 4.166664568298827e-2f);
  const float c = fmaf(r2 * r2, pc, fmaf(-0.5f, r2, 1.0f));
  const int q = (int)kf;
  const float s1 = (q & 1) ? c : s;
  const float c1 = (q & 1) ? s : c;
  *sn = (q & 2) ? -s1 : s1;
  *cs = ((q + 1) & 2) ? -c1 : c1;
}

// The same through the hardware's sine and cosine (arguments in revolutions): the argument is first reduced
// to a remainder of at most half a turn in two steps, as above, so what the units see is accurate to a rounding.
__device__ __forceinline__ void sincos_small_hw(float x, float* sn, float* cs) {
  const float kf = rintf(x * 0.159154943091895336f);
  float r = fmaf(-kf, 6.283185482025146484375f, x);
  r = fmaf(-kf, -1.74845560007449e-7f, r);
  const float t = r * 0.159154943091895336f;
  *sn = __builtin_amdgcn_sinf(t);
  *cs = __builtin_amdgcn_cosf(t);
}

__device__ __forceinline__ void touch4(const f4& v) { touch_vgpr(v[0]); touch_vgpr(v[1]); touch_vgpr(v[2]); touch_vgpr(v[3]); }

// Sum `v` over the lanes of each aligned group of 32 lanes; result valid in every lane.
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
  for (int o = 16; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

}  // namespace aussm
