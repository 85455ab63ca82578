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

namespace aussm {

constexpr int CH = 64;        // channels per workgroup == lanes per wavefront
constexpr int T = 32;         // timesteps per staged tile (AUSSM_TILE)
constexpr int TS = CH + 1;    // padded row stride of [t][channel] LDS tiles (bank-conflict free)
constexpr int NXCD = 8;       // accelerator complex dies, each with a private L2

enum { VAR_UNITARY = 0, VAR_COMPLEX = 1, VAR_REAL = 2 };

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

// Sum `v` over the lanes of each aligned group of 32 lanes; result valid in every lane.
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
  for (int o = 16; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

}  // namespace aussm
