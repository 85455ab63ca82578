// Reverse scan (gradients) of the adaptive-unitary core scan.
//
// The recurrence h_l = a_l h_{l-1} + B_l w_l with |a_l| = 1 is invertible without loss:
// h_{l-1} = conj(a_l) (h_l - B_l w_l).  The backward pass therefore walks the sequence right to
// left ONCE, regenerating the states from the final state (re-synchronised at every checkpoint
// written by the forward pass) while it propagates the adjoint state g_l = dLoss/dh_l:
//     g_l      = conj(C_l) dy_l + conj(a_{l+1}) g_{l+1}
//     dC_l[n]  = sum_d dy_l conj(h_l)            dB_l[n] = sum_d w_l g_l          (w = delta u, real)
//     dw_l     = sum_n Re(conj(B_l) g_l)         du = dw delta + D dy,  ddelta = dw u
//     dtheta_l = -sum_n Im(conj(g_l) a_l h_{l-1})
// Gradient formulas: the recurrence form of
// extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_backward.cu:154-403.
//
// dB/dC are sums over channels, i.e. over the lanes of a wavefront and over the workgroups of
// one batch element.  The lane sum is an LDS transpose (every lane writes its products as a row,
// then reads one column), the sum over workgroups uses float atomics on the output.
// dw and dtheta are sums over states, i.e. over the wavefronts of a workgroup: every wavefront
// writes its partial sums to its own LDS slab and the epilogue adds the slabs in a fixed order
// (LDS float atomics were measured to be several times slower than this).
#pragma once
#include "scan_common.h"

namespace aussm {


constexpr int RED_COLS = 4 * TG;        // products per lane per turn: TG x (dB re, dB im) then TG x (dC re, dC im)
constexpr int RED_RS = RED_COLS + 4;    // padded row stride (floats), keeps rows 16-byte aligned

// Column sums over the lanes of a wavefront through an LDS transpose, split in two halves so that
// the LDS latency overlaps the next turn's arithmetic:
//   issue()   every lane writes its RED_COLS products as a row, then starts reading column
//             (lane % 32) over the 32 rows of its half of the wavefront;
//   finish()  adds the 32 values.  Lanes c and c + 32 then hold the two half sums of column c.
// LDS operations of one wavefront execute in order, so the column reads see the row writes of
// the other lanes, and a later issue() cannot overtake these reads.
struct LaneTranspose {
  float v[32];
  __device__ __forceinline__ void issue(const float (&vals)[RED_COLS], float* red, int lane) {
    float4* row = reinterpret_cast<float4*>(red + lane * RED_RS);
#pragma unroll
    for (int j = 0; j < RED_COLS / 4; ++j)
      row[j] = make_float4(vals[4 * j], vals[4 * j + 1], vals[4 * j + 2], vals[4 * j + 3]);
    __builtin_amdgcn_wave_barrier();
    const float* colp = red + ((lane >> 5) * 32) * RED_RS + (lane & 31);
#pragma unroll
    for (int i = 0; i < 32; ++i) v[i] = colp[i * RED_RS];
    sched_fence();
  }
  __device__ __forceinline__ float finish() {
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1)
#pragma unroll
      for (int i = 0; i < s; ++i) v[i] += v[i + s];
    return v[0];
  }
};

// TT: timesteps per staged tile (16 or 32; the checkpoint interval is a multiple of 32 either way).
template <int NW, int NT, int TT, typename Tin>
__global__ __launch_bounds__(NT) void unitary_bwd_kernel(const UniBwdArgs p) {
  constexpr int NWV = NT / 64;
  constexpr int E = CH * TT / NT;
  constexpr int RSTEP = NT / TT;
  constexpr int NGRP = TT / TG;
  static_assert(RED_COLS == 32, "the lane transpose assumes 32 columns");
  static_assert(E >= 1 && NGRP >= 1, "tile too small for this workgroup size");

  __shared__ float4 s_in[TT * TS];                         // (Re a, Im a, delta*u, dy) per (t, channel)
  __shared__ float2 s_part[NWV * TT * TS];                 // per wavefront partial (dw, dtheta)
  __shared__ __align__(16) float s_red[NWV * 64 * RED_RS]; // lane-transpose scratch, one slab per wavefront

  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  // vb: (batch, segment) pair of a launch that is split along the sequence (p.ns segments of p.L steps,
  // the last one possibly shorter; p.ld = row stride of the [.., L] tensors), else the batch element
  const int vb = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int b = vb / p.ns, sg = vb - b * p.ns;
  const int lbeg = sg * p.L, ld = p.ld;
  const int N = p.N, D = p.D;
  const int L = (ld - lbeg < p.L) ? ld - lbeg : p.L;        // steps of this segment
  const int n0 = wave * NW;
  const bool active = n0 < N;
  const bool full_group = active && n0 + NW <= N;
  const int d = d0 + lane;
  const bool dok = d < D;

  // u and delta may be shared by p.urep consecutive batch elements (tensors [B / urep, D, L]): every
  // address below is formed for batch element b, so their base steps back by the difference
  const size_t uback = (size_t)(b - b / p.urep) * p.D * ld;
  const Tin* __restrict__ gu = static_cast<const Tin*>(p.u) - uback;
  const Tin* __restrict__ gdl = static_cast<const Tin*>(p.delta) - uback;
  const Tin* __restrict__ gB = static_cast<const Tin*>(p.Bm);
  const Tin* __restrict__ gC = static_cast<const Tin*>(p.Cm);
  float* red = s_red + wave * 64 * RED_RS;
  float2* part = s_part + wave * TT * TS;
  // lane -> element of the (row, 8 timesteps) output block of a turn: columns 0..15 are dB
  // (re, im interleaved), 16..31 dC; both halves of the wavefront add their half sum.
  // The sums over the channels of a turn's dB / dC products: through the LDS lane transpose, whose latency hides
  // behind the next turn, or on the vector ALU alone (`lanes_sum16`).  Measured at B=32, D=512, L=2048: with eight
  // states per wavefront (N = 64) the vector-ALU form is 10 % faster, with four or two (N = 32, 16) 2-5 % slower.
  // (With lanes_sum16: lane (g, c) holds column 4 (c % 4) + g of dB for c / 4 == 0, of dC for c / 4 == 1.)
  constexpr bool VALU_SUMS = NW >= 8;
  float* const red_dst = VALU_SUMS ? ((lane & 4) ? p.dC : p.dB) : (((lane & 31) < 2 * TG) ? p.dB : p.dC);
  const int red_off = VALU_SUMS ? 4 * (lane & 3) + (lane >> 4) : (lane & (2 * TG - 1));
  const bool red_mine = VALU_SUMS ? (lane & 8) == 0 : true;

  auto load_ck = [&](int kb, float (&xr)[NW], float (&xi)[NW]) {
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const int n = n0 + k;
      xr[k] = 0.f; xi[k] = 0.f;
      if (dok && n < N) {
        const size_t o = ((((size_t)b * p.nck + kb) * N + n) * 2) * D + d;
        xr[k] = p.hck[o];
        xi[k] = p.hck[o + D];
      }
    }
  };

  // ---- state and adjoint at the end of the segment (checkpoints are numbered along the whole sequence, a
  // segment is a whole number of checkpoint blocks, the sequence's last block may be shorter)
  float hr[NW], hi[NW], gr[NW], gi[NW];
  load_ck((lbeg + L + p.ck - 1) / p.ck - 1, hr, hi);
#pragma unroll
  for (int k = 0; k < NW; ++k) {
    const int n = n0 + k;
    gr[k] = 0.f; gi[k] = 0.f;
    if (p.dhL && dok && n < N) {
      const size_t o = (((size_t)vb * D + d) * N + n) * 2;
      gr[k] = p.dhL[o]; gi[k] = p.dhL[o + 1];
    }
  }

  // ---- staging-side mapping (lanes run along time)
  const int col = tid % TT, row0 = tid / TT;
  // Raw inputs travel through two register sets: `rdy` holds the tile that is staged next and
  // `fly` the tile after it, whose loads are still in flight.  Loads are issued TWO tiles ahead
  // and collected one tile later, right after a barrier (see the forward kernel).
  struct RawTile { Tin u[E], dl[E]; float th[E], gy[E]; };
  RawTile rdy, fly;
  float dsk[E], accD[E];
  size_t goff[E];
  bool rowok[E];
#pragma unroll
  for (int k = 0; k < E; ++k) {
    const int dd = d0 + row0 + k * RSTEP;
    rowok[k] = dd < D;
    goff[k] = ((size_t)b * D + (rowok[k] ? dd : 0)) * ld + lbeg;
    dsk[k] = (p.Dskip && rowok[k]) ? p.Dskip[dd] : 0.f;
    accD[k] = 0.f;
    fly.u[k] = fly.dl[k] = Tin(0);
    fly.th[k] = fly.gy[k] = 0.f;
  }
  auto load_tile = [&](RawTile& r, int l0) {
#pragma unroll
    for (int k = 0; k < E; ++k) {
      // unconditional loads from a clamped address; out-of-range elements are zeroed at staging
      const int ll = (l0 + col < L) ? l0 + col : L - 1;
      const size_t o = goff[k] + ll;
      r.u[k] = gu[o];
      r.dl[k] = gdl[o];
      r.th[k] = p.theta[o];
      r.gy[k] = p.dy[o];
    }
  };
  // A use of every register of a set: the compiler puts its wait for the loads here.
  auto collect_tile = [&](RawTile& r) {
#pragma unroll
    for (int k = 0; k < E; ++k) { touch_vgpr(r.u[k]); touch_vgpr(r.dl[k]); touch_vgpr(r.th[k]); touch_vgpr(r.gy[k]); }
  };

  const int ntiles = (L + TT - 1) / TT;
  load_tile(rdy, (ntiles - 1) * TT);
  collect_tile(rdy);
  if (ntiles > 1) load_tile(fly, (ntiles - 2) * TT);

  // scalar-cache warm-up of the B_t/C_t lines, one tile ahead of the scan (see the forward kernel)
  constexpr bool WARM = NW <= 4;
  constexpr int RB = (int)sizeof(Tin) * 2;
  const size_t row_base = ((size_t)b * N + n0) * ld + lbeg;
  TileWarm<WARM ? NW : 1, RB, TT> warm;
  if (WARM && full_group && ntiles * TT == L) {
    warm.issue(gB, gC, row_base + (size_t)(ntiles - 1) * TT, ld);
    warm.retire();
  }

  // a wavefront that owns no state never writes its slab of partial sums: it clears it once, so that the epilogue
  // can add the slabs of all wavefronts without asking which of them exist (the loop's first barrier orders the two)
  if (!active) {
    for (int i = lane; i < TT * TS; i += 64) part[i] = make_float2(0.f, 0.f);
  }

  for (int it = ntiles - 1; it >= 0; --it) {
    const int l0 = it * TT;
    const int tmax = (L - l0 < TT) ? (L - l0) : TT;
    const bool warm_next = WARM && full_group && it > 0;
    if (warm_next) warm.issue(gB, gC, row_base + l0 - TT, ld);

    // ---- stage
    float eu[E], edl[E], egy[E];
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const bool ok = rowok[k] && l0 + col < L;
      eu[k] = ok ? to_f32(rdy.u[k]) : 0.f;
      edl[k] = ok ? to_f32(rdy.dl[k]) : 0.f;
      egy[k] = ok ? rdy.gy[k] : 0.f;
      float sn, cs;
      fast_sincosf(ok ? rdy.th[k] : 0.f, &sn, &cs);
      s_in[col * TS + row0 + k * RSTEP] = make_float4(cs, sn, edl[k] * eu[k], egy[k]);
    }
    if (warm_next) warm.retire();
    __syncthreads();

    const size_t brow = row_base + l0;
    const bool fast = full_group && tmax == TT;
    float rres[NGRP * NW];      // finished dB/dC sums of this tile's turns (fast path)
    if (fast) {
      // ---- fast path: groups of TG timesteps right to left; inside a group the wavefront's
      // state rows take turns, each turn consuming ONE scalar load of B_t and one of C_t that
      // was issued a turn earlier.  The channel reduction of a turn's dB/dC products is started
      // at the end of the turn and collected at the end of the NEXT turn.
      float rc[TG], rs[TG], rw[TG], rg[TG];
#pragma unroll
      for (int t = 0; t < TG; ++t) {
        const float4 v = s_in[(TT - TG + t) * TS + lane];
        rc[t] = v.x; rs[t] = v.y; rw[t] = v.z; rg[t] = v.w;
      }
      f32x16 bn = ld_c8(gB, brow + (TT - TG)), cn = ld_c8(gC, brow + (TT - TG));
      LaneTranspose xp;
#pragma unroll
      for (int g = NGRP - 1; g >= 0; --g) {
        float kacc[TG], qacc[TG], nc[TG], ns[TG], nw_[TG], ng[TG];
#pragma unroll
        for (int t = 0; t < TG; ++t) { kacc[t] = 0.f; qacc[t] = 0.f; }
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          const f32x16 bc = bn, cc = cn;
          touch_uniform(bc[0]);
          touch_uniform(cc[0]);
          sched_fence();
          if (k + 1 < NW) {
            bn = ld_c8(gB, brow + (size_t)(k + 1) * ld + g * TG);
            cn = ld_c8(gC, brow + (size_t)(k + 1) * ld + g * TG);
          } else if (g > 0) {
            bn = ld_c8(gB, brow + (g - 1) * TG);
            cn = ld_c8(gC, brow + (g - 1) * TG);
          }
          if (k == 0 && g > 0) {
#pragma unroll
            for (int t = 0; t < TG; ++t) {
              const float4 v = s_in[((g - 1) * TG + t) * TS + lane];
              nc[t] = v.x; ns[t] = v.y; nw_[t] = v.z; ng[t] = v.w;
            }
          }
          sched_fence();
          float vals[RED_COLS];
#pragma unroll
          for (int t = TG - 1; t >= 0; --t) {
            const float br = bc[2 * t], bi = bc[2 * t + 1], cr = cc[2 * t], ci = cc[2 * t + 1];
            const float w = rw[t], gy = rg[t], cs = rc[t], sn = rs[t];
            gr[k] = fmaf(cr, gy, gr[k]);
            gi[k] = fmaf(-ci, gy, gi[k]);
            vals[2 * t] = w * gr[k];
            vals[2 * t + 1] = w * gi[k];
            vals[2 * TG + 2 * t] = gy * hr[k];
            vals[2 * TG + 2 * t + 1] = -gy * hi[k];
            kacc[t] = fmaf(br, gr[k], kacc[t]);
            kacc[t] = fmaf(bi, gi[k], kacc[t]);
            const float pr = fmaf(-br, w, hr[k]);
            const float pi = fmaf(-bi, w, hi[k]);
            qacc[t] = fmaf(gi[k], pr, qacc[t]);
            qacc[t] = fmaf(-gr[k], pi, qacc[t]);
            hr[k] = fmaf(cs, pr, sn * pi);
            hi[k] = fmaf(cs, pi, -sn * pr);
            const float tg = fmaf(cs, gr[k], sn * gi[k]);
            gi[k] = fmaf(cs, gi[k], -sn * gr[k]);
            gr[k] = tg;
          }
          sched_fence();
          if constexpr (VALU_SUMS) {
            // the turn's 16 dB and 16 dC products summed over the channels on the vector ALU
            float hb[16], hc[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) { hb[j] = vals[j]; hc[j] = vals[16 + j]; }
            const float sb = lanes_sum16(hb, lane), sc = lanes_sum16(hc, lane);
            rres[g * NW + k] = (lane & 4) ? sc : sb;
          } else {
            // collect the previous turn's sums (turn (g, k-1), or (g+1, NW-1) across a group)
            if (k > 0) rres[g * NW + k - 1] = xp.finish();
            else if (g < NGRP - 1) rres[(g + 1) * NW + NW - 1] = xp.finish();
            xp.issue(vals, red, lane);
          }
        }
#pragma unroll
        for (int t = 0; t < TG; ++t) {
          part[(g * TG + t) * TS + lane] = make_float2(kacc[t], qacc[t]);
          if (g > 0) { rc[t] = nc[t]; rs[t] = ns[t]; rw[t] = nw_[t]; rg[t] = ng[t]; }
        }
      }
      if constexpr (!VALU_SUMS) rres[NW - 1] = xp.finish();   // the last turn was (g = 0, k = NW-1)
    } else if (active) {
      // ---- general path (ragged tile or partial state group): one timestep at a time
      for (int t = tmax - 1; t >= 0; --t) {
        const float4 v = s_in[t * TS + lane];
        const float cs = v.x, sn = v.y, w = v.z, gy = v.w;
        float kacc = 0.f, qacc = 0.f;
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          float2 bv = make_float2(0.f, 0.f), cv = make_float2(0.f, 0.f);
          const bool nok = n0 + k < N;
          const size_t bi = brow + (size_t)k * ld + t;
          if (nok) { bv = ld_c(gB, bi); cv = ld_c(gC, bi); }
          gr[k] = fmaf(cv.x, gy, gr[k]);
          gi[k] = fmaf(-cv.y, gy, gi[k]);
          float vals[RED_COLS];
#pragma unroll
          for (int j = 0; j < RED_COLS; ++j) vals[j] = 0.f;
          vals[0] = w * gr[k];
          vals[1] = w * gi[k];
          vals[2] = gy * hr[k];
          vals[3] = -gy * hi[k];
          kacc = fmaf(bv.x, gr[k], kacc);
          kacc = fmaf(bv.y, gi[k], kacc);
          const float pr = fmaf(-bv.x, w, hr[k]);
          const float pi = fmaf(-bv.y, w, hi[k]);
          qacc = fmaf(gi[k], pr, qacc);
          qacc = fmaf(-gr[k], pi, qacc);
          hr[k] = fmaf(cs, pr, sn * pi);
          hi[k] = fmaf(cs, pi, -sn * pr);
          const float tg = fmaf(cs, gr[k], sn * gi[k]);
          gi[k] = fmaf(cs, gi[k], -sn * gr[k]);
          gr[k] = tg;
          LaneTranspose xs;
          xs.issue(vals, red, lane);
          const float tot = xs.finish();
          if (nok && (lane & 31) < 4) {
            float* dst = ((lane & 31) < 2) ? p.dB : p.dC;
            atomicAdd(dst + 2 * bi + (lane & 1), tot);
          }
        }
        part[t * TS + lane] = make_float2(kacc, qacc);
      }
    }
    __syncthreads();

    // ---- the tile's vector-memory traffic, in ONE burst.  Loads, stores and atomics share one
    // in-order completion counter and the compiler can only wait for "everything": so the wait
    // comes first, when every outstanding operation is a whole tile old, then the new loads,
    // then this tile's atomics and stores.
    // (re-synchronise the regenerated state with the forward pass's checkpoint first, so that
    // its rare load is part of the same wait)
    if (active && l0 > 0 && (l0 % p.ck) == 0) {
      load_ck((lbeg + l0) / p.ck - 1, hr, hi);
#pragma unroll
      for (int k = 0; k < NW; ++k) { touch_vgpr(hr[k]); touch_vgpr(hi[k]); }
    }
    if (it > 0) { collect_tile(fly); rdy = fly; }          // tile it-1 has arrived
    sched_fence();
    if (it > 1) load_tile(fly, l0 - 2 * TT);               // request tile it-2
    sched_fence();
    if (fast) {
#pragma unroll
      for (int g = 0; g < NGRP; ++g)
#pragma unroll
        for (int k = 0; k < NW; ++k)
          if (red_mine) atomicAdd(red_dst + 2 * (brow + (size_t)k * ld + g * TG) + red_off, rres[g * NW + k]);
    }

    // ---- epilogue: channel-wise gradients, coalesced along time
    // all partial sums are fetched before the first add, so their LDS latencies overlap
    float2 pv[E][NWV];
#pragma unroll
    for (int k = 0; k < E; ++k)
#pragma unroll
      for (int w = 0; w < NWV; ++w)
        pv[k][w] = s_part[(w * TT + col) * TS + row0 + k * RSTEP];   // (wavefronts without states hold zeros)
    sched_fence();
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const int ll = l0 + col;
      float kk = 0.f, qq = 0.f;
#pragma unroll
      for (int w = 0; w < NWV; ++w) { kk += pv[k][w].x; qq += pv[k][w].y; }
      if (rowok[k] && ll < L) {
        const size_t o = goff[k] + ll;
        p.du[o] = fmaf(kk, edl[k], dsk[k] * egy[k]);
        p.ddelta[o] = kk * eu[k];
        p.dtheta[o] = qq;
        accD[k] = fmaf(egy[k], eu[k], accD[k]);
      }
    }
    // No barrier here: the next stage writes only s_in (its readers are behind the barrier above)
    // and the next scan writes s_part only after the next barrier.
  }

  if (p.dh0 && active && dok) {
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const int n = n0 + k;
      if (n < N) {
        const size_t o = (((size_t)vb * D + d) * N + n) * 2;
        p.dh0[o] = gr[k]; p.dh0[o + 1] = gi[k];
      }
    }
  }
  if (p.dD) {
    // the TT lanes that share a channel row are consecutive: sum them with xor-shuffles
#pragma unroll
    for (int k = 0; k < E; ++k) {
      float s = accD[k];
#pragma unroll
      for (int o = TT / 2; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
      if (col == 0 && rowok[k]) atomicAdd(p.dD + d0 + row0 + k * RSTEP, s);
    }
  }
}

}  // namespace aussm
