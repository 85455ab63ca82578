// Forward core scan for the three variants (adaptive-unitary, complex, real/S6).
//
// Reference semantics: extension-cpp/extension_cpp/ops.py:215-223 (unitary loop),
// :270-291 (complex loop), :349-356 (real loop) and the selective-scan call at
// ai-modules/wavesAI/model/aussm.py:791-802.
#pragma once
#include "scan_common.h"

namespace aussm {


// VAR: variant.  NW: states per wavefront.  NT: threads per workgroup.  Tin: float or bf16_t (u, delta).
// Tbc: type of B_t / C_t (bf16 rows cost scalar-ALU conversions in the scan; the complex and real entry
// points convert them to float once per call instead).
template <int VAR, int NW, int NT, typename Tin, typename Tbc = Tin>
__global__ __launch_bounds__(NT) void core_fwd_kernel(const FwdArgs p) {
  constexpr int C = (VAR == VAR_REAL) ? 1 : 2;   // floats per state
  constexpr int NWV = NT / 64;                   // wavefronts per workgroup
  using SG = StageGeom<NT, T>;                   // staging: runs of 4 timesteps per thread
  constexpr int PASS = SG::PASS;

  __shared__ float4 s_in[T * TS];                // per (t, channel): unitary/complex (Re a, Im a, delta*u, -)
                                                 //                   real            (delta, delta*u, -, -)
  constexpr int TSP = CH + 2;                    // row stride of the partial slabs (conflict-free both ways)
  __shared__ float s_part[NWV * T * TSP];        // per wavefront partial read-outs  sum_n Re(C h)

  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  // vb: (batch, segment) pair of a launch that is split along the sequence (p.ns segments of p.L
  // steps, the last one possibly shorter), else the batch element itself
  const int vb = wg / p.ncg, d0 = (wg % p.ncg) * CH;
  const int b = vb / p.ns, sg = vb - b * p.ns;
  const int lbeg = sg * p.L, ld = p.ld;
  const int N = p.N, D = p.D;
  const int L = (ld - lbeg < p.L) ? ld - lbeg : p.L;      // steps of this segment
  const int n0 = wave * NW;
  const bool active = n0 < N;                    // wave-uniform
  const int d = d0 + lane;
  const bool dok = d < D;

  // u and delta may be shared by p.urep consecutive batch elements (tensors [B / urep, D, L]): every
  // address below is formed for batch element b, so their base steps back by the difference
  const size_t uback = (size_t)(b - b / p.urep) * p.D * ld;
  const Tin* __restrict__ gu = static_cast<const Tin*>(p.u) - uback;
  const Tin* __restrict__ gdl = static_cast<const Tin*>(p.delta) - uback;
  const Tbc* __restrict__ gB = static_cast<const Tbc*>(p.Bm);
  const Tbc* __restrict__ gC = static_cast<const Tbc*>(p.Cm);

  // ---- scan-side state (lane == channel)
  float hr[NW], hi[NW], a2[NW];
#pragma unroll
  for (int k = 0; k < NW; ++k) {
    const int n = n0 + k;
    hr[k] = 0.f; hi[k] = 0.f; a2[k] = 0.f;
    if (dok && n < N) {
      if (p.h0) {
        const size_t o = (((size_t)vb * D + d) * N + n) * C;
        hr[k] = p.h0[o];
        if (C == 2) hi[k] = p.h0[o + C - 1];
      }
      if (VAR == VAR_REAL) a2[k] = p.A[(size_t)d * N + n] * LOG2E;
    }
  }

  // ---- staging-side mapping: a thread owns 4 consecutive timesteps (t0..t0+3) of PASS channel rows
  // (inside a wavefront the row index runs fastest: the 64 lanes cover RW rows x TPR runs, which
  // is the same set of 128-byte row segments for the memory system and conflict-free in LDS)
  const int t0 = 4 * (lane / SG::RW), row0 = wave * SG::RW + lane % SG::RW;
  // Raw inputs travel through two register sets: `rdy` holds the tile that is staged next and
  // `fly` the tile after it, whose loads are still in flight.  Loads are issued TWO tiles ahead
  // (the memory latency is longer than one tile's scan) and collected one tile later, right
  // after a barrier, where the shared load/store counter has nothing recent to drain.
  struct RawTile { Quad<Tin> u[PASS], dl[PASS]; Quad<float> th[PASS], rho[PASS], z[PASS]; };
  RawTile rdy, fly;
  float dsk[PASS], dbias[PASS];
  size_t goff[PASS];
  int srow[PASS];
  bool rowok[PASS], inrow[PASS];
#pragma unroll
  for (int k = 0; k < PASS; ++k) {
    srow[k] = row0 + k * SG::RP;
    inrow[k] = srow[k] < CH;                     // this thread has a row in this pass
    const int dd = d0 + srow[k];
    rowok[k] = inrow[k] && dd < D;
    goff[k] = ((size_t)b * D + (rowok[k] ? dd : 0)) * ld + lbeg;
    dsk[k] = (p.Dskip && rowok[k]) ? p.Dskip[dd] : 0.f;
    dbias[k] = (VAR == VAR_REAL && p.delta_bias && rowok[k]) ? p.delta_bias[dd] : 0.f;
    rdy.u[k].zero(); rdy.dl[k].zero(); rdy.th[k].zero(); rdy.rho[k].zero(); rdy.z[k].zero();
    fly.u[k].zero(); fly.dl[k].zero(); fly.th[k].zero(); fly.rho[k].zero(); fly.z[k].zero();
  }
  // 16-byte accesses need every row start (L % 4 == 0) and every tensor base aligned
  auto al = [](const void* q, size_t a) { return q == nullptr || (reinterpret_cast<uintptr_t>(q) % a) == 0; };
  const bool vec = (ld % 4 == 0) && (L % 4 == 0) && al(p.u, 4 * sizeof(Tin)) && al(p.delta, 4 * sizeof(Tin)) && al(p.theta, 16) &&
                   al(p.rho, 16) && al(p.z, 16) && al(p.y, 16);

  auto load_tile = [&](RawTile& r, int l0) {
#pragma unroll
    for (int k = 0; k < PASS; ++k) {
      if (!inrow[k]) continue;
      // Unconditional loads from clamped (always valid) addresses: nothing may depend on the
      // loaded value before it is collected, or the wait for it would move up to here.
      // Out-of-range elements are zeroed when the tile is staged.
      const int ll = l0 + t0;
      int idx[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) idx[i] = (ll + i < L) ? ll + i : L - 1;
      const size_t o = goff[k] + (vec ? ((ll < L) ? ll : L - 4) : 0);
      r.u[k].load(gu, o, vec, idx);
      r.dl[k].load(gdl, o, vec, idx);
      if (VAR != VAR_REAL) r.th[k].load(p.theta, o, vec, idx);
      if (VAR == VAR_COMPLEX) r.rho[k].load(p.rho, o, vec, idx);
      if (p.z) r.z[k].load(p.z, o, vec, idx);
    }
  };
  // A use of every register of a set: the compiler puts its wait for the loads here.
  auto collect_tile = [&](RawTile& r) {
#pragma unroll
    for (int k = 0; k < PASS; ++k) {
      r.u[k].touch(); r.dl[k].touch();
      if (VAR != VAR_REAL) r.th[k].touch();
      if (VAR == VAR_COMPLEX) r.rho[k].touch();
      if (p.z) r.z[k].touch();
    }
  };
  load_tile(rdy, 0);
  collect_tile(rdy);
  if (T < L) load_tile(fly, T);

  // The scan consumes every B_t/C_t line exactly once, so each of its scalar loads would miss
  // the scalar cache and pay the full memory latency.  Instead the lines of the NEXT tile are
  // touched here, a whole tile ahead, while the vector ALUs are busy with the staging maths.
  constexpr bool WARM = NW <= 4;
  constexpr int RB = (int)sizeof(Tbc) * C;
  const bool full_group = active && n0 + NW <= N;
  TileWarm<WARM ? NW : 1, RB> warm;
  const size_t bc_row = ((size_t)b * N + n0) * ld + lbeg;   // B_t / C_t: row n0, first step of the segment
  if (WARM && full_group && T <= L) {
    warm.issue(gB, gC, bc_row, ld);
    warm.retire();
  }

  // product of the a_l over the segment (complex) or sum of the step sizes (real), kept by wavefront 0
  // of a launch that wants it (a split launch chains its segments with it)
  const bool want_tot = p.ptot != nullptr && wave == 0;   // wave-uniform
  float fr = (VAR == VAR_REAL) ? 0.f : 1.f, fi = 0.f;

  // a wavefront that owns no state never writes its slab of partial read-outs: it clears it once, so that the
  // epilogue can add the slabs of all wavefronts without asking which of them exist (the first barrier of the loop
  // orders the two)
  if (!active) {
    for (int i = lane; i < T * TSP; i += 64) s_part[wave * T * TSP + i] = 0.f;
  }

  for (int l0 = 0; l0 < L; l0 += T) {
    const bool warm_next = WARM && full_group && l0 + 2 * T <= L;
    if (warm_next) warm.issue(gB, gC, bc_row + l0 + T, ld);
    // ---- stage: convert this tile once per (channel, t) and transpose into LDS
    float yin[PASS][4], gate[PASS][4];
#pragma unroll
    for (int k = 0; k < PASS; ++k) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool ok = rowok[k] && l0 + t0 + i < L;
        const float uu = ok ? rdy.u[k].get(i) : 0.f;
        float dl = ok ? rdy.dl[k].get(i) : 0.f;
        float4 rec;
        if (VAR == VAR_REAL) {
          dl += dbias[k];
          if (p.delta_softplus) dl = softplusf_(dl);
          rec = make_float4(dl, dl * uu, 0.f, 0.f);
        } else {
          float sn, cs;
          fast_sincosf(ok ? rdy.th[k].get(i) : 0.f, &sn, &cs);
          if (VAR == VAR_COMPLEX) { const float r = expf(ok ? rdy.rho[k].get(i) : 0.f); cs *= r; sn *= r; }
          rec = make_float4(cs, sn, dl * uu, 0.f);
        }
        if (inrow[k]) s_in[(t0 + i) * TS + srow[k]] = rec;
        yin[k][i] = dsk[k] * uu;
        gate[k][i] = rdy.z[k].get(i);
      }
    }
    if (warm_next) warm.retire();
    __syncthreads();

    // ---- scan: lane == channel, sequential over the tile's timesteps
    const int tmax = (L - l0 < T) ? (L - l0) : T;
    const size_t brow = bc_row + l0;
    // fast path: a full tile and a full group of states.  (bf16 real rows need an even offset
    // so that the 8-element scalar load is 4-byte aligned.)
    const bool fast = tmax == T && n0 + NW <= N &&
                      !(VAR == VAR_REAL && sizeof(Tbc) == 2 && (ld & 1));
    float mr[NW], mi[NW];                        // state after the first half of the tile
#pragma unroll
    for (int k = 0; k < NW; ++k) { mr[k] = 0.f; mi[k] = 0.f; }
    if (active && fast) {
      // The tile is walked in groups of TG timesteps; inside a group the wavefront's states take
      // turns.  One turn = one state row x TG timesteps: its B_t and C_t values are ONE scalar
      // load each, issued a full turn ahead so the load latency hides behind the previous turn's
      // arithmetic.  The (channel, timestep) records of the next group are read from LDS a group
      // ahead for the same reason.
      float rx[TG], ry[TG], rz[TG];
#pragma unroll
      for (int t = 0; t < TG; ++t) {
        const float4 v = s_in[t * TS + lane];
        rx[t] = v.x; ry[t] = v.y; rz[t] = v.z;
      }
      if constexpr (VAR == VAR_REAL) {
        f32x8 bn = ld_r8(gB, brow), cn = ld_r8(gC, brow);
#pragma unroll
        for (int g = 0; g < T / TG; ++g) {
          float yacc[TG], nx[TG], ny[TG];
#pragma unroll
          for (int t = 0; t < TG; ++t) yacc[t] = 0.f;
          if (want_tot) {
#pragma unroll
            for (int t = 0; t < TG; ++t) fr += rx[t];
          }
#pragma unroll
          for (int k = 0; k < NW; ++k) {
            const f32x8 bc = bn, cc = cn;
            touch_uniform(bc[0]);
            touch_uniform(cc[0]);
            sched_fence();
            if (k + 1 < NW) {
              bn = ld_r8(gB, brow + (size_t)(k + 1) * ld + g * TG);
              cn = ld_r8(gC, brow + (size_t)(k + 1) * ld + g * TG);
            } else if (g + 1 < T / TG) {
              bn = ld_r8(gB, brow + (g + 1) * TG);
              cn = ld_r8(gC, brow + (g + 1) * TG);
            }
            if (k == 0 && g + 1 < T / TG) {
#pragma unroll
              for (int t = 0; t < TG; ++t) {
                const float4 v = s_in[((g + 1) * TG + t) * TS + lane];
                nx[t] = v.x; ny[t] = v.y;
              }
            }
            sched_fence();
#pragma unroll
            for (int t = 0; t < TG; ++t) {
              const float a = __builtin_amdgcn_exp2f(rx[t] * a2[k]);
              hr[k] = fmaf(a, hr[k], bc[t] * ry[t]);
              yacc[t] = fmaf(cc[t], hr[k], yacc[t]);
            }
            // (keeps the next turn's wait for its scalar loads behind this turn's arithmetic: without the fence
            // the compiler hoists it to the top of the turn, right behind the loads it waits for)
            sched_fence();
          }
#pragma unroll
          for (int t = 0; t < TG; ++t) {
            s_part[(wave * T + g * TG + t) * TSP + lane] = yacc[t];
            if (g + 1 < T / TG) { rx[t] = nx[t]; ry[t] = ny[t]; }
          }
          if (g == T / 2 / TG - 1) {
#pragma unroll
            for (int k = 0; k < NW; ++k) mr[k] = hr[k];
          }
        }
      } else {
        f32x16 bn = ld_c8(gB, brow), cn = ld_c8(gC, brow);
#pragma unroll
        for (int g = 0; g < T / TG; ++g) {
          float yacc[TG], nx[TG], ny[TG], nz[TG];
#pragma unroll
          for (int t = 0; t < TG; ++t) yacc[t] = 0.f;
          if (want_tot) {
#pragma unroll
            for (int t = 0; t < TG; ++t) {
              const float nr = fmaf(fr, rx[t], -fi * ry[t]);
              fi = fmaf(fr, ry[t], fi * rx[t]);
              fr = nr;
            }
          }
#pragma unroll
          for (int k = 0; k < NW; ++k) {
            const f32x16 bc = bn, cc = cn;
            touch_uniform(bc[0]);
            touch_uniform(cc[0]);
            sched_fence();
            if (k + 1 < NW) {
              bn = ld_c8(gB, brow + (size_t)(k + 1) * ld + g * TG);
              cn = ld_c8(gC, brow + (size_t)(k + 1) * ld + g * TG);
            } else if (g + 1 < T / TG) {
              bn = ld_c8(gB, brow + (g + 1) * TG);
              cn = ld_c8(gC, brow + (g + 1) * TG);
            }
            if (k == 0 && g + 1 < T / TG) {
#pragma unroll
              for (int t = 0; t < TG; ++t) {
                const float4 v = s_in[((g + 1) * TG + t) * TS + lane];
                nx[t] = v.x; ny[t] = v.y; nz[t] = v.z;
              }
            }
            sched_fence();
#pragma unroll
            for (int t = 0; t < TG; ++t) {
              const float nr = fmaf(rx[t], hr[k], fmaf(-ry[t], hi[k], bc[2 * t] * rz[t]));
              const float ni = fmaf(rx[t], hi[k], fmaf(ry[t], hr[k], bc[2 * t + 1] * rz[t]));
              hr[k] = nr; hi[k] = ni;
              yacc[t] = fmaf(cc[2 * t], nr, yacc[t]);
              yacc[t] = fmaf(-cc[2 * t + 1], ni, yacc[t]);
            }
            sched_fence();
          }
#pragma unroll
          for (int t = 0; t < TG; ++t) {
            s_part[(wave * T + g * TG + t) * TSP + lane] = yacc[t];
            if (g + 1 < T / TG) { rx[t] = nx[t]; ry[t] = ny[t]; rz[t] = nz[t]; }
          }
          if (g == T / 2 / TG - 1) {
#pragma unroll
            for (int k = 0; k < NW; ++k) { mr[k] = hr[k]; mi[k] = hi[k]; }
          }
        }
      }
    } else if (active) {
#pragma unroll 4
      for (int t = 0; t < tmax; ++t) {
        const float4 v = s_in[t * TS + lane];
        float yacc = 0.f;
        if (want_tot) {
          if (VAR == VAR_REAL) {
            fr += v.x;
          } else {
            const float nr = fmaf(fr, v.x, -fi * v.y);
            fi = fmaf(fr, v.y, fi * v.x);
            fr = nr;
          }
        }
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          if (n0 + k < N) {                      // wave-uniform
            const size_t bi = brow + (size_t)k * ld + t;
            if (VAR == VAR_REAL) {
              const float bv = ld_r(gB, bi), cv = ld_r(gC, bi);
              const float a = __builtin_amdgcn_exp2f(v.x * a2[k]);
              hr[k] = fmaf(a, hr[k], bv * v.y);
              yacc = fmaf(cv, hr[k], yacc);
            } else {
              const float2 bv = ld_c(gB, bi), cv = ld_c(gC, bi);
              const float nr = fmaf(v.x, hr[k], fmaf(-v.y, hi[k], bv.x * v.z));
              const float ni = fmaf(v.x, hi[k], fmaf(v.y, hr[k], bv.y * v.z));
              hr[k] = nr; hi[k] = ni;
              yacc = fmaf(cv.x, nr, yacc);
              yacc = fmaf(-cv.y, ni, yacc);
            }
          }
        }
        s_part[(wave * T + t) * TSP + lane] = yacc;
        if (t == T / 2 - 1) {
#pragma unroll
          for (int k = 0; k < NW; ++k) { mr[k] = hr[k]; mi[k] = hi[k]; }
        }
      }
    }
    __syncthreads();

    // ---- the tile's vector-memory traffic, in ONE burst.  Loads, stores and atomics share one
    // in-order completion counter and the compiler can only wait for "everything": so the wait
    // comes first, when every outstanding operation (the loads of tile l0+T and the stores of
    // the previous tile) is a whole tile old, then the new loads, then this tile's stores.
    if (l0 + T < L) { collect_tile(fly); rdy = fly; }      // tile l0+T has arrived
    sched_fence();
    if (l0 + 2 * T < L) load_tile(fly, l0 + 2 * T);        // request tile l0+2T
    sched_fence();

    // ---- epilogue: add the wavefronts' partial read-outs, skip term and gate; coalesced store
    if (p.y) {
      // all partial sums are fetched before the first add, so their LDS latencies overlap
      float pv[PASS][4][NWV];
#pragma unroll
      for (int k = 0; k < PASS; ++k)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int w = 0; w < NWV; ++w)
            pv[k][i][w] = (SG::RP == CH || inrow[k]) ? s_part[(w * T + t0 + i) * TSP + srow[k]] : 0.f;
      sched_fence();
#pragma unroll
      for (int k = 0; k < PASS; ++k) {
        float acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[i] = yin[k][i];
#pragma unroll
          for (int w = 0; w < NWV; ++w) acc[i] += pv[k][i][w];
          if (p.z) acc[i] *= siluf_(gate[k][i]);
        }
        const int nvalid = L - (l0 + t0);
        if (rowok[k] && nvalid > 0) store4(p.y, goff[k] + l0 + t0, acc, vec, nvalid);
      }
    }
    // ---- checkpoint at the end of every ck-step block (and at the end of the sequence).
    // ck is a multiple of the tile, or half a tile (then the mid-tile state saved by the scan
    // is written as well).
    if (p.hck && active && dok) {
      auto put = [&](int kb, const float (&xr)[NW], const float (&xi)[NW]) {
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          const int n = n0 + k;
          if (n < N) {
            const size_t o = ((((size_t)b * p.nck + sg * (p.L / p.ck) + kb) * N + n) * C) * D + d;
            p.hck[o] = xr[k];
            if (C == 2) p.hck[o + D] = xi[k];
          }
        }
      };
      if (p.ck == T / 2) {
        if (tmax > T / 2) put(l0 / (T / 2), mr, mi);
        put((l0 + tmax - 1) / (T / 2), hr, hi);
      } else if (((l0 + T) % p.ck) == 0 || l0 + T >= L) {
        put(l0 / p.ck, hr, hi);
      }
    }
    // No third barrier: the next stage only writes s_in (all scan reads of it are behind the
    // barrier above) and the next scan writes s_part only after the next barrier, by which time
    // every wavefront has finished this epilogue.
  }

  if (want_tot && dok) {
    p.ptot[((size_t)vb * D + d) * 2] = fr;
    p.ptot[((size_t)vb * D + d) * 2 + 1] = fi;
  }
  if (p.hL && active && dok) {
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const int n = n0 + k;
      if (n < N) {
        const size_t o = (((size_t)vb * D + d) * N + n) * C;
        p.hL[o] = hr[k];
        if (C == 2) p.hL[o + 1] = hi[k];
      }
    }
  }
}

}  // namespace aussm
