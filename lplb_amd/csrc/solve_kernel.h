// LP solver, device side: one wave64 per EP group (or four small LPs per wave), no
// workgroup barriers.  Included by the kernels that run it (solve.hip, plan.hip).
//
// Problem (reference: minilp.cu:199-293).  For a group of G ranks with D replica
// slots each, n = G*D replica edges.  Edge j = (k, d) carries the normalised
// token count w_j of rank k's d-th replicated expert set; a copy lives on the
// rank i with r2o[i][d] == k.  Variables: x_o[j] (share kept on k), x_r[j] (share
// sent to the copy), slack s_i per rank, the maximum load t and a Big-M
// artificial x_M.  Constraints: per rank i,
//     sum_{j on i} w_j x_o[j] + sum_{j copied to i} w_j x_r[j] + s_i - t + m_i x_M = b_i,
// per edge x_o[j] + x_r[j] - x_M = 1; minimise t + 1000 x_M.  m makes x = 1 feasible.
//
// Method (reference: minilp.cu:331-400): a fixed number of primal affine-scaling
// steps x <- x (1 - alpha d), d = x (c - A^T w), (A X^2 A^T) w = A X^2 c,
// alpha = 0.999 / d_max, then a feasibility test; same iteration count, step
// rule, thresholds and fallback as the reference.
//
// What is different is how (A X^2 A^T) w = A X^2 c is solved.  The reference
// forms the dense (G+n) x (G+n) matrix and calls a block Cholesky.  A has two
// structural non-zeros per edge column, so eliminating the n edge rows by hand
// (they are diagonal plus a rank-one term) leaves a G x G system
//     S = sum_j lambda_j (e_k - e_i)(e_k - e_i)^T + diag(s^2) + t^2 11^T + kappa v v^T
// -- a weighted graph Laplacian of the replica topology plus a diagonal and two
// rank-one terms -- with right-hand side -t^2 1 + 1000 kappa v, where
//     E_j = x_o^2 + x_r^2, u_j = 1/E_j, lambda_j = w_j^2 x_o^2 x_r^2 u_j,
//     kappa = x_M^2 / (1 + x_M^2 sum u), q = B u, v = m + q.
// Lane i of the wave owns rank i, lane j owns edge j (two edges per lane beyond 64).  S is
// assembled and [S | rhs] reduced by Gauss-Jordan elimination in fp64: the system is tiny,
// and fp64 here removes the 1e-4..1e-3 rounding scatter a 32-bit factorisation shows on
// nearly balanced loads.  Everything else is fp32.  For the elimination, lane i holds row i
// of S (8 and 64 ranks, and four LPs per wave), or the 4 or 2 lanes per rank that a wave has
// at 16 or 32 ranks share the row; pivots are broadcast with v_readlane, the pivot row's
// entries with v_readlane or through LDS, and every lane updates what it holds.
#pragma once
#include "common.h"

namespace lplb {

typedef float f32x4 __attribute__((ext_vector_type(4)));
// Group sizes from which the elimination takes its pivot rows from LDS (exact-fit variants; padded
// ones from 16), and from which a lane's row of S is put together in LDS instead of registers.
constexpr int kRowsFromLdsMin = 8, kTileAssemblyMin = 16;
// With 16 or 32 ranks a wave has 4 or 2 lanes per rank: they share the rank's row of S (one LP per wave).
constexpr bool rows_are_shared(int gm) { return gm == 16 || gm == 32; }

struct SolveArgs {
  const int32_t *workload;   // [n_inst][n_experts]
  float *gw_out;             // [n_inst][n_experts] or null
  const int32_t *r2o;        // [G][D]
  const int32_t *phy2log;    // [n_group][G][P]
  int32_t *avail;
  float *result;             // [n_inst][n_group][G][D]
  int n_group, G, D, C, n_fixed, n_experts, step_rule, n_steps, n_units;
  int staged_stride;   // floats of LDS per LP for its counts, 0 = read them from global memory
  const int *counts_ready;   // or null.  LDS flag: once it is non-zero the caller has put the counts of this
                             // wave's LP into staged_counts (as floats) and a.workload is not read
  int counts_wait_polls;     // how many times to look at that flag before giving up on it
  unsigned long long *tagged_result;  // or null: a copy of a.result for other workgroups of the same launch,
  uint32_t tag_valid;                 // each value written through to memory as (tag_valid << 32) | its bits
  int tagged_copies, tagged_stride;   // ... tagged_copies times, tagged_stride words apart (the pollers spread over the copies)
                                      // (the caller writes tag_valid + 1 for "no result: use the neutral fallback")
  long long *clocks;         // debug builds: wall-clock stamps of wave 0, lane 0 (else null)
};

// Stamps of the first wave (debug builds only).
#define LPLB_STAMP(k) LPLB_STAMP_AT(blockIdx.x == 0 ? a.clocks : nullptr, k)

template <int CTRL> __device__ inline float dpp(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
constexpr int kQuadSwap1 = 0xB1;    // quad_perm [1,0,3,2]
constexpr int kQuadSwap2 = 0x4E;    // quad_perm [2,3,0,1]
constexpr int kHalfMirror = 0x141;  // reverse within 8 lanes
constexpr int kRowMirror = 0x140;   // reverse within 16 lanes

// Sum of lanes [0, W) (W = 8, 16, 32 or 64; lanes beyond W may hold anything for
// W < 64 as long as whole 16-lane rows are either inside or outside).  The result
// is wave-uniform.
template <int W> __device__ inline float reduce_sum(float v) {
  v += dpp<kQuadSwap1>(v);
  v += dpp<kQuadSwap2>(v);
  v += dpp<kHalfMirror>(v);
  if (W <= 8)
    return readlane(v, 0);
  v += dpp<kRowMirror>(v);
  if (W <= 16)
    return readlane(v, 0);
  if (W <= 32)
    return readlane(v, 0) + readlane(v, 16);
  return (readlane(v, 0) + readlane(v, 16)) + (readlane(v, 32) + readlane(v, 48));
}
// Max with fmaxf semantics (NaN ignored unless everything is NaN).
template <int W> __device__ inline float reduce_max(float v) {
  v = fmaxf(v, dpp<kQuadSwap1>(v));
  v = fmaxf(v, dpp<kQuadSwap2>(v));
  v = fmaxf(v, dpp<kHalfMirror>(v));
  if (W <= 8)
    return readlane(v, 0);
  v = fmaxf(v, dpp<kRowMirror>(v));
  if (W <= 16)
    return readlane(v, 0);
  if (W <= 32)
    return fmaxf(readlane(v, 0), readlane(v, 16));
  return fmaxf(fmaxf(readlane(v, 0), readlane(v, 16)), fmaxf(readlane(v, 32), readlane(v, 48)));
}

// 1/a in fp64: hardware estimate (about 2^-23) + one Newton step.
__device__ inline double rcp_f64(double a) {
  double r = __builtin_amdgcn_rcp(a);
  return __builtin_fma(__builtin_fma(-a, r, 1.0), r, r);
}

// ---- one LP per wave (ROWS == 1) or one LP per 16-lane DPP row (ROWS == 4) ----
// With ROWS == 4 a lane's position inside its row plays the part of the lane id,
// broadcasts are row-local DPP moves (row_newbcast) and reductions stop at the
// row, so four independent LPs share the wave's instruction stream.
constexpr int kRowLanes = 16;
template <int ROWS> struct Layout {
  static constexpr int kWidth = ROWS == 1 ? kWave : kRowLanes;   // lanes that serve one LP
};

template <int LANE> __device__ inline float row_bcast(float v) { return dpp<0x150 + LANE>(v); }
template <int LANE> __device__ inline double row_bcast(double v) {
  int2 p = __builtin_bit_cast(int2, v);
  p.x = __builtin_amdgcn_update_dpp(0, p.x, 0x150 + LANE, 0xF, 0xF, false);
  p.y = __builtin_amdgcn_update_dpp(0, p.y, 0x150 + LANE, 0xF, 0xF, false);
  return __builtin_bit_cast(double, p);
}
// Value of `v` in lane LANE of this LP's lanes.
template <int ROWS, int LANE, typename T> __device__ inline T lp_bcast(T v) {
  if constexpr (ROWS == 1)
    return readlane(v, LANE);
  else
    return row_bcast<LANE>(v);
}
// `old` with lane LANE of this LP's lanes replaced by `v`, a value that is the same in
// all of them.  One LP per wave: v sits in scalar registers and v_writelane puts it into
// the lane (a select would first have to copy it into a vector register).
template <int ROWS, int LANE> __device__ inline double lp_set_lane(double old, double v, int lane) {
  if constexpr (ROWS == 1) {
    int2 o = __builtin_bit_cast(int2, old);
    const int2 n = __builtin_bit_cast(int2, v);
    const int lo = __builtin_amdgcn_readfirstlane(n.x), hi = __builtin_amdgcn_readfirstlane(n.y);
    asm("v_writelane_b32 %0, %1, %2" : "+v"(o.x) : "s"(lo), "n"(LANE));
    asm("v_writelane_b32 %0, %1, %2" : "+v"(o.y) : "s"(hi), "n"(LANE));
    return __builtin_bit_cast(double, o);
  } else {
    return lane == LANE ? v : old;
  }
}
// `old` with lane LANE of this LP's lanes made zero.  One LP per wave: only the high word is
// cleared (one v_writelane instead of two, and it sits in the chain from one pivot to the next).
// What is left is a denormal below 2^-1022 (or zero where denormals are flushed): as a multiplier
// in S[k] -= f * x it changes no entry that is not itself that small.
template <int ROWS, int LANE> __device__ inline double lp_clear_lane(double old, int lane) {
  if constexpr (ROWS == 1) {
    int2 o = __builtin_bit_cast(int2, old);
    asm("v_writelane_b32 %0, 0, %1" : "+v"(o.y) : "n"(LANE));
    return __builtin_bit_cast(double, o);
  } else {
    return lane == LANE ? 0.0 : old;
  }
}
// Reductions over the first W lanes of this LP (W <= 16 when ROWS == 4).
template <int ROWS, int W> __device__ inline float lp_sum(float v) {
  if constexpr (ROWS == 1) {
    return reduce_sum<W>(v);
  } else {
    v += dpp<kQuadSwap1>(v);
    v += dpp<kQuadSwap2>(v);
    v += dpp<kHalfMirror>(v);
    if (W > 8)
      v += dpp<kRowMirror>(v);
    return row_bcast<0>(v);
  }
}
template <int ROWS, int W> __device__ inline float lp_max(float v) {
  if constexpr (ROWS == 1) {
    return reduce_max<W>(v);
  } else {
    v = fmaxf(v, dpp<kQuadSwap1>(v));
    v = fmaxf(v, dpp<kQuadSwap2>(v));
    v = fmaxf(v, dpp<kHalfMirror>(v));
    if (W > 8)
      v = fmaxf(v, dpp<kRowMirror>(v));
    return row_bcast<0>(v);
  }
}


// Stores a share, and if asked also the copy other workgroups of the running kernel
// poll: the high word says "valid, from this launch", so value and flag arrive in one 8-byte store.
__device__ inline void store_share(float *p, unsigned long long *tagged, uint32_t tag, int copies, int stride,
                                   int64_t i, float v) {
  p[i] = v;
  if (tagged)
    for (int k = 0; k < copies; ++k)
      __hip_atomic_store(tagged + (int64_t)k * stride + i, ((unsigned long long)tag << 32) | __builtin_bit_cast(uint32_t, v),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// From 16 ranks on a lane's row of S is put together in LDS instead of registers: floats the
// caller provides per wave (row i at i * (GM + 4), so that 16-byte reads of different lanes'
// rows fall into different banks; then GM floats for a broadcast copy of v).
// (Also below 16 ranks when a lane holds two edges: the selectors would be 32 per column then.)
constexpr int assembly_tile_floats_of(int gm, int epl = 1) {
  return (gm >= kTileAssemblyMin || epl > 1) ? gm * (gm + 4) + gm : 4;
}
template <int GM, int EPL = 1> constexpr int assembly_tile_floats() { return assembly_tile_floats_of(GM, EPL); }

// GM, DM: register-array sizes (group size and replica slots rounded up).
// EXACT: the group is exactly GM x DM, so every loop bound is a compile-time
// constant; otherwise rows and columns G..GM-1 of the normal-equation system are
// padded with the identity, which keeps the factorisation free of branches.
// ROWS: LPs per wave (1, or 4 when GM <= 16 and GM * DM <= 16).
// EPL: replica edges per lane, 1 or 2 (ROWS == 1 only).  Edge j lives in lane j % 64, place j / 64;
// groups with 65..128 edges take two places.  Everything per rank (the G x G system included) is
// the same either way; what is per edge is done once per place, and a value of edge j is fetched
// from place j / 64 of lane j % 64.
//
// Called by all 64 lanes of a wave; waves share nothing and never synchronise.
//   first_unit     LP (instance * n_group + group) of the wave's first row
//   staged_counts  LDS, ROWS * a.staged_stride floats (unused if the stride is 0)
//   rep_of_edge    LDS, EPL * kWave ints
//   pivot_rows     LDS, 2 * kWave doubles of this wave, 16-byte aligned
//   tile           LDS, assembly_tile_floats<GM, EPL>() floats of this wave, 16-byte aligned
// Returns how many of the wave's LPs passed the feasibility test (same value in
// every lane); the caller adds it to a.avail.  -1: the counts the caller promised through
// a.counts_ready never came; nothing was solved or stored.
template <int GM, int DM, bool EXACT, int ROWS, int EPL = 1>
__device__ inline int solve_lp(const SolveArgs &a, int first_unit, float *staged_counts_of_wave,
                               int *rep_of_edge, double *pivot_rows, float *tile) {
  constexpr int WL = Layout<ROWS>::kWidth;   // lanes of one LP
  static_assert(ROWS == 1 || (ROWS == 4 && GM <= kRowLanes && GM * DM <= kRowLanes), "an LP must fit its lanes");
  static_assert(EPL == 1 || (EPL == 2 && ROWS == 1), "two edges per lane only with one LP per wave");
  static_assert(GM % 8 == 0, "pivot rows are read from LDS eight columns at a time");
  constexpr int T = WL / GM;         // lanes that share the work of one rank's b_i
  constexpr int NE = 2 * DM;         // replica edges that touch one rank
  constexpr int KB = ROWS == 1 ? 4 : 16;   // fixed-expert counts a lane prefetches for b_i
  constexpr int WR = GM;             // lanes that can hold a rank
  constexpr int WE = (GM * DM < WL && EPL == 1) ? (GM * DM < 8 ? 8 : GM * DM) : WL;  // ... an edge
  constexpr int KG = ROWS == 1 ? 4 : 16;   // normalised counts a lane prefetches for the output (and loop unrolling)
  const int wave_lane = threadIdx.x % kWave;

  // `lane` is the position inside this LP's lanes, `lane0` the wave lane where they start.
  const int lane = wave_lane % WL, lane0 = wave_lane - lane;
  const int G = EXACT ? GM : a.G, D = EXACT ? DM : a.D;
  const int C = a.C, n = G * D, n_fixed = a.n_fixed;
  const int L = D * C + n_fixed, P = L + D * C;
  // A wave whose last rows have no LP left repeats the last one and discards the result.
  const int n_units = a.n_units;
  const int unit_raw = first_unit + wave_lane / WL;
  const bool unit_on = unit_raw < n_units;
  const int unit = unit_on ? unit_raw : n_units - 1;
  const int grp = unit % a.n_group, inst = unit / a.n_group;
  float *staged_counts = staged_counts_of_wave + wave_lane / WL * a.staged_stride;
  auto gather = [&](auto v, int src) { return bpermute(v, lane0 + src); };
  // value of edge `e` (v[place] of the lane that holds it)
  auto gather_edge = [&](const auto (&v)[EPL], int e) {
    if constexpr (EPL == 1) {
      return bpermute(v[0], lane0 + e);
    } else {
      const auto lo = bpermute(v[0], e & (kWave - 1)), hi = bpermute(v[1], e & (kWave - 1));
      return e < kWave ? lo : hi;
    }
  };
  const int32_t *__restrict__ wl = a.workload + (int64_t)inst * a.n_experts;
  const int32_t *__restrict__ p2l = a.phy2log + (int64_t)grp * G * P;
  const bool is_rank = lane < G;
  bool is_edge[EPL];
  int ek[EPL], ed[EPL];   // original rank of my edge, its replica slot
#pragma unroll
  for (int p = 0; p < EPL; ++p) {
    const int j = lane + p * kWave;
    is_edge[p] = j < n;
    ek[p] = is_edge[p] ? j / D : 0;
    ed[p] = is_edge[p] ? j % D : 0;
  }
  // When they fit, the counts are staged in LDS as floats, so that the gathers
  // through phy2log do not need a second round trip to global memory.
  const bool staged = a.staged_stride > 0;
  auto count_of = [&](int e) -> float {
    if (e < 0 || e >= a.n_experts)
      return 0.0f;
    return staged ? staged_counts[e] : (float)wl[e];
  };

  LPLB_STAMP(0);
  // ---- all global reads up front, as independent loads ----
  // (a) my edge's experts: raw count of the first, the rest in the loop below
  int e_first[EPL];
#pragma unroll
  for (int p = 0; p < EPL; ++p)
    e_first[p] = (is_edge[p] && C > 0) ? p2l[ek[p] * P + ed[p]] : -1;
  // (b) the experts of "my" rank that cannot move (T lanes share a rank)
  const int br = lane / T, bsub = lane % T;
  int fixed_e[KB];
#pragma unroll
  for (int u = 0; u < KB; ++u) {
    const int j = bsub + u * T;
    fixed_e[u] = (br < G && j < n_fixed) ? p2l[br * P + D * C + j] : -1;
  }
  // (c) topology row of my rank
  int r2o_row[DM];
#pragma unroll
  for (int d = 0; d < DM; ++d) {
    int k = (is_rank && d < D) ? a.r2o[lane * D + d] : 0;
    r2o_row[d] = k < 0 ? 0 : (k >= G ? G - 1 : k);
  }
  // (d) the counts: the maximum over all experts of all groups, minilp.cu:181-189, and
  // (e) this group's counts, for the normalised-count output at the end.  A caller
  // that is still producing the counts hands them over in LDS; the table loads
  // above are on their way meanwhile.
  const bool prestaged = a.counts_ready != nullptr;
  float wmax = 0.0f;
  float out_cnt[KG];
  if (prestaged) {
    // 1 = the counts are staged, 2 = the caller gave up on them; the wait itself is bounded
    // as well, so that this wave ends whatever happens to the flag.
    int ready = 0;
    for (int polls = 0; polls < a.counts_wait_polls; ++polls) {
      ready = __hip_atomic_load(a.counts_ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (ready != 0)
        break;
      __builtin_amdgcn_s_sleep(1);
    }
    if (ready != 1)
      return -1;   // nothing has been written
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    for (int i = lane; i < a.n_experts; i += WL)
      wmax = fmaxf(wmax, staged_counts[i]);
#pragma unroll
    for (int u = 0; u < KG; ++u) {
      const int i = lane + u * WL;
      out_cnt[u] = (a.gw_out && i < G * L) ? staged_counts[grp * G * L + i] : 0.0f;
    }
  } else {
#pragma unroll KG
    for (int i = lane; i < a.n_experts; i += WL) {
      const float cnt = (float)wl[i];
      wmax = fmaxf(wmax, cnt);
      if (staged)
        staged_counts[i] = cnt;
    }
#pragma unroll
    for (int u = 0; u < KG; ++u) {
      const int i = lane + u * WL;
      out_cnt[u] = (a.gw_out && i < G * L) ? (float)wl[grp * G * L + i] : 0.0f;
    }
  }
  __builtin_amdgcn_wave_barrier();   // staged counts are visible to the whole wave
  float w_first[EPL];
#pragma unroll
  for (int p = 0; p < EPL; ++p)
    w_first[p] = count_of(e_first[p]);
  float fixed_cnt[KB];
#pragma unroll
  for (int u = 0; u < KB; ++u)
    fixed_cnt[u] = count_of(fixed_e[u]);
  wmax = lp_max<ROWS, WL>(wmax);

  LPLB_STAMP(1);
  // ---- per-edge constants (lane j < n): w_j, minilp.cu:203-221 ----
  float w[EPL];
  int erep[EPL];
#pragma unroll
  for (int p = 0; p < EPL; ++p) {
    w[p] = is_edge[p] && C > 0 ? w_first[p] / wmax : 0.0f;
    if (is_edge[p])
      for (int c = 1; c < C; ++c)
        w[p] += count_of(p2l[ek[p] * P + c * D + ed[p]]) / wmax;
    // rank that holds the copy of each edge: invert r2o through LDS
    rep_of_edge[lane0 + lane + p * kWave] = ek[p];
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int d = 0; d < DM; ++d)
    if (is_rank && d < D)
      rep_of_edge[lane0 + r2o_row[d] * D + d] = lane;
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int p = 0; p < EPL; ++p)
    erep[p] = rep_of_edge[lane0 + lane + p * kWave];

  LPLB_STAMP(2);
  // ---- per-rank constants (lane i < G) ----
  // Edge e < DM: my own edge (i, e), other end = where its copy lives.
  // Edge DM + d: the edge copied into my slot d, other end = its original rank.
  // An inactive edge points at myself, which makes all its terms vanish.
  int src[NE], oth[NE];
  float w_e[NE];
  bool slot_on[DM];
#pragma unroll
  for (int d = 0; d < DM; ++d) {
    const bool on = is_rank && d < D;
    slot_on[d] = on;
    src[d] = on ? lane * D + d : 0;
    src[DM + d] = on ? r2o_row[d] * D + d : 0;
    // cross-lane reads stay outside lane-dependent conditions
    const int other = gather_edge(erep, src[d]);
    const float w_own = gather_edge(w, src[d]), w_copy = gather_edge(w, src[DM + d]);
    oth[d] = on ? other : lane;
    oth[DM + d] = on ? r2o_row[d] : lane;
    w_e[d] = on ? w_own : 0.0f;
    w_e[DM + d] = on ? w_copy : 0.0f;
  }
  // Selectors for assembling my row of S: 1 on my own column, -1 on the column
  // of each edge's other end.
  // (From 32 ranks on the selectors alone would be 160 registers: there the row is put
  // together in LDS instead, see kTileAssembly below.)
  constexpr bool kTileAssembly = ROWS == 1 && (GM >= kTileAssemblyMin || EPL > 1);
  constexpr int GS = kTileAssembly ? 1 : GM;
  float mask[NE][GS], diag_mask[GS];
#pragma unroll
  for (int c = 0; c < GS; ++c) {
    diag_mask[c] = (lane == c) ? 1.0f : 0.0f;
#pragma unroll
    for (int e = 0; e < NE; ++e)
      mask[e][c] = (oth[e] == c) ? -1.0f : 0.0f;
  }
  // Shared rows (16 and 32 ranks, one LP per wave): for the elimination, wave lane l works on row
  // l / TS of S and holds its columns k * TS + l % TS, k < KC.  Rows and the copy of v are laid out
  // in LDS so that the columns of one lane are adjacent: column r at (r % TS) * KC + r / TS.
  constexpr bool kShared = ROWS == 1 && rows_are_shared(GM);
  constexpr int TS = kShared ? kWave / GM : 1, KC = GM / TS;
  auto tile_pos = [](int r) { return (r % TS) * KC + r / TS; };
  const int row_of_lane = wave_lane / TS, sub = wave_lane % TS;
  float *my_tile_row = tile + (lane < GM ? lane : GM - 1) * (GM + 4);
  float *v_copy = tile + GM * (GM + 4);
  int oth_at[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e)
    oth_at[e] = tile_pos(oth[e]);
  const int own_at = tile_pos(lane < GM ? lane : GM - 1);
  const float *shared_row = tile + row_of_lane * (GM + 4) + sub * KC;   // my KC columns of my row ...
  const float *shared_v = v_copy + sub * KC;                            // ... and v of those columns' ranks
  const int v_of_row_at = tile_pos(row_of_lane);
  const bool row_real = row_of_lane < G;

  LPLB_STAMP(3);
  // b_i = -(load of the experts that cannot move), minilp.cu:223-234
  float part = 0.0f;
#pragma unroll
  for (int u = 0; u < KB; ++u)
    part += fixed_cnt[u] / wmax;
  // ranks with more fixed experts than were prefetched: the rest in batches of
  // independent loads (added in the same order as one by one)
  if (br < G)
    for (int j0 = bsub + KB * T; j0 < n_fixed; j0 += KB * T) {
      int more_e[KB];
#pragma unroll
      for (int u = 0; u < KB; ++u)
        more_e[u] = j0 + u * T < n_fixed ? p2l[br * P + D * C + j0 + u * T] : -1;
#pragma unroll
      for (int u = 0; u < KB; ++u)
        if (j0 + u * T < n_fixed)
          part += count_of(more_e[u]) / wmax;
    }
  if (T >= 2) part += dpp<kQuadSwap1>(part);
  if (T >= 4) part += dpp<kQuadSwap2>(part);
  if (T >= 8) part += dpp<kHalfMirror>(part);
  const float part_of_rank = gather(part, (lane * T) & (WL - 1));
  const float b = is_rank ? -part_of_rank : 0.0f;
  // Big-M column, minilp.cu:275-281: b_i minus the other entries of row i.
  float m = b;
#pragma unroll
  for (int e = 0; e < NE; ++e)
    m -= w_e[e];
  m = (m - 1.0f) + 1.0f;
  if (!is_rank)
    m = 0.0f;

  LPLB_STAMP(4);
  // ---- affine scaling ----
  float xo[EPL], xr[EPL], xs = 1.0f, xt = 1.0f, xM = 1.0f;
#pragma unroll
  for (int p = 0; p < EPL; ++p)
    xo[p] = xr[p] = 1.0f;
  float d_max = 0.0f;
  const int NV = 2 * n + G + 2;
  const int win_lo = a.step_rule == LPLB_STEP_REFERENCE_WINDOW ? (NV > 32 ? NV - 32 : 0) : 0;
  const bool with_zero = a.step_rule != LPLB_STEP_REFERENCE_WINDOW || NV < 32;
  bool win_o[EPL], win_r[EPL];
#pragma unroll
  for (int p = 0; p < EPL; ++p) {
    win_o[p] = is_edge[p] && lane + p * kWave >= win_lo;
    win_r[p] = is_edge[p] && n + lane + p * kWave >= win_lo;
  }
  const bool win_s = is_rank && 2 * n + lane >= win_lo;
  const double row_on = is_rank ? 1.0 : 0.0;

  for (int step = 0; step < a.n_steps; ++step) {
    const float ss = xs * xs, st = xt * xt, sM = xM * xM;
    float so[EPL], sr[EPL], u[EPL], ao[EPL], ar[EPL], lam[EPL];
    float u_all = 0.0f;
#pragma unroll
    for (int p = 0; p < EPL; ++p) {
      so[p] = xo[p] * xo[p];
      sr[p] = xr[p] * xr[p];
      u[p] = is_edge[p] ? __builtin_amdgcn_rcpf(so[p] + sr[p]) : 0.0f;
      const float wu = w[p] * u[p];
      ao[p] = wu * so[p];
      ar[p] = wu * sr[p];
      lam[p] = w[p] * ao[p] * sr[p];             // w^2 so sr / (so + sr)
      u_all = p == 0 ? u[p] : u_all + u[p];
    }
    const float sigma = lp_sum<ROWS, WE>(u_all);
    const float kappa = sM * __builtin_amdgcn_rcpf(1.0f + sM * sigma);

    float q = 0.0f, lam_e[NE], lam_sum = ss;
#pragma unroll
    for (int d = 0; d < DM; ++d) {
      const float q_own = gather_edge(ao, src[d]), q_copy = gather_edge(ar, src[DM + d]);
      const float l_own = gather_edge(lam, src[d]), l_copy = gather_edge(lam, src[DM + d]);
      // an inactive slot or a self-loop (oth == lane) contributes nothing to S;
      // an inactive slot contributes nothing to q either
      q += slot_on[d] ? q_own + q_copy : 0.0f;
      lam_e[d] = (oth[d] == lane) ? 0.0f : l_own;
      lam_e[DM + d] = (oth[DM + d] == lane) ? 0.0f : l_copy;
      lam_sum += lam_e[d] + lam_e[DM + d];
    }
    const float v = is_rank ? m + q : 0.0f;

    if (step == 0) LPLB_STAMP(5);
    // Row `lane` of S and its right-hand side, fp64.
    double S[KC];
    double rhs;
    const double dst = (double)st, dkv = (double)kappa * (double)v;
    const float st_col = is_rank ? st : 0.0f;
    if constexpr (kTileAssembly) {
      // The Laplacian part of my row: zero it, subtract every edge's weight at the column of
      // its other end, add the diagonal (LDS float adds, no return value: they queue up in
      // program order, so each entry is the same sum, in the same order, as with selectors),
      // read it back.  A lane touches only its own row.  v of every rank comes back from a
      // copy in LDS, four ranks per read from a wave-uniform address.
      const f32x4 zero{0.0f, 0.0f, 0.0f, 0.0f};
      if (lane < GM) {
#pragma unroll
        for (int c4 = 0; c4 < GM / 4; ++c4)
          reinterpret_cast<f32x4 *>(my_tile_row)[c4] = zero;
        v_copy[own_at] = v;
#pragma unroll
        for (int e = 0; e < NE; ++e)
          __hip_atomic_fetch_add(my_tile_row + oth_at[e], -lam_e[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        __hip_atomic_fetch_add(my_tile_row + own_at, lam_sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if constexpr (kShared) {
        // every lane of a row takes its KC columns; the row's own v comes from the copy as well
        const double dkv_row = (double)kappa * (double)v_copy[v_of_row_at];
        static_for<KC / 4>([&](auto k4c) {
          constexpr int k4 = decltype(k4c)::value;
          const f32x4 t4 = reinterpret_cast<const f32x4 *>(shared_row)[k4];
          const f32x4 v4 = reinterpret_cast<const f32x4 *>(shared_v)[k4];
          const float t[4] = {t4.x, t4.y, t4.z, t4.w}, vc[4] = {v4.x, v4.y, v4.z, v4.w};
          static_for<4>([&](auto uu) {
            constexpr int u = decltype(uu)::value, k = 4 * k4 + u;
            const double base = (EXACT || (row_real && k * TS + sub < G)) ? dst : 0.0;
            S[k] = __builtin_fma(dkv_row, (double)vc[u], base) + (double)t[u];
          });
        });
        rhs = (EXACT || row_real) ? 1000.0 * dkv_row - dst : 0.0;
      } else
      static_for<GM / 4>([&](auto c4c) {
        constexpr int c4 = decltype(c4c)::value;
        const f32x4 t4 = reinterpret_cast<const f32x4 *>(my_tile_row)[c4];
        const f32x4 v4 = reinterpret_cast<const f32x4 *>(v_copy)[c4];
        const float t[4] = {t4.x, t4.y, t4.z, t4.w}, vc[4] = {v4.x, v4.y, v4.z, v4.w};
        static_for<4>([&](auto uu) {
          constexpr int u = decltype(uu)::value, c = 4 * c4 + u;
          const double base = EXACT ? dst : (double)lp_bcast<ROWS, c>(st_col) * row_on;
          S[c] = __builtin_fma(dkv, (double)vc[u], base) + (double)t[u];
        });
      });
    } else {
      static_for<GM>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        float t = diag_mask[c] * lam_sum;
#pragma unroll
        for (int e = 0; e < NE; ++e)
          t = __builtin_fmaf(mask[e][c], lam_e[e], t);
        const double base = EXACT ? dst : (double)lp_bcast<ROWS, c>(st_col) * row_on;
        S[c] = __builtin_fma(dkv, (double)lp_bcast<ROWS, c>(v), base) + (double)t;
      });
    }
    if constexpr (!kShared)
      rhs = (1000.0 * dkv - dst) * (EXACT ? 1.0 : row_on);

    if (step == 0) LPLB_STAMP(6);
    // Gauss-Jordan elimination of [S | rhs] by columns: lane i owns row i, column c
    // is cleared in every other row at once, so no triangular solves (and no
    // transposed factor) are needed afterwards.  Row c's entries are read from lane
    // c, whose own multiple f is zero.  S is symmetric positive definite: no pivoting.
    // The only serial chain is pivot -> reciprocal -> f -> entry (c+1, c+1) -> next
    // pivot; it is written out in that order, with the rest of column step c (which
    // nothing waits for) placed between the links of the next reciprocal, because
    // the compiler keeps the order it is given here.  (Computing the next pivot one step
    // ahead from three more broadcasts, in uniform arithmetic, gives bit-identical results
    // and takes the vector update out of the chain, but costs 9 instructions per pivot and
    // was slower at 8 ranks.)
    // A lane's own multiple must be zero.  Rather than selecting on the chain (f is the
    // link between reciprocal and update), the lane's diagonal entry is cleared as soon
    // as it has been read as the pivot, one step ahead.
    float y;
    if constexpr (kShared) {
      // Shared rows.  The T lanes of row i all need the multiple f_i = S[i][c] / pivot: the lane that
      // holds column c hands its entry to the others of its row with one quad-permute DPP move per
      // half (rows are groups of 2 or 4 adjacent lanes).  That value is also what the row adds to
      // the pivot row in LDS (S[c][i] = S[i][c]), stored part by part like the rows themselves, so
      // a lane reads the entries under its own columns, two per 16-byte read, from one of TS
      // addresses.  The pivot is read from, and the diagonal entry cleared in, the one lane that
      // holds it, before the move: all lanes of row c then get f = 0.  A lane also updates columns
      // left of the pivot that share a register index with live ones; nothing reads them again.
      // The right-hand side is kept by every lane of a row (same arithmetic in each), the pivot of
      // a row by its first lane, where y is complete.  Operation for operation this is the
      // elimination below; only who holds what differs.
      constexpr int kStride = KC + 2;                 // doubles between the parts of a pivot row (distinct banks)
      constexpr int kPart = KC < 8 ? KC : 8;          // columns per batch of LDS reads
      constexpr int kParts = KC / kPart;
      static_assert(kParts <= 2 && TS * kStride <= kWave, "pivot rows are fetched in at most two batches");
      const int publish_at = (row_of_lane % TS) * kStride + row_of_lane / TS;
      const double *my_part = pivot_rows + sub * kStride;
      auto share = [](auto jc, double v) {     // v of lane j of every group of TS lanes
        constexpr int j = decltype(jc)::value;
        constexpr int ctrl = TS == 4 ? j * 0x55 : (j == 0 ? 0xA0 : 0xF5);
        int2 p = __builtin_bit_cast(int2, v);
        p.x = __builtin_amdgcn_mov_dpp(p.x, ctrl, 0xF, 0xF, false);   // (every lane has a source: no old value)
        p.y = __builtin_amdgcn_mov_dpp(p.y, ctrl, 0xF, 0xF, false);
        return __builtin_bit_cast(double, p);
      };
      // columns [q * kPart, (q + 1) * kPart) of the pivot row in buffer `parity`, those from k_from on
      auto load_part = [&](int parity, int q, int k_from, double (&buf)[kPart]) {
        const double2 *src = reinterpret_cast<const double2 *>(my_part + parity * kWave + q * kPart);
#pragma unroll
        for (int j = 0; j < kPart / 2; ++j)
          if (q * kPart + 2 * j + 1 >= k_from) {
            const double2 both = src[j];
            buf[2 * j] = both.x;
            buf[2 * j + 1] = both.y;
          }
        __builtin_amdgcn_sched_barrier(0);   // the reads stay here, ahead of their use
      };
      double head[2][kPart];
      double my_pivot = 1.0;
      double pivot = readlane(S[0], 0);
      double rinv = rcp_f64(pivot);
      S[0] = lp_clear_lane<1, 0>(S[0], 0);
      double col = share(std::integral_constant<int, 0>{}, S[0]);
      pivot_rows[publish_at] = col;
      __builtin_amdgcn_wave_barrier();
      load_part(0, 0, 0, head[0]);
      static_for<GM>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        constexpr int k1 = (c + 1) / TS;              // register of column c + 1, the first one still live
        constexpr int q0 = k1 / kPart;
        double body[kPart];
        auto clear = [&](auto kc, double f) {
          constexpr int k = decltype(kc)::value;
          if constexpr (k < KC) {
            if constexpr (k / kPart == q0)
              S[k] = __builtin_fma(-f, head[c % 2][k % kPart], S[k]);
            else
              S[k] = __builtin_fma(-f, body[k % kPart], S[k]);
          }
        };
        my_pivot = lp_set_lane<1, c * TS>(my_pivot, pivot, 0);
        const double f = col * rinv;   // multiple of row c to subtract from my row (0 in row c)
        double next_pivot = 1.0, estimate = 1.0, error = 0.0, next_col = 0.0;
        if constexpr (q0 + 1 < kParts)
          load_part(c % 2, q0 + 1, 0, body);
        clear(std::integral_constant<int, k1>{}, f);
        if constexpr (c + 1 < GM) {
          constexpr int holder = (c + 1) * TS + (c + 1) % TS;   // lane with entry (c + 1, c + 1)
          next_pivot = readlane(S[k1], holder);
          estimate = __builtin_amdgcn_rcp(next_pivot);
          S[k1] = lp_clear_lane<1, holder>(S[k1], 0);
          next_col = share(std::integral_constant<int, (c + 1) % TS>{}, S[k1]);
          pivot_rows[((c + 1) % 2) * kWave + publish_at] = next_col;
          __builtin_amdgcn_wave_barrier();
          constexpr int k1_next = (c + 2) / TS;
          if constexpr (k1_next < KC)
            load_part((c + 1) % 2, k1_next / kPart, k1_next, head[(c + 1) % 2]);
        }
        rhs = __builtin_fma(-f, readlane(rhs, c * TS), rhs);
        clear(std::integral_constant<int, k1 + 1>{}, f);
        if constexpr (c + 1 < GM)
          error = __builtin_fma(-next_pivot, estimate, 1.0);
        clear(std::integral_constant<int, k1 + 2>{}, f);
        clear(std::integral_constant<int, k1 + 3>{}, f);
        if constexpr (c + 1 < GM) {
          rinv = __builtin_fma(error, estimate, estimate);   // = rcp_f64(next_pivot)
          pivot = next_pivot;
        }
        static_for<(KC > k1 + 4 ? KC - k1 - 4 : 0)>([&](auto kk) {
          clear(std::integral_constant<int, k1 + 4 + decltype(kk)::value>{}, f);
        });
        col = next_col;
      });
      if (step == 0) LPLB_STAMP(7);
      const float y_of_row = (float)(rhs * rcp_f64(my_pivot));   // in the first lane of each row
      const float y_mine = gather(y_of_row, (lane * TS) & (kWave - 1));
      y = is_rank ? y_mine : 0.0f;
    } else {
      double my_pivot = 1.0;
      double pivot = lp_bcast<ROWS, 0>(S[0]);
      double rinv = rcp_f64(pivot);
      // One LP per wave: the entries of pivot row c that the other rows need, S[c][c2] for
      // c2 > c, are not fetched from lane c one by one (two v_readlane each).  The part of S
      // that is still being eliminated stays symmetric (up to rounding), so they are also
      // column c as it is spread over the lanes, S[c2][c] in lane c2: one LDS write of that
      // register puts the whole row into LDS, and reads from a wave-uniform address hand two
      // entries at a time to every lane.  LDS instructions do not take the vector ALU's issue
      // slots, which are what bounds a lone wave.  Column c + 1 is final right after the first
      // update of step c; it is written then, so the round trip through LDS overlaps the rest
      // of step c and the reciprocal of the next pivot and is not part of the serial chain.
      // Two buffers take turns, so a step's reads need not all be issued before the next write.
      // (Measured per LP: 32 ranks 31.5 -> 22.2 us, 16 ranks 12.6 -> 11.2 us, 8 ranks 7.5 -> 7.2 us; four
      // LPs per wave, each 16-lane row reading its own LP's column: 16384 LPs 30.9 -> 27.6 us.  The
      // padded 8-rank variants keep the scalar broadcasts: inside the one-launch plan they have
      // no register to spare at four waves per SIMD.)
      constexpr bool kRowFromLds = (ROWS == 1 && (GM >= 16 || (GM >= kRowsFromLdsMin && EXACT))) || ROWS == 4;
      constexpr int kChunk = 8;                       // columns per batch of LDS reads (GM is a multiple)
      constexpr int kChunks = GM / kChunk;
      constexpr int kBodySets = kChunks > 2 ? 2 : 1;  // chunks after a step's first are fetched one chunk ahead
      // chunk q of the row in buffer `parity`: columns 8 q .. 8 q + 7, four 16-byte reads
      auto load_chunk = [&](int parity, int q, double (&buf)[kChunk]) {
        const double2 *src = reinterpret_cast<const double2 *>(pivot_rows + parity * kWave + lane0 + q * kChunk);
#pragma unroll
        for (int j = 0; j < kChunk / 2; ++j) {
          const double2 both = src[j];
          buf[2 * j] = both.x;
          buf[2 * j + 1] = both.y;
        }
        // The reads stay where they are written, ahead of their use: left alone, the compiler
        // moves each one down to the instruction that needs it (fewer live registers) and the
        // wave then waits out every LDS round trip.
        __builtin_amdgcn_sched_barrier(0);
      };
      // The first chunk a step needs is fetched during the step before, right after the column
      // has been written (two sets of registers take turns).
      double head[2][kChunk];
      auto publish_column = [&](auto cc) {
        constexpr int c = decltype(cc)::value;
        if constexpr (kRowFromLds && c < GM) {
          pivot_rows[(c % 2) * kWave + lane0 + lane] = S[c];   // (every lane writes: no branch; lanes >= GM are never read)
          __builtin_amdgcn_wave_barrier();
          if constexpr (c + 1 < GM)
            load_chunk(c % 2, (c + 1) / kChunk, head[c % 2]);
        }
      };
      publish_column(std::integral_constant<int, 0>{});
      S[0] = lp_clear_lane<ROWS, 0>(S[0], lane);
      static_for<GM>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        constexpr int q0 = (c + 1) / kChunk;          // chunk of column c + 1
        double body[kBodySets][kChunk];
        // S[c2] -= f * (row c)[c2]
        auto clear = [&](auto c2c, double f) {
          constexpr int c2 = decltype(c2c)::value;
          if constexpr (c2 < GM) {
            if constexpr (!kRowFromLds) {
              S[c2] = __builtin_fma(-f, lp_bcast<ROWS, c>(S[c2]), S[c2]);
            } else if constexpr (c2 / kChunk == q0) {
              S[c2] = __builtin_fma(-f, head[c % 2][c2 % kChunk], S[c2]);
            } else {
              // entering a new chunk: fetch the one after it, and keep the compiler from pulling
              // every later fetch up here (the rows would not fit the registers)
              if constexpr (c2 % kChunk == 0 && kBodySets == 2) {
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (c2 / kChunk + 1 < kChunks)
                  load_chunk(c % 2, c2 / kChunk + 1, body[(c2 / kChunk + 1) % kBodySets]);
              }
              S[c2] = __builtin_fma(-f, body[(c2 / kChunk) % kBodySets][c2 % kChunk], S[c2]);
            }
          }
        };
        my_pivot = lp_set_lane<ROWS, c>(my_pivot, pivot, lane);
        const double f = S[c] * rinv;   // multiple of row c to subtract from my row (0 in lane c)
        double next_pivot = 1.0, estimate = 1.0, error = 0.0;
        if constexpr (kRowFromLds && q0 + 1 < kChunks)
          load_chunk(c % 2, q0 + 1, body[(q0 + 1) % kBodySets]);
        clear(std::integral_constant<int, c + 1>{}, f);
        publish_column(std::integral_constant<int, c + 1>{});
        if constexpr (c + 1 < GM) {
          next_pivot = lp_bcast<ROWS, c + 1>(S[c + 1]);
          estimate = __builtin_amdgcn_rcp(next_pivot);
          S[c + 1] = lp_clear_lane<ROWS, c + 1>(S[c + 1], lane);
        }
        rhs = __builtin_fma(-f, lp_bcast<ROWS, c>(rhs), rhs);
        clear(std::integral_constant<int, c + 2>{}, f);
        if constexpr (c + 1 < GM)
          error = __builtin_fma(-next_pivot, estimate, 1.0);
        clear(std::integral_constant<int, c + 3>{}, f);
        clear(std::integral_constant<int, c + 4>{}, f);
        if constexpr (c + 1 < GM) {
          rinv = __builtin_fma(error, estimate, estimate);   // = rcp_f64(next_pivot)
          pivot = next_pivot;
        }
        static_for<(GM > c + 5 ? GM - c - 5 : 0)>([&](auto kk) {
          constexpr int k = decltype(kk)::value;
          // From 32 ranks on a row's broadcasts would fill the scalar registers if the
          // compiler hoisted them all; fence them off in groups of eight columns.
          if constexpr (!kRowFromLds && GM >= 32 && k % 8 == 0)
            __builtin_amdgcn_sched_barrier(0);
          clear(std::integral_constant<int, c + 5 + k>{}, f);
        });
      });
      if (step == 0) LPLB_STAMP(7);
      y = is_rank ? (float)(rhs * rcp_f64(my_pivot)) : 0.0f;
    }

    if (step == 0) LPLB_STAMP(8);
    // r = A^T w and the direction d = x (c - r); the edge part of w is
    // z = u (h - kappa u.h + kappa (m.y - 1000)), h = -B^T y.
    float yk[EPL], yrep[EPL], hp[EPL];
    float uhp_all = 0.0f;
#pragma unroll
    for (int p = 0; p < EPL; ++p) {
      yk[p] = gather(y, ek[p]);
      yrep[p] = gather(y, erep[p]);
      hp[p] = -w[p] * (so[p] * yk[p] + sr[p] * yrep[p]);
      uhp_all = p == 0 ? u[p] * hp[p] : uhp_all + u[p] * hp[p];
    }
    const float my = lp_sum<ROWS, WR>(m * y);
    const float sumy = lp_sum<ROWS, WR>(y);
    const float uh = lp_sum<ROWS, WE>(uhp_all);
    const float shift = kappa * (my - 1000.0f) - kappa * uh;
    const float sumz = uh + shift * sigma;       // = sum of z over the edges
    float d_o[EPL], d_r[EPL];
#pragma unroll
    for (int p = 0; p < EPL; ++p) {
      const float z = u[p] * (hp[p] + shift);
      d_o[p] = -xo[p] * (w[p] * yk[p] + z);
      d_r[p] = -xr[p] * (w[p] * yrep[p] + z);
    }
    const float d_s = -xs * y;
    const float d_t = xt * (1.0f + sumy);
    const float d_M = xM * (1000.0f - (my - sumz));

    if (step == 0) LPLB_STAMP(9);
    // Step length, minilp.cu:354-362.  NaN marks "not in the window".
    float cand = __builtin_nanf("");
#pragma unroll
    for (int p = 0; p < EPL; ++p) {
      cand = win_o[p] ? fmaxf(cand, d_o[p]) : cand;
      cand = win_r[p] ? fmaxf(cand, d_r[p]) : cand;
    }
    cand = win_s ? fmaxf(cand, d_s) : cand;
    cand = lane == 0 ? fmaxf(fmaxf(cand, d_t), d_M) : cand;
    d_max = lp_max<ROWS, WE>(cand);
    if (with_zero)
      d_max = fmaxf(d_max, 0.0f);
    const float alpha = (float)(0.999 / (double)d_max);
#pragma unroll
    for (int p = 0; p < EPL; ++p) {
      xo[p] *= 1.0f - alpha * d_o[p];
      xr[p] *= 1.0f - alpha * d_r[p];
    }
    xs *= 1.0f - alpha * d_s;
    xt *= 1.0f - alpha * d_t;
    xM *= 1.0f - alpha * d_M;
    if (step == 0) LPLB_STAMP(10);
  }

  LPLB_STAMP(11);
  // Feasibility, minilp.cu:369-385.
  float res = 0.0f;
  {
    float row = xs - xt + m * xM - b;
#pragma unroll
    for (int d = 0; d < DM; ++d) {
      const float a_o = gather_edge(xo, src[d]), a_r = gather_edge(xr, src[DM + d]);
      row += w_e[d] * a_o + w_e[DM + d] * a_r;
    }
    if (is_rank)
      res = fmaxf(res, fabsf(row));
#pragma unroll
    for (int p = 0; p < EPL; ++p)
      if (is_edge[p])
        res = fmaxf(res, fabsf(xo[p] + xr[p] - xM - 1.0f));
    res = lp_max<ROWS, WE>(res);
  }
  const bool ok = (double)d_max < 0.1 && 0.0 <= (double)xM && (double)xM < 1e-4 &&
                  (double)res < 0.05;
  const int n_ok = __popcll(__ballot(lane == 0 && ok && unit_on));
#pragma unroll
  for (int p = 0; p < EPL; ++p)
    if (is_edge[p] && unit_on)
      store_share(a.result, a.tagged_result, a.tag_valid, a.tagged_copies, a.tagged_stride,
                  (int64_t)unit * n + lane + p * kWave, ok ? xo[p] : 0.5f);
  // Normalised counts of this group, for the caller.
  if (a.gw_out && unit_on) {
    float *gw = a.gw_out + (int64_t)inst * a.n_experts + grp * G * L;
#pragma unroll
    for (int u = 0; u < KG; ++u)
      if (lane + u * WL < G * L)
        gw[lane + u * WL] = out_cnt[u] / wmax;
    for (int i = lane + KG * WL; i < G * L; i += WL)
      gw[i] = count_of(grp * G * L + i) / wmax;
  }
  LPLB_STAMP(12);
  return n_ok;
}

} // namespace lplb
