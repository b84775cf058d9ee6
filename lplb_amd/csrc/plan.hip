// Whole plan in one call: histogram -> LP solve -> redirect on one stream.
//
// Two ways to run it.
//
// Chain: the three entry points' kernels one after the other (histogram, scan,
// LP, redirect).  With the global counts supplied the LP does not depend on this
// GPU's histogram: it is enqueued first and the histogram launch does not wait for
// it (it still starts after everything the LP launch waited for).  Running the LP
// as a parallel branch of a captured HIP graph (side stream + events) was measured
// and rejected: 24.6 us per plan against 20.0 us for the plain chain in the graph.
//
// One launch (plan_in_one_launch): for batches of up to 64 slices of 8192 indices
// (4096 with 512-thread workgroups) and LP shapes whose registers fit beside a 512-
// or 1024-thread workgroup.  Every
// kernel boundary of the chain costs 3-5 us on this GPU although the kernels have
// 1-3 us of work, and the LP (8 us, one wave) sits on the critical path.  Here one
// workgroup per slice and one more per four LPs run side by side in a single grid:
//   slice workgroup: load indices -> per-wave LDS histograms -> publish the slice's
//     histogram row -> wait until all rows are there -> add up the rows (totals and
//     counts before this slice) -> tables and per-wave starting ordinals -> wait for
//     the LP's shares -> redirect and store;
//   LP workgroup: (own-histogram mode: wait for the rows, add them up) -> solve ->
//     publish the shares.
// What crosses workgroups (rows, shares, three counters) is written and read with
// agent-scope atomics, which go through the XCD's L2 to memory; nothing else is
// shared, so no cache write-back or invalidate is needed.  The grid is far smaller
// than the GPU (at most 72 workgroups on 256 CUs), so all workgroups are resident
// and the waits end; each wait is bounded all the same, and a wait that runs out is
// counted (lplb_plan_sync_timeouts) instead of hanging the GPU.  The counters live
// in a per-device array of this library, one block per stream (the first eight streams
// that run a plan; further streams get the chain); the last workgroup to leave
// clears its block, so a captured launch can be replayed.  Launches that share a
// block must not overlap in time: that holds for one stream's launches, not for
// graphs captured on one stream and replayed concurrently on several; and no more
// than three plans may execute at the same time on a device -- callers outside
// these limits switch this path off with lplb_plan_set_cooperative(0).
#include "map_kernel.h"
#include "solve_kernel.h"
#include <atomic>
#include <mutex>

namespace lplb {

constexpr int kMaxSlices = 64;         // slice workgroups of the one-launch plan
constexpr int kChunksPerWave = 8;     // its longest slice: 8 chunks of 64 indices per wave
constexpr int kPlanLdsLimit = 160 * 1024 - 8 * 1024;   // dynamic LDS; the kernel has 4 KB of static LDS besides
constexpr int kMaxPolls = 1 << 22;    // a few seconds of polling before a wait gives up
// LPs per LP workgroup: waves 0..3 of a workgroup sit on the CU's four SIMDs, and an LP
// wave is bound by instruction issue, so a fifth LP on the same CU would slow two of them
// down (8 LPs in one workgroup: 17.0 us per plan against 13.5 us).  Batches with more
// groups get more LP workgroups.
constexpr int kLpsPerWorkgroup = 4, kMaxLpWorkgroups = 8;

// [0] slices whose histogram row is published, [1] workgroups that have left,
// [3] waits that ran out since the library was loaded; from kSharesAt on, the LP's
// shares as 8-byte words (1 << 32) | float bits, 0 = not there yet.
// From kTotalsAt on (own-histogram mode), one 8-byte word per logical expert: the
// batch's tokens of that expert in the high half and the number of slices that have
// added theirs in the low half -- one atomic add per slice and expert delivers both,
// so the reader needs no second round trip for a "done" counter.
constexpr int kSharesAt = 16, kMaxShares = 1024;
constexpr int kTotalsAt = kSharesAt + 2 * kMaxShares, kMaxTotals = 1024;
// One such block per stream that has run a plan (the compute stream, a warm-up
// stream, a graph-capture stream ...), so that plans enqueued on different streams
// do not share counters.  A launch takes at most a quarter of the CUs (+ 8): up to three
// plans that really execute at the same time are all resident; with four or more,
// workgroups could wait for workgroups that cannot start.
constexpr int kSlotInts = kTotalsAt + 2 * kMaxTotals, kSyncSlots = 8;
static __device__ __attribute__((aligned(64))) int g_plan_sync[kSyncSlots * kSlotInts];
static std::atomic<bool> g_cooperative{true};   // any thread may flip it while others plan

struct PlanArgs {
  const int64_t *idx;
  int64_t n, per;
  int n_slices, n_lp_workgroups;
  const int32_t *o2r, *phy2log;
  int32_t *rows;     // [n_slices][n_logical] per-slice histograms, exchanged between workgroups
  int32_t *totals;   // [n_logical] this GPU's tokens per expert, out
  int64_t *out;
  int32_t *physical_counts;   // [n_ranks * P] tokens per physical expert, or null
  RedirectShape sh;
  SolveArgs solve;   // result = the shares (o_weight); workload is replaced by totals if local_counts
  int local_counts;
  int *sync;
};

__device__ inline int agent_load(const int *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void agent_store(int *p, int v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// One lane polls *word until it reaches `target`; a wait that runs out is counted.
// Afterwards this CU's L1 and this XCD's L2 drop what they hold of other XCDs'
// memory, so that the plain (batched) loads that follow the workgroup barrier see
// what the other workgroups wrote through to memory before they counted up.
// (Agent-scope atomic loads would see it too, but the compiler issues those one
// at a time: 16 of them cost 5 us.)
__device__ inline void wait_for(int *sync, int word, int target) {
  int polls = 0;
  while (agent_load(sync + word) < target && ++polls < kMaxPolls)
    __builtin_amdgcn_s_sleep(2);
  if (polls >= kMaxPolls)
    __hip_atomic_fetch_add(sync + 3, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}
// rows[r][e] summed over r = first, first + step, ...: all rows (t) and those before
// slice `pid` (before).
__device__ inline void add_up_rows(const int32_t *rows, int n_rows, int nl, int e, int first, int step, int pid,
                                   int32_t &t, int32_t &before) {
  t = 0;
  before = 0;
  constexpr int kInFlight = 16;   // loads issued before the first is used (clamped addresses, masked values)
  for (int r0 = first; r0 < n_rows; r0 += kInFlight * step) {
    int32_t v[kInFlight];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k)
      v[k] = rows[(int64_t)min(r0 + k * step, n_rows - 1) * nl + e];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      const int r = r0 + k * step;
      t += r < n_rows ? v[k] : 0;
      before += r < pid ? v[k] : 0;
    }
  }
}

// Called by a whole workgroup when it is done.  The last of the grid's workgroups
// to leave clears the counters and the shares for the next launch.
__device__ inline void leave(int *sync, int n_workgroups, int n_shares, int n_totals) {
  __shared__ int last_to_leave;
  if (threadIdx.x == 0)
    last_to_leave =
        __hip_atomic_fetch_add(sync + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == n_workgroups - 1;
  __syncthreads();
  if (!last_to_leave)
    return;
  unsigned long long *shares = reinterpret_cast<unsigned long long *>(sync + kSharesAt);
  for (int i = threadIdx.x; i < n_shares; i += blockDim.x)
    __hip_atomic_store(shares + i, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (int i = threadIdx.x; i < 2 * n_totals; i += blockDim.x)
    agent_store(sync + kTotalsAt + i, 0);
  if (threadIdx.x == 0) {
    agent_store(sync + 0, 0);
    agent_store(sync + 1, 0);
  }
}

// LDS of a slice workgroup.
static size_t plan_lds_bytes(int n_logical, int n_waves) {
  const size_t groups = (size_t)n_waves * kWave >= (size_t)n_logical ? (size_t)n_waves * kWave / n_logical : 1;
  return (size_t)n_logical * (sizeof(ExpertEntry) + 4 + 4 + (size_t)n_waves * (sizeof(WaveSlot) + 4) + groups * 8);
}

// Debug builds: stamps of the first and the last slice workgroup and of the LP's.
#define LPLB_PLAN_STAMP(k)                                                                     \
  LPLB_STAMP_AT(a.solve.clocks == nullptr ? nullptr                                            \
                : blockIdx.x == 0 ? a.solve.clocks + 64                                        \
                : blockIdx.x == a.n_slices - 1 ? a.solve.clocks + 80                           \
                : blockIdx.x == a.n_slices ? a.solve.clocks + 96 : nullptr, k)

// K: 64-index chunks per wave.  WAVES: waves per workgroup.
template <int GM, int DM, bool EXACT, int K, int WAVES>
__global__ __launch_bounds__(WAVES *kWave) void plan_in_one_launch(PlanArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ int rep_of_edge_all[WAVES * kWave];
  const int nl = a.sh.n_logical;
  const int tid = threadIdx.x;
  constexpr int nt = WAVES * kWave;
  const int lane = tid % kWave, wave = tid / kWave;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);   // the same, but known to be wave-uniform
  const int pid = blockIdx.x;
  const int n_workgroups = a.n_slices + a.n_lp_workgroups;
  const int n_shares = a.sh.n_ranks * a.sh.D;
  const int n_groups = nt >= nl ? nt / nl : 1;   // threads per expert when rows are added up

  if (pid >= a.n_slices) {
    // ------------------------------------------------------------ the LPs
    SolveArgs sa = a.solve;
    const int first_lp = (pid - a.n_slices) * kLpsPerWorkgroup;          // of this workgroup
    const int n_lps = min(kLpsPerWorkgroup, sa.n_units - first_lp);
    LPLB_PLAN_STAMP(0);
    // Own-histogram mode: the LP waves start at once (their table loads do not need
    // the counts) and pick the counts up from LDS; the wave after them waits for the
    // slices, fetches the totals the slices have added up in memory and hands them over.
    __shared__ int counts_ready;
    float *staged = reinterpret_cast<float *>(smem_raw);
    if (a.local_counts) {
      if (tid == 0)
        counts_ready = 0;
      __syncthreads();
      sa.counts_ready = &counts_ready;
      if (wave == n_lps) {
        // Poll the totals until every expert's word says that all slices have added
        // theirs (plain loads after an acquire fence: they can be batched).
        const unsigned long long *words = reinterpret_cast<const unsigned long long *>(a.sync + kTotalsAt);
        for (int polls = 0;; ++polls) {
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
          bool all_in = true;
          for (int e0 = lane; e0 < nl; e0 += 8 * kWave) {
            unsigned long long t[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
              t[k] = words[min(e0 + k * kWave, nl - 1)];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
              all_in = all_in && (uint32_t)t[k] == (uint32_t)a.n_slices;
              if (e0 + k * kWave < nl)
                staged[e0 + k * kWave] = (float)(uint32_t)(t[k] >> 32);
            }
          }
          if (__all(all_in))
            break;
          if (polls >= kMaxPolls) {
            if (lane == 0)
              __hip_atomic_fetch_add(a.sync + 3, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
          __builtin_amdgcn_s_sleep(2);
        }
        if (pid == a.n_slices)
          for (int e = lane; e < nl; e += kWave)   // this GPU's totals, for the caller
            a.totals[e] = (int32_t)staged[e];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0)
          __hip_atomic_store(&counts_ready, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
    LPLB_PLAN_STAMP(1);
    if (wave < n_lps) {
      // (own-histogram mode: every LP of the batch reads the one staged copy)
      float *mine = a.local_counts ? staged : staged + (size_t)wave * sa.staged_stride;
      const int n_ok = solve_lp<GM, DM, EXACT, 1>(sa, first_lp + wave, mine, rep_of_edge_all + wave * kWave);
      if (lane == 0 && n_ok > 0)
        atomicAdd(sa.avail, n_ok);
    }
    LPLB_PLAN_STAMP(2);
    leave(a.sync, n_workgroups, n_shares, a.local_counts ? nl : 0);
    return;
  }

  // --------------------------------------------------------------- a slice
  ExpertEntry *table = reinterpret_cast<ExpertEntry *>(smem_raw);              // [nl]
  WaveSlot *slots = reinterpret_cast<WaveSlot *>(table + nl);                 // [WAVES][nl]
  int32_t *replica = reinterpret_cast<int32_t *>(slots + (size_t)WAVES * nl); // [nl]
  int32_t *start = replica + nl;                                              // [nl]
  int32_t *counts = start + nl;                                               // [WAVES][nl]
  int32_t *partial = counts + (size_t)WAVES * nl;                             // [2][n_groups][nl]
  WaveSlot *mine = slots + (size_t)wave * nl;
  const unsigned long long my_bit = 1ull << lane;
  const int64_t begin = slice_begin(a.n, a.per, pid);
  const int64_t end = slice_begin(a.n, a.per, pid + 1);

  LPLB_PLAN_STAMP(0);
  // Small table reads that depend on nothing go out first; they are used much later.
  const int cd = a.sh.C * a.sh.D, n_sets = a.sh.n_ranks * cd;
  const int le_of_tid = tid < nl ? a.phy2log[(tid / a.sh.L) * a.sh.P + (tid % a.sh.L)] : -1;
  // first (usually only) replicated expert set of this thread
  const bool set0 = tid < n_sets;
  const int rank0 = set0 ? tid / cd : 0, local0 = set0 ? tid % cd : 0;
  const int rle0 = set0 ? a.phy2log[rank0 * a.sh.P + local0] : -1;
  const int host0 = set0 ? a.o2r[(rank0 % a.sh.G) * a.sh.D + local0 % a.sh.D] : 0;
  int32_t ev[K];   // expert ids, -1 for masked / out-of-range / past the end
#pragma unroll
  for (int c = 0; c < K; ++c) {
    const int64_t i = begin + ((int64_t)wave * K + c) * kWave + lane;
    const int64_t v = i < end ? __builtin_nontemporal_load(a.idx + i) : -1;
    ev[c] = (v >= 0 && v < nl) ? (int32_t)v : -1;
  }
  for (int i = tid; i < WAVES * nl; i += nt) {
    slots[i] = WaveSlot{0, 0, 0ull};
    counts[i] = 0;
  }
  __syncthreads();
  // tokens per expert in this wave's chunks
#pragma unroll
  for (int c = 0; c < K; ++c)
    if (ev[c] >= 0)
      atomicAdd(&counts[(size_t)wave * nl + ev[c]], 1);
  __syncthreads();
  // this slice's histogram row, for every workgroup to read
  for (int e = tid; e < nl; e += nt) {
    int32_t h = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
      h += counts[(size_t)w * nl + e];
    agent_store(a.rows + (int64_t)pid * nl + e, h);
    if (a.local_counts)
      __hip_atomic_fetch_add(reinterpret_cast<unsigned long long *>(a.sync + kTotalsAt) + e,
                             ((unsigned long long)(uint32_t)h << 32) | 1ull, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(0);   // the row has left this CU
  __syncthreads();
  LPLB_PLAN_STAMP(1);
  if (tid == 0) {
    __hip_atomic_fetch_add(a.sync + 0, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    wait_for(a.sync, 0, a.n_slices);
  }
  __syncthreads();
  LPLB_PLAN_STAMP(2);
  // add up the rows: tokens per expert in the whole batch and before this slice
  {
    const int g = nt >= nl ? tid / nl : 0;
    if (g < n_groups)
      for (int e = nt >= nl ? tid % nl : tid; e < nl; e += nt >= nl ? nl : nt) {
        int32_t t, before;
        add_up_rows(a.rows, a.n_slices, nl, e, g, n_groups, pid, t, before);
        partial[(size_t)g * nl + e] = t;
        partial[(size_t)(n_groups + g) * nl + e] = before;
      }
  }
  __syncthreads();
  LPLB_PLAN_STAMP(6);
  for (int e = tid; e < nl; e += nt) {
    int32_t t = 0, before = 0;
    for (int g = 0; g < n_groups; ++g) {
      t += partial[(size_t)g * nl + e];
      before += partial[(size_t)(n_groups + g) * nl + e];
    }
    init_entry(table, replica, start, e, t, before);
    if (pid == 0 && !a.local_counts)
      a.totals[e] = t;
  }
  __syncthreads();
  if (tid < nl)
    set_original(table, a.sh, tid, le_of_tid);
  for (int e = tid + nt; e < nl; e += nt)
    set_original(table, a.sh, e, a.phy2log[(e / a.sh.L) * a.sh.P + (e % a.sh.L)]);
  LPLB_PLAN_STAMP(7);
  // each wave's starting ordinals: tokens before this slice + those of the waves before
  // it; specialised by the (wave-uniform) number of those, so that the loop is
  // straight-line with exactly that many reads
  static_for<WAVES>([&](auto wc) {
    constexpr int kEarlier = decltype(wc)::value;
    if (wave_s != kEarlier)
      return;
    for (int e = lane; e < nl; e += kWave) {
      int32_t before[kEarlier + 1];
#pragma unroll
      for (int w = 0; w < kEarlier; ++w)
        before[w] = counts[(size_t)w * nl + e];
      int32_t run = start[e];
#pragma unroll
      for (int w = 0; w < kEarlier; ++w)
        run += before[w];
      mine[e].next = run;
    }
  });
  // The LP's shares decide how many tokens stay on the original, and nothing else:
  // replica slots, ordinals and hashes are worked out while the LP is still running,
  // so that one multiplication and one comparison per token are left for afterwards.
  LPLB_PLAN_STAMP(3);
  const unsigned long long *shares = reinterpret_cast<const unsigned long long *>(a.sync + kSharesAt);
  int le0 = -1;
  int32_t total0 = 0;
  if (set0) {
    set_replica_slot(replica, a.sh, rank0, local0, rle0, host0);
    if (rle0 >= 0 && rle0 < nl) {
      le0 = rle0;
      total0 = table[le0].total;
    }
  }
  for (int i = tid + nt; i < n_sets; i += nt) {
    const int ep_rank = i / cd, local = i % cd;
    set_replica_slot(replica, a.sh, ep_rank, local, a.phy2log[ep_rank * a.sh.P + local],
                     a.o2r[(ep_rank % a.sh.G) * a.sh.D + local % a.sh.D]);
  }
  __builtin_amdgcn_wave_barrier();   // the wave's starting ordinals above are read by other lanes below
  int32_t h[K];
#pragma unroll
  for (int c = 0; c < K; ++c) {
    ExpertEntry unused;
    h[c] = hash_of_token<false>(ev[c], mine, table, my_bit, unused);
    __builtin_amdgcn_wave_barrier();
  }
  // Every thread that needs a share polls it itself: value and "valid" arrive in the
  // same 8-byte word.
  auto share_of = [&](int ep_rank, int d) {
    unsigned long long word = 0;
    int polls = 0;
    while ((word = __hip_atomic_load(shares + ep_rank * a.sh.D + d, __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT)) == 0 && ++polls < kMaxPolls)
      __builtin_amdgcn_s_sleep(2);
    if (polls >= kMaxPolls)
      __hip_atomic_fetch_add(a.sync + 3, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(float, (uint32_t)word);
  };
  if (set0) {
    const float share = share_of(rank0, local0 % a.sh.D);
    if (le0 >= 0)
      table[le0].expected = expected_on_original(share, total0);
  }
  for (int i = tid + nt; i < n_sets; i += nt) {
    const int ep_rank = i / cd, local = i % cd;
    const float share = share_of(ep_rank, local % a.sh.D);
    const int le = a.phy2log[ep_rank * a.sh.P + local];
    if (le >= 0 && le < nl)
      table[le].expected = expected_on_original(share, table[le].total);
  }
  __syncthreads();
#pragma unroll
  for (int c = 0; c < K; ++c) {
    int64_t o = -1;
    if (ev[c] >= 0) {
      const ExpertEntry x = table[ev[c]];
      o = h[c] >= x.expected ? replica[ev[c]] : x.original;
    }
    const int64_t i = begin + ((int64_t)wave * K + c) * kWave + lane;
    if (i < end)
      __builtin_nontemporal_store(o, a.out + i);
  }
  if (pid == 0 && a.physical_counts)
    emit_physical_counts(table, replica, a.sh, a.phy2log, a.physical_counts, tid, nt);
  LPLB_PLAN_STAMP(5);
  leave(a.sync, n_workgroups, n_shares, a.local_counts ? nl : 0);
}

template <int GM, int DM, bool EXACT, int K, int WAVES>
static hipError_t launch_plan_variant(const PlanArgs &a, size_t lds, hipStream_t s) {
  if (lds > 64 * 1024) {
    const hipError_t err = allow_dynamic_lds(&plan_in_one_launch<GM, DM, EXACT, K, WAVES>, kPlanLdsLimit);
    if (err != hipSuccess)
      return err;
  }
  launch(plan_in_one_launch<GM, DM, EXACT, K, WAVES>, dim3(a.n_slices + a.n_lp_workgroups), dim3(WAVES * kWave), lds, s, a);
  return hipGetLastError();
}

// LP shapes the one-launch plan is built for, in the order they are tried, and the
// workgroup size that leaves the LP its registers: 128 VGPRs per lane at 16 waves,
// 256 at 8.
constexpr int kPlanShapes[][2] = {{8, 1}, {8, 2}, {8, 4}, {16, 1}, {16, 2}, {32, 1}, {32, 2}};
constexpr int plan_waves(int gm, int dm) { return (gm * dm <= 16 && gm <= 16) ? 16 : 8; }
static bool plan_lp_shape(int G, int D, int *gm, int *dm) {
  for (const auto &shape : kPlanShapes)
    if (G <= shape[0] && D <= shape[1]) {
      *gm = shape[0];
      *dm = shape[1];
      return true;
    }
  return false;
}

template <int GM, int DM, bool EXACT, int W> static hipError_t launch_plan_shape(PlanArgs &a, hipStream_t s) {
  const int64_t chunks = (a.per + kWave - 1) / kWave;
  const int k = (int)((chunks + W - 1) / W);
  const size_t lds_slices = plan_lds_bytes(a.sh.n_logical, W);
  const size_t lds_lp = (size_t)min(a.solve.n_units, kLpsPerWorkgroup) * a.solve.n_experts * sizeof(float);
  a.solve.staged_stride = lds_lp <= lds_slices ? a.solve.n_experts : 0;
  if (a.local_counts && a.solve.staged_stride == 0)   // the LP takes its counts from LDS in that mode
    return hipErrorInvalidValue;
  if (k <= 1)
    return launch_plan_variant<GM, DM, EXACT, 1, W>(a, lds_slices, s);
  if (k <= 2)
    return launch_plan_variant<GM, DM, EXACT, 2, W>(a, lds_slices, s);
  if (k <= 4)
    return launch_plan_variant<GM, DM, EXACT, 4, W>(a, lds_slices, s);
  return launch_plan_variant<GM, DM, EXACT, 8, W>(a, lds_slices, s);
}

// The block of counters a stream uses: the first kSyncSlots streams that run a plan
// each get their own, -1 for any further one (which then runs the chain).
static int sync_slot_of(hipStream_t s) {
  static std::mutex guard;
  static hipStream_t owner[kSyncSlots];
  static int used = 0;
  std::lock_guard<std::mutex> lock(guard);
  for (int i = 0; i < used; ++i)
    if (owner[i] == s)
      return i;
  if (used == kSyncSlots)
    return -1;
  owner[used] = s;
  return used++;
}

// Per-device address of the counters and CU count, looked up once (threads that race
// for the first look-up store the same values).
static int plan_device_state(int **sync, int *n_cus) {
  static std::atomic<int *> sync_of[64];
  int dev = -1;
  LPLB_HIP_TRY(hipGetDevice(&dev));
  LPLB_REQUIRE(dev >= 0 && dev < 64, LPLB_EUNSUPPORTED, "plan: device ordinal %d", dev);
  int *p = sync_of[dev].load(std::memory_order_acquire);
  if (!p) {
    LPLB_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(g_plan_sync)));
    sync_of[dev].store(p, std::memory_order_release);
  }
  *sync = p;
  *n_cus = current_device_cu_count();
  LPLB_REQUIRE(*n_cus > 0, LPLB_EHIP, "plan: cannot read the CU count of device %d", dev);
  return LPLB_OK;
}

// Tries the one-launch plan.  *done = false: shape or size outside what it covers.
static int try_one_launch(const int64_t *idx, int64_t n_elements, const int32_t *counts, const int32_t *r2o,
                          const int32_t *o2r, const int32_t *phy2log, int n_group, int G, int D, int C, int P,
                          int n_blocks, int32_t *counts_by_block, float *global_workload, float *o_weight,
                          int32_t *avail_num, int64_t *out, int32_t *physical_counts, int step_rule, int n_steps,
                          hipStream_t s, bool *done) {
  *done = false;
  const int L = P - D * C, n_fixed = L - D * C;
  const int n_logical = n_group * G * L;
  if (!g_cooperative || n_elements <= 0 || n_blocks < 2)
    return LPLB_OK;
  int gm = 0, dm = 0;
  if (!plan_lp_shape(G, D, &gm, &dm) || n_group > kLpsPerWorkgroup * kMaxLpWorkgroups ||
      n_group * G * D > kMaxShares || global_workload == nullptr)
    return LPLB_OK;
  // Shapes built for 16 waves also exist with 8: a slice workgroup's LDS grows with
  // waves x logical experts, and from about 400 experts on only 8 waves fit.
  int waves = plan_waves(gm, dm);
  if (waves == 16 && plan_lds_bytes(n_logical, 16) > (size_t)kPlanLdsLimit)
    waves = 8;
  const int n_lp_workgroups = (n_group + kLpsPerWorkgroup - 1) / kLpsPerWorkgroup;
  // own-histogram mode: the totals fit the accumulator (and with it the LDS)
  if (counts == nullptr && n_logical > kMaxTotals)
    return LPLB_OK;
  // slices of 1024 indices while kMaxSlices of them cover the batch, else of 2048, 4096,
  // 8192; at most n_blocks - 1 of them (the caller's bound on parallelism; the last row of
  // its table takes the totals)
  int64_t slices = kMaxSlices + 1;
  for (int64_t len = 1024; len <= (int64_t)waves * kChunksPerWave * kWave && slices > kMaxSlices; len *= 2)
    slices = (n_elements + len - 1) / len;
  if (slices > kMaxSlices)
    return LPLB_OK;
  if (slices > n_blocks - 1)
    slices = n_blocks - 1;
  const int64_t per = slice_len(n_elements, (int)slices);
  if (per > (int64_t)waves * kChunksPerWave * kWave || plan_lds_bytes(n_logical, waves) > (size_t)kPlanLdsLimit)
    return LPLB_OK;
  int *sync = nullptr, n_cus = 0;
  int rc = plan_device_state(&sync, &n_cus);
  if (rc != LPLB_OK)
    return rc;
  const int slot = sync_slot_of(s);
  // a quarter of the CUs for the slices, so that three plans that execute at once are all resident
  if (slices > n_cus / 4 || slot < 0)
    return LPLB_OK;
  sync += (size_t)slot * kSlotInts;

  PlanArgs a{};   // every field the host does not set below is zero
  a.idx = idx; a.n = n_elements; a.per = per; a.n_slices = (int)slices; a.n_lp_workgroups = n_lp_workgroups;
  a.o2r = o2r; a.phy2log = phy2log; a.rows = counts_by_block;
  a.totals = counts_by_block + (int64_t)(n_blocks - 1) * n_logical; a.out = out;
  a.physical_counts = physical_counts;
  a.sh = RedirectShape{n_logical, n_group * G, G, D, C, L, P};
  a.local_counts = counts == nullptr; a.sync = sync;
  SolveArgs &sa = a.solve;
  sa.workload = counts; sa.gw_out = global_workload; sa.r2o = r2o; sa.phy2log = phy2log;
  sa.avail = avail_num; sa.result = o_weight; sa.n_group = n_group; sa.G = G; sa.D = D; sa.C = C;
  sa.n_fixed = n_fixed; sa.n_experts = n_logical; sa.step_rule = step_rule; sa.n_steps = n_steps;
  sa.n_units = n_group; sa.staged_stride = 0;
  sa.tagged_result = reinterpret_cast<unsigned long long *>(sync + kSharesAt);
  sa.clocks = debug_clocks();

  hipError_t err = hipErrorInvalidValue;
#define LPLB_PLAN_CASE_W(GM, DM, W)                                                            \
  if (gm == GM && dm == DM && waves == W)                                                      \
    err = (G == GM && D == DM) ? launch_plan_shape<GM, DM, true, W>(a, s)                     \
                               : launch_plan_shape<GM, DM, false, W>(a, s);
  LPLB_PLAN_CASE_W(8, 1, 16) LPLB_PLAN_CASE_W(8, 1, 8) LPLB_PLAN_CASE_W(8, 2, 16) LPLB_PLAN_CASE_W(8, 2, 8)
  LPLB_PLAN_CASE_W(8, 4, 8) LPLB_PLAN_CASE_W(16, 1, 16) LPLB_PLAN_CASE_W(16, 1, 8) LPLB_PLAN_CASE_W(16, 2, 8)
  LPLB_PLAN_CASE_W(32, 1, 8) LPLB_PLAN_CASE_W(32, 2, 8)
#undef LPLB_PLAN_CASE_W
  LPLB_HIP_TRY(err);
  *done = true;
  return LPLB_OK;
}

} // namespace lplb

extern "C" int lplb_plan_set_cooperative(int enabled) {
  lplb::g_cooperative = enabled != 0;
  return LPLB_OK;
}

extern "C" int lplb_plan_sync_timeouts(int *count) {
  using namespace lplb;
  LPLB_REQUIRE(count != nullptr, LPLB_EINVAL, "plan_sync_timeouts: null pointer");
  int *sync = nullptr, n_cus = 0;
  int rc = plan_device_state(&sync, &n_cus);
  if (rc != LPLB_OK)
    return rc;
  *count = 0;
  for (int slot = 0; slot < kSyncSlots; ++slot) {
    int n = 0;
    LPLB_HIP_TRY(hipMemcpy(&n, sync + (size_t)slot * kSlotInts + 3, sizeof(int), hipMemcpyDeviceToHost));
    *count += n;
  }
  return LPLB_OK;
}

namespace lplb {

// The body of lplb_plan: argument checks, then the one-launch form or the chain.
static int plan_checked(const int64_t *idx, int64_t n_elements, const int32_t *global_counts, const int32_t *r2o,
                        const int32_t *o2r, const int32_t *phy2log, int n_group, int group_size, int dup_per_rank,
                        int n_combined_experts, int n_local_experts, int n_blocks, int32_t *counts_by_block,
                        float *global_workload, float *o_weight, int32_t *avail_num, int64_t *out,
                        int32_t *physical_counts, int step_rule, int n_steps, lplb_stream_t stream) {
  LPLB_REQUIRE(n_group > 0 && group_size > 0 && dup_per_rank > 0 && n_blocks > 0, LPLB_EINVAL,
               "plan: n_group=%d group_size=%d dup_per_rank=%d n_blocks=%d must be positive",
               n_group, group_size, dup_per_rank, n_blocks);
  const int L = n_local_experts - dup_per_rank * n_combined_experts;
  const int n_fixed = L - dup_per_rank * n_combined_experts;
  LPLB_REQUIRE(L > 0 && n_fixed >= 0 && n_combined_experts >= 0, LPLB_EINVAL,
               "plan: n_local_experts=%d does not fit %d x %d replicas", n_local_experts,
               dup_per_rank, n_combined_experts);
  LPLB_REQUIRE(counts_by_block != nullptr, LPLB_EINVAL, "plan: null counts_by_block");
  LPLB_REQUIRE(n_elements >= 0 && n_elements <= INT32_MAX && (idx || n_elements == 0), LPLB_EINVAL,
               "plan: bad idx / n_elements=%lld", (long long)n_elements);
  LPLB_REQUIRE((reinterpret_cast<uintptr_t>(idx) & 7) == 0, LPLB_EINVAL, "plan: idx must be 8-byte aligned");
  LPLB_REQUIRE(r2o && o2r && phy2log && o_weight && avail_num && (out || n_elements == 0), LPLB_EINVAL,
               "plan: null pointer");
  LPLB_REQUIRE(step_rule == LPLB_STEP_REFERENCE_WINDOW || step_rule == LPLB_STEP_FULL_MAX, LPLB_EINVAL,
               "plan: unknown step_rule %d", step_rule);
  LPLB_REQUIRE(n_steps >= 0, LPLB_EINVAL, "plan: n_steps=%d", n_steps);
  // refused before anything is enqueued, not by the last of the chain's kernels
  LPLB_REQUIRE(!(physical_counts && n_elements > (INT32_MAX - 41) / 499), LPLB_EUNSUPPORTED,
               "plan: physical_counts needs n_elements <= %d", (INT32_MAX - 41) / 499);
  const int n_logical = n_group * group_size * L;
  hipStream_t s = static_cast<hipStream_t>(stream);
  bool done = false;
  int rc = try_one_launch(idx, n_elements, global_counts, r2o, o2r, phy2log, n_group, group_size, dup_per_rank,
                          n_combined_experts, n_local_experts, n_blocks, counts_by_block, global_workload,
                          o_weight, avail_num, out, physical_counts, step_rule, n_steps, s, &done);
  if (rc != LPLB_OK || done)
    return rc;
  if (global_counts) {
    rc = lplb_solve(global_counts, global_workload, r2o, phy2log, n_group, group_size, dup_per_rank,
                    n_combined_experts, n_fixed, avail_num, o_weight, step_rule, n_steps, stream);
    if (rc != LPLB_OK)
      return rc;
    rc = enqueue_count(idx, n_elements, n_logical, n_blocks, counts_by_block, s, /*any_order=*/true);
    if (rc != LPLB_OK)
      return rc;
  } else {
    rc = lplb_count_idx(idx, n_elements, n_logical, n_blocks, counts_by_block, stream);
    if (rc != LPLB_OK)
      return rc;
    rc = lplb_solve(counts_by_block + (int64_t)(n_blocks - 1) * n_logical, global_workload, r2o, phy2log,
                    n_group, group_size, dup_per_rank, n_combined_experts, n_fixed, avail_num, o_weight,
                    step_rule, n_steps, stream);
    if (rc != LPLB_OK)
      return rc;
  }
  return lplb_map_idx(idx, o_weight, counts_by_block, o2r, phy2log, n_elements, n_group,
                      group_size, dup_per_rank, n_combined_experts, n_local_experts, n_blocks, out,
                      physical_counts, stream);
}

// ---- the plan for callers that cannot allocate ----
// The slice table of a plan (counts_by_block of lplb_plan: n_blocks rows of n_logical
// counters that the workgroups exchange) lives in this array instead of a buffer of the
// caller's.  Every GPU the library runs on holds its own copy until the process ends.
constexpr int64_t kScratchInts = 1 << 18;   // 1 MiB: e.g. 256 slices x 1024 logical experts
static __device__ __align__(256) int32_t scratch[kScratchInts];

// Device address of `scratch` on the current device, looked up once per device (the
// array's name is only a host-side handle; threads that race for the first look-up
// store the same value).
static int scratch_of_current_device(int32_t **ptr) {
  static std::atomic<int32_t *> scratch_of[64];
  int dev = -1;
  LPLB_HIP_TRY(hipGetDevice(&dev));
  LPLB_REQUIRE(dev >= 0 && dev < 64, LPLB_EUNSUPPORTED, "plan_noalloc: device ordinal %d", dev);
  int32_t *p = scratch_of[dev].load(std::memory_order_acquire);
  if (!p) {
    LPLB_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
    LPLB_REQUIRE(p != nullptr, LPLB_EHIP, "plan_noalloc: no device address for the slice table");
    scratch_of[dev].store(p, std::memory_order_release);
  }
  *ptr = p;
  return LPLB_OK;
}

__global__ void copy_ints(const int32_t *__restrict__ src, int32_t *__restrict__ dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    dst[i] = src[i];
}

} // namespace lplb

extern "C" int lplb_plan(const int64_t *idx, int64_t n_elements,
                         const int32_t *global_counts, const int32_t *r2o,
                         const int32_t *o2r, const int32_t *phy2log, int n_group,
                         int group_size, int dup_per_rank, int n_combined_experts,
                         int n_local_experts, int n_blocks, int32_t *counts_by_block,
                         float *global_workload, float *o_weight, int32_t *avail_num,
                         int64_t *out, int32_t *physical_counts, int step_rule, int n_steps,
                         lplb_stream_t stream) {
  return lplb::plan_checked(idx, n_elements, global_counts, r2o, o2r, phy2log, n_group, group_size, dup_per_rank,
                            n_combined_experts, n_local_experts, n_blocks, counts_by_block, global_workload,
                            o_weight, avail_num, out, physical_counts, step_rule, n_steps, stream);
}

extern "C" int lplb_plan_noalloc(const int64_t *idx, int64_t n_elements,
                                 const int32_t *global_counts, const int32_t *r2o,
                                 const int32_t *o2r, const int32_t *phy2log, int n_group,
                                 int group_size, int dup_per_rank, int n_combined_experts,
                                 int n_local_experts, int n_blocks, int32_t *local_counts,
                                 float *global_workload, float *o_weight, int32_t *avail_num,
                                 int64_t *out, int32_t *physical_counts, int step_rule, int n_steps,
                                 lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(n_group > 0 && group_size > 0 && dup_per_rank > 0 && n_blocks > 0 && n_combined_experts >= 0,
               LPLB_EINVAL, "plan_noalloc: n_group=%d group_size=%d dup_per_rank=%d n_blocks=%d must be positive",
               n_group, group_size, dup_per_rank, n_blocks);
  const int64_t L = (int64_t)n_local_experts - (int64_t)dup_per_rank * n_combined_experts;
  LPLB_REQUIRE(L > 0, LPLB_EINVAL, "plan_noalloc: n_local_experts=%d does not fit %d x %d replicas", n_local_experts,
               dup_per_rank, n_combined_experts);
  const int64_t n_logical = (int64_t)n_group * group_size * L;
  LPLB_REQUIRE((int64_t)n_blocks * n_logical <= kScratchInts, LPLB_EUNSUPPORTED,
               "plan_noalloc: n_blocks=%d x %lld logical experts = %lld counters exceed the built-in slice table of "
               "%lld; use fewer slices or lplb_plan with a workspace of your own",
               n_blocks, (long long)n_logical, (long long)((int64_t)n_blocks * n_logical), (long long)kScratchInts);
  int32_t *table = nullptr;
  int rc = scratch_of_current_device(&table);
  if (rc != LPLB_OK)
    return rc;
  // Nothing in the table has to start at zero: every row is written (by the slice that
  // owns it) before anything reads it, and rows beyond n_blocks are never read.
  rc = plan_checked(idx, n_elements, global_counts, r2o, o2r, phy2log, n_group, group_size, dup_per_rank,
                    n_combined_experts, n_local_experts, n_blocks, table, global_workload, o_weight, avail_num, out,
                    physical_counts, step_rule, n_steps, stream);
  if (rc != LPLB_OK || local_counts == nullptr)
    return rc;
  launch(copy_ints, dim3((unsigned)((n_logical + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
         table + (int64_t)(n_blocks - 1) * n_logical, local_counts, (int)n_logical);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}
