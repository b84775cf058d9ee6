// Whole plan in one call: histogram -> LP solve -> redirect on one stream.
//
// Two ways to run it.
//
// Chain: the three entry points' kernels one after the other (histogram, scan,
// LP, redirect).  With the global counts supplied the LP does not depend on this
// GPU's histogram: it is enqueued first and the histogram launch does not wait for
// it (it still starts after everything the LP launch waited for).
//
// One launch (plan_in_one_launch): every kernel boundary of the chain costs 3-5 us
// on this GPU although the kernels have 1-8 us of work, and the LP (8 us, one wave)
// sits on the critical path.  Here the LP workgroups (one per four LPs, first in the
// grid) and one workgroup per slice of the indices run side by side in a single grid:
//   slice workgroup: load indices (once; they stay in registers) -> LDS histogram and
//     per-chunk bitmaps of the replicated sets -> add the histogram to the batch's
//     totals and publish the slice's counts of the replicated sets -> wait until all
//     slices have -> tokens of each set before this slice and in the batch -> ordinals
//     and hashes -> wait for the LP's shares -> choose original or replica, store;
//   LP workgroup: (own-histogram mode: wait for the totals ->) solve -> publish the shares.
// What crosses workgroups is written and read with agent-scope atomics (plan_sync.h).
// The workgroups wait for each other, so the whole grid has to be resident: its size is
// bounded by what fits the GPU, and the host admits a launch only while the plans still
// executing leave room for it (it asks the runtime whether the streams that planned last
// still have work pending; it never waits); everything else runs as the chain.
// Nothing is cleared at the end of a launch (finding out which workgroup is the last costs
// two more round trips through memory on the critical path): a launch counter in device
// memory tags the shares and selects one of two sets of counters, and every launch clears,
// while it waits for its indices, the set that the launch before it used.
// Every wait is bounded all the same.  A wait that runs out is counted, the workgroup sends
// every token of its slice to the expert's original slot (which needs nothing from other
// workgroups), physical_counts is filled with -1 by the workgroup that writes them if it
// is among those, and the block of counters is marked as unusable: plans that use it later
// send every token to the original slot and count one more failure each, until
// lplb_plan_sync_timeouts has reported the failures and cleared the block.
#include "map_kernel.h"
#include "plan_sync.h"
#include "solve_kernel.h"
#include <atomic>
#include <mutex>
#include <stdio.h>

namespace lplb {

// Slices are 1024, 2048, ... indices long: the shortest of these with which this many slices
// cover the batch (about one workgroup per CU; with 64, batches of 0.25 to 1 M indices took
// up to 12 % longer).
constexpr int kPreferredSlices = 250;
constexpr int kPlanLdsLimit = 160 * 1024 - 8 * 1024;   // dynamic LDS; the kernel has static LDS besides
// An LP workgroup's dynamic LDS starts with the areas its (up to four) LP waves work in, then
// come the staged counts: per wave the pivot rows (2 * kWave doubles) and the assembly tile.
constexpr size_t plan_lp_area_bytes(int gm) {
  return 2 * kWave * sizeof(double) + (size_t)assembly_tile_floats_of(gm) * sizeof(float);
}
constexpr int kDefaultMaxPolls = 1 << 22;   // a few seconds of polling before a wait gives up
// LPs per LP workgroup: waves 0..3 of a workgroup sit on the CU's four SIMDs, and an LP
// wave is bound by instruction issue, so a fifth LP on the same CU would slow two of them
// down (8 LPs in one workgroup: 17.0 us per plan against 13.5 us).  Batches with more
// groups get more LP workgroups.
constexpr int kLpsPerWorkgroup = 4, kMaxLpWorkgroups = 8;

// One block of these per stream that plans (kSyncSlots of them per device):
//   [kGenAt] launches that have completed their exchange of counts; its parity p selects the
//   set of counters a launch uses, and (value + 1) tags what the LP publishes;
//   [kPoisonAt] non-zero: a wait ran out in this block (see above); [kTimeoutsAt] waits that
//   ran out since the library was loaded (never cleared);
//   [kDirtyAt + p] how many words of set p's totals the last launch that used it may have left non-zero;
//   [kAvailAt + 2 p] (8 bytes) who has touched the caller's counter of feasible LPs in the launch that uses
//   set p: bit k = LP k was feasible and has been (or is being) added, bit 32 = a wait ran out, so the
//   batch is not balanced as a whole and whoever set the bit took the LPs added so far back out; an LP
//   that finds bit 32 set does not add itself.  The reference's callers read "counter == number of
//   groups" as "this batch was balanced" (tests/test_solve.py:58, scripts/run_ep16_cube8p2e.py:61).
//   from kArrivedAt: workgroups that have published (slices) or started (LP): per set p,
//   kArrivalCopies copies of a striped counter (plan_sync.h);
//   from kSharesAt: the LP's shares as 8-byte words (tag << 32) | float bits with
//   tag = (launch tag << 2) | 1 (valid) or 2 (there will be none); a word with another
//   launch's tag is "not there yet"; up to kShareCopies copies, kMaxShares words apart: polls of
//   one line queue up in memory, so slice s polls copy s % copies;
//   from kTotalsAt: two sets of partial histograms of the batch, [p][copy][n_logical] 8-byte
//   words with the tokens in the high half and the number of slices that have contributed in
//   the low half (one atomic add delivers both, so whoever polls the words needs no second
//   round trip for a "done" counter).  Slice s adds its histogram to copy s % n_copies:
//   updates of one address queue up behind each other, so one copy per 16 slices (at most
//   kTotalCopies; more copies cost whoever adds them up more than they save: measured);
//   whoever needs the batch's tokens per expert adds the copies up.
constexpr int kGenAt = 0, kPoisonAt = 1, kTimeoutsAt = 4, kDirtyAt = 8, kAvailAt = 10;
constexpr unsigned long long kGaveUp = 1ull << 32;
constexpr int kSharesAt = 16, kMaxShares = 1024, kShareCopies = 8;
constexpr int kTotalsAt = kSharesAt + 2 * kMaxShares * kShareCopies, kMaxTotals = 1024, kTotalCopies = 16;
constexpr int kTotalsWords = kTotalCopies * kMaxTotals;   // 8-byte words of one set
constexpr int kArrivedAt = kTotalsAt + 2 * 2 * kTotalsWords;   // [2][kArrivalCopies][kArrivalCopyInts]
constexpr int kSlotInts = kArrivedAt + 2 * kArrivalCopies * kArrivalCopyInts, kSyncSlots = 8;
static_assert(kArrivedAt % 16 == 0 && kSlotInts % 16 == 0, "the counters' lines are 64-byte aligned");
static __device__ __attribute__((aligned(4096))) int g_plan_sync[kSyncSlots * kSlotInts];
static std::atomic<bool> g_cooperative{true};   // any thread may flip it while others plan
static std::atomic<long long> g_one_launch_plans{0};
// Test hook (lplb_plan_inject_fault): the next one-launch plan expects this many slices
// more than its grid has and gives up after this many polls.
static std::atomic<int> g_fault_extra_slices{0}, g_fault_max_polls{0};

struct PlanArgs {
  const int64_t *idx;
  int64_t n, per;
  int n_slices, n_lp_workgroups;
  int n_copies;          // partial histograms of the batch: a power of two, at most kTotalCopies
  int n_arrival_copies;  // copies of the arrival counter: a power of two, at most kArrivalCopies
  int n_share_copies;    // copies of the LP's shares: a power of two, at most kShareCopies
  int expected_slices;   // = n_slices unless a fault is injected
  int max_polls;
  const int32_t *o2r, *phy2log;
  int32_t *rows;     // [n_slices << row_shift] per slice: its tokens of each replicated set
  int row_shift;
  int32_t *totals;   // [n_logical] this GPU's tokens per expert, out
  int64_t *out;
  int32_t *physical_counts;   // [n_ranks * P] tokens per physical expert, or null
  int32_t *avail;
  RedirectShape sh;
  int n_rep;
  uint32_t magic_L, magic_cd, magic_D, magic_G;   // fast_div_magic of L, C * D, D, G
  SolveArgs solve;   // result = the shares (o_weight); workload is replaced by the totals if local_counts
  int local_counts;
  int *sync;
  int *arrived_word;   // pinned host memory, or null: receives arrived_seq once every workgroup of the launch has arrived
  int arrived_seq;
};

// A wait ran out: count it, switch the block of counters off, and make sure the caller's counter of
// feasible LPs does not vouch for this batch (the first to give up takes back what the LPs have added).
__device__ inline void give_up(const PlanArgs &a, unsigned long long *avail_state) {
  agent_add(a.sync + kTimeoutsAt, 1);
  agent_store(a.sync + kPoisonAt, 1);
  const unsigned long long before = __hip_atomic_fetch_or(avail_state, kGaveUp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int added = __popcll(before & 0xffffffffull);
  if (!(before & kGaveUp) && added > 0)
    atomicAdd(a.avail, -added);
}

// LDS of a slice workgroup: route and histogram per logical expert, a ranking record per
// (wave, replicated set), the constants of the sets.
static size_t plan_lds_bytes(int n_logical, int n_rep, int n_waves, int k) {
  return (size_t)(n_rep + 1) * sizeof(RepEntry) + (size_t)n_waves * (n_rep + 1) * rank_record_bytes_single(k) +
         (size_t)(n_logical + 1) * sizeof(Route) + (size_t)n_logical * sizeof(int32_t) +
         (size_t)(3 + n_waves) * n_rep * sizeof(int32_t) + 16;
}

// Debug builds: stamps of the first and the last slice workgroup and of the first LP workgroup.
#define LPLB_PLAN_STAMP(k)                                                                     \
  LPLB_STAMP_AT(a.solve.clocks == nullptr ? nullptr                                            \
                : blockIdx.x == a.n_lp_workgroups ? a.solve.clocks + 64                        \
                : blockIdx.x == gridDim.x - 1 ? a.solve.clocks + 80                            \
                : blockIdx.x == 0 ? a.solve.clocks + 96 : nullptr, k)

// Debug builds: stamps of every slice workgroup (the buffer must hold 128 + 8 * slices).
#ifdef LPLB_PHASE_CLOCKS
#define LPLB_SLICE_STAMP(k)                                                                    \
  do {                                                                                         \
    if (a.solve.clocks && threadIdx.x == 0)                                                    \
      a.solve.clocks[128 + 8 * (blockIdx.x - a.n_lp_workgroups) + (k)] = wall_clock64();       \
  } while (0)
#else
#define LPLB_SLICE_STAMP(k) do { } while (0)
#endif

// K: 64-index chunks per wave.  WAVES: waves per workgroup.
// Registers: with LP shapes that fit 128 VGPRs the kernel as a whole is held to 128 (four
// waves per SIMD: one 16-wave or two 8-wave workgroups per CU), which is what lets the 257
// workgroups of a [262144 x 8] batch be resident together.
template <int GM, int DM, bool EXACT, int K, int WAVES>
__global__ __launch_bounds__(WAVES *kWave, (GM * DM <= 16 && GM <= 8) ? 4 : 2) void plan_in_one_launch(PlanArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ int rep_of_edge_all[kLpsPerWorkgroup * kWave];
  __shared__ int flags[2];   // [0] the exchange of counts worked, [1] some share will not come
  const int nl = a.sh.n_logical, R = a.n_rep;
  const int tid = threadIdx.x;
  constexpr int nt = WAVES * kWave;
  const int lane = tid % kWave;
  const int wave_s = __builtin_amdgcn_readfirstlane(tid / kWave);   // wave-uniform
  const int pid = blockIdx.x;
  // Which launch of this block of counters this is (the same value in every workgroup: it
  // is advanced only once all of them have read it), and whether the block is switched off.
  const int gen = agent_load(a.sync + kGenAt);
  const bool poisoned = agent_load(a.sync + kPoisonAt) != 0;
  const int parity = gen & 1;
  const uint32_t tag_valid = (((uint32_t)gen + 1u) << 2) | 1u, tag_none = tag_valid + 1u;
  int *arrived_stripes = a.sync + kArrivedAt + parity * (kArrivalCopies * kArrivalCopyInts);
  unsigned long long *shares = reinterpret_cast<unsigned long long *>(a.sync + kSharesAt);
  unsigned long long *avail_state = reinterpret_cast<unsigned long long *>(a.sync + kAvailAt) + parity;
  unsigned long long *totals_acc =
      reinterpret_cast<unsigned long long *>(a.sync + kTotalsAt) + (size_t)parity * kTotalsWords;   // [n_copies][nl]
  // The batch's tokens of expert e and the number of slices that have contributed: the copies
  // added up (all loads in flight together); complete once every slice has arrived.
  auto batch_totals = [&](int e, int32_t &tokens, int32_t &slices) {
    unsigned long long sum = 0;
    if (a.n_copies <= 4) {   // (short batches: a quarter of the loads per look)
      unsigned long long v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        v[k] = agent_load(totals_acc + (k & (a.n_copies - 1)) * nl + e);
#pragma unroll
      for (int k = 0; k < 4; ++k)
        sum += k < a.n_copies ? v[k] : 0ull;
    } else {
      unsigned long long v[kTotalCopies];
#pragma unroll
      for (int k = 0; k < kTotalCopies; ++k)
        v[k] = agent_load(totals_acc + (k & (a.n_copies - 1)) * nl + e);
#pragma unroll
      for (int k = 0; k < kTotalCopies; ++k)
        sum += k < a.n_copies ? v[k] : 0ull;
    }
    tokens = (int32_t)(sum >> 32);
    slices = (int32_t)(uint32_t)sum;
  };

  if (pid < a.n_lp_workgroups) {
    // ------------------------------------------------------------ the LPs
    SolveArgs sa = a.solve;
    const int first_lp = pid * kLpsPerWorkgroup;          // of this workgroup
    const int n_lps = min(kLpsPerWorkgroup, sa.n_units - first_lp);
    LPLB_PLAN_STAMP(0);
    // Own-histogram mode: the LP waves start at once (their table loads do not need
    // the counts) and pick the counts up from LDS; the wave after them waits for the
    // slices, fetches the totals the slices have added up in memory and hands them over.
    __shared__ int counts_ready;
    // dynamic LDS of an LP workgroup: [LP wave][pivot rows | assembly tile], then the counts
    constexpr size_t kLpArea = plan_lp_area_bytes(GM);
    static_assert(kLpArea % 16 == 0, "the LP waves' areas keep 16-byte alignment");
    unsigned char *my_area = smem_raw + (size_t)min(wave_s, kLpsPerWorkgroup - 1) * kLpArea;
    float *staged = reinterpret_cast<float *>(smem_raw + kLpsPerWorkgroup * kLpArea);
    if (tid == 0)
      counts_ready = 0;
    __syncthreads();
    // This workgroup has read the launch counter: the first slice may advance it once
    // every workgroup has said so.  (The last wave says it: the LP waves do not wait for
    // the counter to arrive before they start.)
    if (wave_s == WAVES - 1)
      announce_arrival(arrived_stripes, a.n_arrival_copies, a.n_slices + pid);
    sa.tag_valid = tag_valid;
    if (a.local_counts) {
      sa.counts_ready = &counts_ready;
      // strictly longer than the poller's own wait (whose polls are each many loads long): the poller is
      // the one that gives up and says so
      sa.counts_wait_polls = a.max_polls < (INT32_MAX >> 6) ? a.max_polls << 6 : INT32_MAX;
      if (wave_s == n_lps) {
        // Poll the batch's totals until every expert's words say that all slices have
        // added theirs.
        bool complete = false;
        for (int polls = 0; polls < a.max_polls && !complete && !poisoned; ++polls) {   // (switched off: no slice will publish)
          bool all_in = true;
          for (int e = lane; e < nl; e += kWave) {
            int32_t tokens, slices;
            batch_totals(e, tokens, slices);
            all_in = all_in && slices == a.expected_slices;
            staged[e] = (float)tokens;
          }
          complete = __all(all_in);
          if (!complete)
            __builtin_amdgcn_s_sleep(2);
        }
        if (!complete && !poisoned && lane == 0)
          give_up(a, avail_state);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0)
          __hip_atomic_store(&counts_ready, complete ? 1 : 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
    LPLB_PLAN_STAMP(1);
    if (wave_s < n_lps) {
      // (own-histogram mode: every LP of the batch reads the one staged copy)
      float *mine = a.local_counts ? staged : staged + (size_t)wave_s * sa.staged_stride;
      const int n_ok = solve_lp<GM, DM, EXACT, 1>(sa, first_lp + wave_s, mine, rep_of_edge_all + wave_s * kWave,
                                                  reinterpret_cast<double *>(my_area),
                                                  reinterpret_cast<float *>(my_area + 2 * kWave * sizeof(double)));
      if (n_ok < 0) {
        // no counts, no solution: tell the slices not to wait for this LP's shares.  (If it was this wave's
        // own wait that ran out and not the poller's, nobody has counted the failure yet.)
        if (lane == 0 && !poisoned &&
            __hip_atomic_load(&counts_ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 2)
          give_up(a, avail_state);
        const int n_edges = sa.G * sa.D;
        for (int j = lane; j < n_edges; j += kWave)
          for (int k = 0; k < a.n_share_copies; ++k)
            agent_store(shares + (int64_t)k * kMaxShares + (int64_t)(first_lp + wave_s) * n_edges + j,
                        (unsigned long long)tag_none << 32);
      } else if (lane == 0 && n_ok > 0 && !poisoned) {
        // feasible: count it for the caller unless some workgroup has already given up on this batch
        const unsigned long long before = __hip_atomic_fetch_or(avail_state, 1ull << (first_lp + wave_s), __ATOMIC_RELAXED,
                                                                 __HIP_MEMORY_SCOPE_AGENT);
        if (!(before & kGaveUp))
          atomicAdd(a.avail, n_ok);
      }
    }
    LPLB_PLAN_STAMP(2);
    return;
  }

  // --------------------------------------------------------------- a slice
  constexpr int kRec = rank_record_bytes_single(K);
  const int slice = pid - a.n_lp_workgroups;
  RepEntry *reps = reinterpret_cast<RepEntry *>(smem_raw);                          // [R + 1]
  unsigned char *records = smem_raw + (size_t)(R + 1) * sizeof(RepEntry);          // [WAVES][R + 1][kRec]
  const int wave_stride = (R + 1) * kRec;
  Route *route = reinterpret_cast<Route *>(records + (size_t)WAVES * wave_stride);  // [nl + 1]
  int32_t *hist = reinterpret_cast<int32_t *>(route + nl + 1);                      // [nl]
  int32_t *set_expert = hist + nl;                                                  // [R]
  int32_t *before = set_expert + R;                                                 // [R] tokens of the set before this slice
  int32_t *total = before + R;                                                      // [R] ... in the whole batch
  int32_t *wave_total = total + R;                                                  // [WAVES][R] ... in each wave's chunks, then in the chunks of the waves before it
  unsigned char *my_records = records + (size_t)wave_s * wave_stride;
  const unsigned long long my_bit = 1ull << lane;
  const int64_t begin = slice_begin(a.n, a.per, slice);
  const int64_t end = slice_begin(a.n, a.per, slice + 1);
  const int cd = a.sh.C * a.sh.D;
  LPLB_PLAN_STAMP(0);
  LPLB_SLICE_STAMP(0);
  // Where a slice shares a CU with an LP workgroup (grids with more workgroups than CUs), its
  // waves go first: the LP wave issues an instruction nearly every cycle it may, and a slice
  // wave on the same SIMD would be starved for as long as the LP runs, with every other slice
  // waiting for it.  The slices spend most of their time asleep, so the LP loses little.
  __builtin_amdgcn_s_setprio(2);

  // ---- small table reads first (they need no counts), then the index loads; all of
  // them unconditional loads from clamped addresses, so that nothing waits here ----
  auto slot_of = [&](int e) { return e + (int)fast_div((uint32_t)e, a.magic_L) * (a.sh.P - a.sh.L); };
  struct SetOf {
    int ep_rank, place, d, group_rank;
  };
  auto set_of = [&](int i) {
    SetOf s;
    s.ep_rank = (int)fast_div((uint32_t)i, a.magic_cd);
    s.place = i - s.ep_rank * cd;
    s.d = s.place - (int)fast_div((uint32_t)s.place, a.magic_D) * a.sh.D;
    s.group_rank = s.ep_rank - (int)fast_div((uint32_t)s.ep_rank, a.magic_G) * a.sh.G;
    return s;
  };
  const int dirty0 = agent_load(a.sync + kDirtyAt), dirty1 = agent_load(a.sync + kDirtyAt + 1);
  const int e0 = min(tid, nl - 1);
  const int slot0 = slot_of(e0);
  const int le0 = a.phy2log[slot0];
  const bool set0 = tid < R;
  const SetOf s0 = set_of(set0 ? tid : 0);
  const int rle0 = a.phy2log[s0.ep_rank * a.sh.P + s0.place];
  const int host0 = a.o2r[s0.group_rank * a.sh.D + s0.d];
  const int64_t w0 = begin + (int64_t)wave_s * (K * kWave);   // first index of this wave's K chunks (uniform)
  const bool whole = w0 + K * kWave <= end;
  int64_t raw[K];
  {
    const int64_t *src = a.idx + w0 + lane;
    if (whole) {
#pragma unroll
      for (int c = 0; c < K; ++c)
        raw[c] = __builtin_nontemporal_load(src + c * kWave);
    } else {
#pragma unroll
      for (int c = 0; c < K; ++c)
        raw[c] = w0 + c * kWave + lane < end ? __builtin_nontemporal_load(src + c * kWave) : -1;
    }
  }

  // ---- tables that need phy2log only: where an expert's tokens go when nothing is
  // redirected, and which replicated set (if any) it belongs to; minilp.cu:466-496 ----
  for (int e = tid; e <= nl; e += nt)
    route[e] = Route{-1, R};
  for (int e = tid; e < nl; e += nt)
    hist[e] = 0;
  {
    const i32x4 zero{0, 0, 0, 0};
    i32x4 *z = reinterpret_cast<i32x4 *>(records);
    for (int i = tid; i < WAVES * wave_stride / 16; i += nt)
      z[i] = zero;
  }
  for (int q = tid; q < R; q += nt) {
    before[q] = 0;
    total[q] = 0;
  }
  if (tid == 0) {
    reps[R] = RepEntry{1, 0xffffffffu, INT32_MAX, -1};   // "no replica": every token stays
    flags[0] = 0;
    flags[1] = 0;
  }
  __syncthreads();
  if (tid < nl && le0 >= 0 && le0 < nl)
    route[le0].original = slot0;
  for (int e = tid + nt; e < nl; e += nt) {
    const int s = slot_of(e), le = a.phy2log[s];
    if (le >= 0 && le < nl)
      route[le].original = s;
  }
  // A set's key is R - 1 - i, so that of two sets that name the same expert the later one
  // wins (as a sequential pass over the sets would have it) with an atomic min.
  auto enter_set = [&](int i, const SetOf &s, int le, int host) {
    const bool ok = le >= 0 && le < nl;
    if (ok)
      atomicMin(&route[le].rep, R - 1 - i);
    reps[R - 1 - i] = RepEntry{0, 0u, 0, ((s.ep_rank - s.group_rank) + host + 1) * a.sh.P - cd + s.place};
    set_expert[R - 1 - i] = ok ? le : -1;
  };
  if (set0)
    enter_set(tid, s0, rle0, host0);
  for (int i = tid + nt; i < R; i += nt) {
    const SetOf s = set_of(i);
    enter_set(i, s, a.phy2log[s.ep_rank * a.sh.P + s.place], a.o2r[s.group_rank * a.sh.D + s.d]);
  }
  // ---- housekeeping while the indices are on their way: the set of counters that the
  // launch before this one used (nobody looks at it during this launch) is cleared for the
  // launch after this one, every slice taking its part; the stores only have to be done
  // when the kernel ends ----
  if (!poisoned) {
    const int dirty_words = min(parity ? dirty0 : dirty1, kTotalsWords);   // of the set with the other parity
    unsigned long long *stale = reinterpret_cast<unsigned long long *>(a.sync + kTotalsAt) + (size_t)(1 - parity) * kTotalsWords;
    for (int i = slice * nt + tid; i < dirty_words; i += a.n_slices * nt)
      agent_store(stale + i, 0ull);
    if (slice == 0) {
      if (tid < kArrivalCopies * kArrivalStripes)
        agent_store(a.sync + kArrivedAt + ((1 - parity) * kArrivalCopies + tid / kArrivalStripes) * kArrivalCopyInts +
                        (tid % kArrivalStripes) * kArrivalStripeInts, 0);
      if (tid == 0) {
        agent_store(a.sync + kDirtyAt + parity, a.n_copies * nl);
        agent_store(reinterpret_cast<unsigned long long *>(a.sync + kAvailAt) + (1 - parity), 0ull);
      }
    }
  }
  __syncthreads();
  LPLB_PLAN_STAMP(10);

  // ---- the tokens: histogram of the slice, bitmaps of the replicated sets per chunk ----
  // Between the phases a token is kept as its expert id only, two ids per register (the
  // route is looked up again where it is needed): the waits below are long and registers
  // are what bounds how many workgroups are resident.
  uint32_t packed[(K + 1) / 2];
  auto expert_of_chunk = [&](int c) { return (int)((packed[c / 2] >> (16 * (c % 2))) & 0xffffu); };
  auto slot_of_chunk = [&](int set, int c) {
    return reinterpret_cast<ChunkSlot *>(my_records + __umul24((uint32_t)set, (uint32_t)kRec)) + c;
  };
#pragma unroll
  for (int c = 0; c < K; ++c) {
    const bool valid = (uint64_t)raw[c] < (uint64_t)nl;   // -1, other negatives and too large ids fail
    const int e = valid ? (int)raw[c] : nl;
    packed[c / 2] = (c % 2) ? packed[c / 2] | ((uint32_t)e << 16) : (uint32_t)e;
    const int set = route[e].rep;
    // a token of a replicated set is counted through the set's bitmaps (the sets hold the hot
    // experts, whose tokens would queue up at one histogram counter), any other one here
    if (set < R)
      atomicOr(reinterpret_cast<unsigned long long *>(slot_of_chunk(set, c)), my_bit);
    else if (valid)
      atomicAdd(&hist[e], 1);
  }
  __syncthreads();
  LPLB_PLAN_STAMP(8);
  LPLB_SLICE_STAMP(1);
  // ---- inside the wave: tokens of each set in the chunks before each chunk (lane = (set,
  // chunk), chunk fastest), and in all of the wave's chunks ----
  if (R > 0) {
    const int c = lane % K;
    for (int p0 = 0; p0 < R * K; p0 += kWave) {
      const bool live = p0 + lane < R * K;
      const int q = live ? (p0 + lane) / K : R;   // lanes past the end read the stand-in record (zeros)
      ChunkSlot *mine = reinterpret_cast<ChunkSlot *>(my_records + __umul24((uint32_t)q, (uint32_t)kRec)) + c;
      const int own = __popcll(*reinterpret_cast<const unsigned long long *>(mine));
      const int in_my_wave = group_sum<K>(own);
      const int in_earlier_chunks = group_exclusive_scan<K>(own, c);
      if (live) {
        mine->start = in_earlier_chunks;
        if (c == 0)
          wave_total[wave_s * R + q] = in_my_wave;
      }
    }
  }
  __syncthreads();
  for (int q = tid; q < R; q += nt) {   // the sets' tokens in this slice, into the histogram
    int32_t n = 0, of_wave[WAVES];
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
      of_wave[w] = wave_total[w * R + q];
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {   // (each wave's count becomes the count of the waves before it)
      wave_total[w * R + q] = n;
      n += of_wave[w];
    }
    const int le = set_expert[q];
    if (le >= 0 && route[le].rep == q)   // (of two sets that name the same expert only one has the tokens)
      hist[le] = n;
  }
  __syncthreads();
  // ---- this slice's counts, for every workgroup: the histogram goes into the batch's
  // totals, the counts of the replicated sets into this slice's row ----
  LPLB_PLAN_STAMP(9);
  if (!poisoned) {
    for (int e = tid; e < nl; e += nt) {
      const int32_t mine = hist[e];
      if (a.local_counts || mine != 0)   // (only the LP's poller looks at the number of contributions)
        agent_add(totals_acc + (slice & (a.n_copies - 1)) * nl + e, ((unsigned long long)(uint32_t)mine << 32) | 1ull);
    }
    for (int q = tid; q < R; q += nt) {
      const int le = set_expert[q];
      agent_store(a.rows + (((int64_t)slice) << a.row_shift) + q, le >= 0 ? hist[le] : 0);
    }
    stores_have_landed();
  }
  __syncthreads();
  LPLB_PLAN_STAMP(1);
  LPLB_SLICE_STAMP(2);
  if (wave_s == 0) {
    if (poisoned) {
      if (slice == 0 && lane == 0)
        agent_add(a.sync + kTimeoutsAt, 1);   // one more plan that this block of counters could not serve
    } else {
      announce_arrival(arrived_stripes, a.n_arrival_copies, slice);
      const bool arrived = wait_for_arrivals(arrived_stripes + (slice & (a.n_arrival_copies - 1)) * kArrivalCopyInts,
                                             a.expected_slices + a.n_lp_workgroups, a.max_polls);
      if (lane == 0) {
        if (!arrived)
          give_up(a, avail_state);
        else if (slice == 0) {
          agent_store(a.sync + kGenAt, (gen + 1) & 0x3fffffff);   // every workgroup has read it by now
          // From here on no workgroup of this launch waits for one that is not resident yet: tell the host, which
          // then stops counting this launch against what the GPU can hold at once (a posted write to host memory).
          if (a.arrived_word)
            __hip_atomic_store(a.arrived_word, a.arrived_seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        flags[0] = arrived;
      }
    }
  }
  __syncthreads();
  LPLB_PLAN_STAMP(2);
  LPLB_SLICE_STAMP(4);
  bool ok = flags[0] != 0;   // (the same in every thread)
  // Hashes of this thread's tokens: worked out while the LP is still running where a
  // thread has few tokens (short batches, where the LP is the longest chain); with many
  // tokens per thread they are worked out at the end, one token at a time, which keeps the
  // kernel inside the registers that let two workgroups share a CU.
  constexpr bool kHashEarly = K <= 4;
  int32_t h[kHashEarly ? K : 1];
  auto hash_of_chunk = [&](int c) {
    const int set = route[expert_of_chunk(c)].rep;
    const i32x4 s = *reinterpret_cast<const i32x4 *>(slot_of_chunk(set, c));   // bits_lo, bits_hi, start
    const i32x4 x = *reinterpret_cast<const i32x4 *>(&reps[set]);              // total, magic, -, -
    const int32_t k =
        __builtin_amdgcn_mbcnt_hi((uint32_t)s.y, __builtin_amdgcn_mbcnt_lo((uint32_t)s.x, (uint32_t)s.z));
    return ordinal_hash<false>(k, x.x, (uint32_t)x.y);
  };
  if (ok) {
    // ---- tokens of each replicated set before this slice and in the whole batch: a thread
    // takes one set of every (threads / row length)-th slice, loads in batches ----
    {
      const int row_len = 1 << a.row_shift;
      const int q_lanes = min(row_len, nt), p_lanes = nt / q_lanes;   // powers of two
      const int p_first = tid / q_lanes;
      constexpr int kInFlight = 8;
      for (int q = tid % q_lanes; q < R; q += q_lanes) {
        int32_t t_sum = 0, b_sum = 0;
        for (int p0 = p_first; p0 < a.n_slices; p0 += kInFlight * p_lanes) {
          int32_t v[kInFlight];
#pragma unroll
          for (int k = 0; k < kInFlight; ++k)
            v[k] = agent_load(a.rows + ((((int64_t)min(p0 + k * p_lanes, a.n_slices - 1)) << a.row_shift) + q));
#pragma unroll
          for (int k = 0; k < kInFlight; ++k) {
            const int p = p0 + k * p_lanes;
            t_sum += p < a.n_slices ? v[k] : 0;
            b_sum += p < slice ? v[k] : 0;
          }
        }
        // lanes of a wave that hold the same set add up first (updates of one LDS word queue up)
        for (int m = q_lanes; m < kWave; m <<= 1) {
          t_sum += __shfl_xor(t_sum, m);
          b_sum += __shfl_xor(b_sum, m);
        }
        if (lane < q_lanes) {
          atomicAdd(&total[q], t_sum);
          atomicAdd(&before[q], b_sum);
        }
      }
    }
    if (slice == 0)   // this GPU's tokens per expert, for the caller (and for the counts below)
      for (int e = tid; e < nl; e += nt) {
        int32_t tokens, slices;
        batch_totals(e, tokens, slices);
        a.totals[e] = tokens;
        hist[e] = tokens;
      }
    __syncthreads();
    LPLB_PLAN_STAMP(3);
    for (int q = tid; q < R; q += nt) {
      const int32_t t = total[q];
      reps[q].total = t;
      reps[q].magic = t >= 1 ? 0xffffffffu / (uint32_t)t : 0u;
    }
    // ---- ordinal of the first token of every (wave, set, chunk): what is there already
    // (tokens in the wave's earlier chunks) plus the tokens before this slice and in the
    // waves before this one ----
    if (R > 0) {
      const int c = lane % K;
      for (int p0 = 0; p0 < R * K; p0 += kWave) {
        const bool live = p0 + lane < R * K;
        const int q = live ? (p0 + lane) / K : 0;
        const int32_t base = before[q] + wave_total[wave_s * R + q];
        if (live)
          atomicAdd(&(reinterpret_cast<ChunkSlot *>(my_records + __umul24((uint32_t)q, (uint32_t)kRec)) + c)->start, base);
      }
    }
    __syncthreads();
    LPLB_PLAN_STAMP(4);
    // ---- ordinals and hashes of the tokens, while the LP is still running ----
    if constexpr (kHashEarly) {
#pragma unroll
      for (int c = 0; c < K; ++c)
        h[c] = hash_of_chunk(c);
    }
    // ---- the LP's shares: every set's thread polls its own; value and tag arrive in
    // the same 8-byte word ----
    for (int i = tid; i < R; i += nt) {
      const SetOf s = set_of(i);
      unsigned long long word = 0;
      int polls = 0;
      uint32_t tag = 0;
      while ((tag = (uint32_t)((word = agent_load(shares + (slice & (a.n_share_copies - 1)) * kMaxShares + s.ep_rank * a.sh.D + s.d)) >> 32)) != tag_valid &&
             tag != tag_none && ++polls < a.max_polls)
        __builtin_amdgcn_s_sleep(2);
      if (tag == tag_valid) {
        reps[R - 1 - i].expected = expected_on_original(__builtin_bit_cast(float, (uint32_t)word), total[R - 1 - i]);
      } else {
        if (tag != tag_none)
          give_up(a, avail_state);
        flags[1] = 1;
      }
    }
    __syncthreads();
    LPLB_PLAN_STAMP(5);
    ok = flags[1] == 0;
  }
  // Tokens per physical expert (= bincount of the output) from the first slice's tables.
  if (slice == 0 && a.physical_counts && ok) {
    for (int i = tid; i < a.sh.n_ranks * a.sh.P; i += nt) {
      const int le = a.phy2log[i];
      int32_t v = 0;
      if (le >= 0 && le < nl) {
        const Route rt = route[le];
        if (rt.rep >= R) {
          v = rt.original == i ? hist[le] : 0;   // (slice 0 keeps the batch's totals there)
        } else {
          const RepEntry x = reps[rt.rep];
          const int32_t kept = kept_on_original(x.total, x.expected);
          v = rt.original == i ? kept : (x.replica == i ? x.total - kept : 0);
        }
      }
      a.physical_counts[i] = v;
    }
  }
  if (slice == 0 && a.physical_counts && !ok)
    for (int i = tid; i < a.sh.n_ranks * a.sh.P; i += nt)
      a.physical_counts[i] = -1;
  LPLB_PLAN_STAMP(6);
  // ---- choose and store; if a wait ran out, every token goes to its original slot ----
  {
    int64_t *dst = a.out + w0 + lane;
    int32_t o[K];
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const Route rt = route[expert_of_chunk(c)];
      o[c] = rt.original;
      if (ok) {
        const RepEntry x = reps[rt.rep];
        o[c] = (kHashEarly ? h[c] : hash_of_chunk(c)) >= x.expected ? x.replica : rt.original;
      }
    }
    if (whole) {
#pragma unroll
      for (int c = 0; c < K; ++c)
        __builtin_nontemporal_store((int64_t)o[c], dst + c * kWave);
    } else {
#pragma unroll
      for (int c = 0; c < K; ++c)
        if (w0 + c * kWave + lane < end)
          __builtin_nontemporal_store((int64_t)o[c], dst + c * kWave);
    }
  }
  LPLB_PLAN_STAMP(7);
  LPLB_SLICE_STAMP(3);
}

// LP shapes the one-launch plan is built for, in the order they are tried, and the
// workgroup size that leaves the LP its registers: 128 VGPRs per lane at 16 waves,
// 256 at 8.
constexpr int kPlanShapes[][2] = {{8, 1}, {8, 2}, {8, 4}, {16, 1}, {16, 2}, {32, 1}, {32, 2}};
constexpr int plan_waves(int gm, int dm) { return (gm * dm <= 16 && gm <= 8) ? 16 : 8; }
constexpr int plan_max_chunks(int waves) { return waves == 16 ? 8 : 16; }   // longest slice: 8192 indices
static bool plan_lp_shape(int G, int D, int *gm, int *dm) {
  for (const auto &shape : kPlanShapes)
    if (G <= shape[0] && D <= shape[1]) {
      *gm = shape[0];
      *dm = shape[1];
      return true;
    }
  return false;
}

// ---- host side: which launches may run as one kernel ----
// Per device: the counters' address and, per slot, which stream owns it and what its
// launches cost.  A slot belongs to one stream at a time (launches that share a slot must
// not overlap, which stream order guarantees); a slot whose stream has no work pending may
// pass to another stream.  A slot with a launch captured into a graph stays with its stream
// for good and counts as executing for good: a replay may come at any time and the host
// does not see it.
struct PlanSlot {
  hipStream_t stream = nullptr;
  int seq = 0;                  // number of the slot's latest launch outside a capture (what it writes when all
                                // of its workgroups have arrived)
  float cost = 0.0f;            // share of the GPU's resident workgroups its launches take
  bool used = false, captured = false;
  bool maybe_executing = false; // a launch was enqueued and has not been seen to have arrived since
};
struct PlanDevice {
  int *sync = nullptr;
  int *arrived = nullptr;       // pinned host memory, one word per slot, written by the kernels (see PlanArgs)
  int n_cus = 0;
  PlanSlot slots[kSyncSlots];
};
static std::mutex g_plan_guard;
static PlanDevice g_plan_devices[64];
// Up to this share of the GPU's resident workgroups may belong to plans that wait for
// their own workgroups; the rest stays free for their stragglers and for other kernels.
constexpr float kResidencyBudget = 0.80f;

// Looks the per-device state up.
static int plan_device(PlanDevice **out) {
  int dev = -1;
  LPLB_HIP_TRY(hipGetDevice(&dev));
  LPLB_REQUIRE(dev >= 0 && dev < 64, LPLB_EUNSUPPORTED, "plan: device ordinal %d", dev);
  PlanDevice &d = g_plan_devices[dev];
  static std::mutex first_use;
  std::lock_guard<std::mutex> lock(first_use);
  if (!d.sync) {
    int *sync = nullptr;
    LPLB_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&sync), HIP_SYMBOL(g_plan_sync)));
    d.n_cus = current_device_cu_count();
    LPLB_REQUIRE(d.n_cus > 0, LPLB_EHIP, "plan: cannot read the CU count of device %d", dev);
    LPLB_HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&d.arrived), kSyncSlots * sizeof(int), hipHostMallocDefault));
    for (int i = 0; i < kSyncSlots; ++i)
      d.arrived[i] = 0;
    d.sync = sync;
  }
  *out = &d;
  return LPLB_OK;
}

// May a launch of this slot still need room on the GPU?  Once all workgroups of a launch have arrived none of
// them waits for a workgroup that is not resident, and the launch says so in a word of pinned host memory:
// looking at it asks nothing of the runtime, the stream (which other threads may be capturing on, or may
// have destroyed) is not touched, and nothing waits.
static bool slot_is_executing(PlanDevice &d, int i) {
  PlanSlot &s = d.slots[i];
  if (!s.used)
    return false;
  if (s.captured)
    return true;
  if (s.maybe_executing && __atomic_load_n(d.arrived + i, __ATOMIC_ACQUIRE) == s.seq)
    s.maybe_executing = false;
  return s.maybe_executing;
}

// Admission of one launch that takes `cost` of the GPU's resident workgroups on stream s.
// Returns the slot, or -1: run the chain.
static int admit_launch(PlanDevice &d, hipStream_t s, float cost, bool capturing) {
  int slot = -1;
  for (int i = 0; i < kSyncSlots && slot < 0; ++i)
    if (d.slots[i].used && d.slots[i].stream == s)
      slot = i;
  for (int i = 0; i < kSyncSlots && slot < 0; ++i)
    if (!d.slots[i].used)
      slot = i;
  for (int i = 0; i < kSyncSlots && slot < 0; ++i)
    if (!slot_is_executing(d, i))
      slot = i;
  if (slot < 0)
    return -1;
  float executing = 0.0f;
  for (int i = 0; i < kSyncSlots; ++i)
    if (i != slot && slot_is_executing(d, i))
      executing += d.slots[i].cost;
  if (executing + cost > kResidencyBudget)
    return -1;
  PlanSlot &ps = d.slots[slot];
  if (!ps.used || ps.stream != s) {
    ps.stream = s;
    ps.cost = 0.0f;
    ps.used = true;
    ps.captured = ps.maybe_executing = false;
  }
  ps.cost = ps.captured ? (cost > ps.cost ? cost : ps.cost) : cost;
  ps.captured = ps.captured || capturing;
  return slot;
}

// Workgroups of one kernel variant that fit a CU: bounded by the vector registers (512 per
// SIMD lane, allocated in blocks of 8, at most 8 waves per SIMD) and by the LDS (160 KiB per
// CU).  Worked out from the kernel's own attributes; the runtime's occupancy query changes
// its answer once a kernel has been allowed more than 64 KiB of dynamic LDS.
struct KernelFootprint {   // one per kernel variant (a static of launch_plan_variant)
  std::atomic<int> regs{-1}, static_lds{0};
};
static int workgroups_per_cu(const void *kernel, KernelFootprint &known, int waves, size_t lds) {
  int regs = known.regs.load(std::memory_order_acquire);
  if (regs < 0) {
    hipFuncAttributes attr;
    if (hipFuncGetAttributes(&attr, kernel) != hipSuccess || attr.numRegs <= 0)
      return 0;
    known.static_lds.store((int)attr.sharedSizeBytes, std::memory_order_relaxed);
    regs = attr.numRegs;
    known.regs.store(regs, std::memory_order_release);
  }
  const int per_wave = (regs + 7) / 8 * 8;
  const int waves_per_simd = min(8, 512 / per_wave);
  const int by_registers = waves_per_simd * 4 / waves;
  const int by_lds = (int)((size_t)(160 * 1024) / (lds + (size_t)known.static_lds.load(std::memory_order_relaxed) + 256));
  return min(by_registers, by_lds);
}

// Launches one variant if the whole grid fits the GPU beside the plans that are still
// executing.  *done = false: it does not; nothing was enqueued.
template <int GM, int DM, bool EXACT, int K, int WAVES>
static int launch_plan_variant(PlanArgs &a, size_t lds, hipStream_t s, bool *done) {
  auto kernel = plan_in_one_launch<GM, DM, EXACT, K, WAVES>;
  if (lds > 64 * 1024)
    LPLB_HIP_TRY(allow_dynamic_lds(kernel, kPlanLdsLimit));
  PlanDevice *d = nullptr;
  int rc = plan_device(&d);
  if (rc != LPLB_OK)
    return rc;
  static KernelFootprint footprint;
  const int fit = workgroups_per_cu(reinterpret_cast<const void *>(kernel), footprint, WAVES, lds);
  const int n_workgroups = a.n_slices + a.n_lp_workgroups;
  if (fit <= 0 || n_workgroups > (int)(kResidencyBudget * fit * d->n_cus))
    return LPLB_OK;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capture) != hipSuccess)
    capture = hipStreamCaptureStatusNone;
  const bool capturing = capture == hipStreamCaptureStatusActive;
  const float cost = (float)n_workgroups / (float)(fit * d->n_cus);
  std::lock_guard<std::mutex> lock(g_plan_guard);   // held over the launch: admission and launch order agree
  const int slot = admit_launch(*d, s, cost, capturing);
  if (slot < 0)
    return LPLB_OK;
  PlanSlot &ps = d->slots[slot];
  a.sync = d->sync + (size_t)slot * kSlotInts;
  a.solve.tagged_result = reinterpret_cast<unsigned long long *>(a.sync + kSharesAt);
  a.solve.tagged_copies = a.n_share_copies;
  a.solve.tagged_stride = kMaxShares;
  a.expected_slices = a.n_slices + g_fault_extra_slices.exchange(0);
  const int fault_polls = g_fault_max_polls.exchange(0);
  a.max_polls = fault_polls > 0 ? fault_polls : kDefaultMaxPolls;
  // (a captured launch keeps its share of the GPU for good and reports nothing)
  if (!capturing) {
    ps.seq = (ps.seq + 1) & 0x3fffffff;
    a.arrived_word = d->arrived + slot;
    a.arrived_seq = ps.seq;
  }
  launch(kernel, dim3(n_workgroups), dim3(WAVES * kWave), lds, s, a);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess)
    return fail(LPLB_EHIP, "plan: launch failed: %s", hipGetErrorString(err));
  ps.maybe_executing = !capturing;
  g_one_launch_plans.fetch_add(1, std::memory_order_relaxed);
  *done = true;
  return LPLB_OK;
}

// Chunks per wave (1, 2, 4, 8 or 16) that cover a slice of `per` indices with `waves` waves.
static int chunks_per_wave(int64_t per, int waves) {
  const int64_t chunks = (per + kWave - 1) / kWave;
  const int64_t needed = (chunks + waves - 1) / waves;
  return needed <= 1 ? 1 : needed <= 2 ? 2 : needed <= 4 ? 4 : needed <= 8 ? 8 : 16;
}

template <int GM, int DM, bool EXACT, int W>
static int launch_plan_shape(PlanArgs &a, hipStream_t s, bool *done) {
  const int k = chunks_per_wave(a.per, W);
  const size_t lds_slices = plan_lds_bytes(a.sh.n_logical, a.n_rep, W, k);
  // LP workgroups: their waves' working areas, then the counts (one copy per LP if they fit,
  // else none and the LPs read global memory; own-histogram mode needs one copy in any case)
  const size_t lp_areas = kLpsPerWorkgroup * plan_lp_area_bytes(GM);
  const size_t one_copy = (size_t)a.solve.n_experts * sizeof(float);
  const size_t all_copies = (size_t)min(a.solve.n_units, kLpsPerWorkgroup) * one_copy;
  size_t lds = max(lds_slices, lp_areas + (a.local_counts ? one_copy : 0));
  if (lds > (size_t)kPlanLdsLimit)
    return LPLB_OK;
  if (lp_areas + all_copies <= max(lds, (size_t)16 * 1024)) {   // (a few KiB more are worth one global round trip less)
    lds = max(lds, lp_areas + all_copies);
    a.solve.staged_stride = a.solve.n_experts;
  } else {
    a.solve.staged_stride = 0;
  }
  switch (k) {
  case 1: return launch_plan_variant<GM, DM, EXACT, 1, W>(a, lds, s, done);
  case 2: return launch_plan_variant<GM, DM, EXACT, 2, W>(a, lds, s, done);
  case 4: return launch_plan_variant<GM, DM, EXACT, 4, W>(a, lds, s, done);
  case 8: return launch_plan_variant<GM, DM, EXACT, 8, W>(a, lds, s, done);
  default:
    if constexpr (W == 8)
      return launch_plan_variant<GM, DM, EXACT, 16, W>(a, lds, s, done);
    return LPLB_OK;
  }
}

// Tries the one-launch plan.  *done = false: shape or size outside what it covers, or no
// room on the GPU right now; nothing was enqueued.
static int try_one_launch(const int64_t *idx, int64_t n_elements, const int32_t *counts, const int32_t *r2o,
                          const int32_t *o2r, const int32_t *phy2log, int n_group, int G, int D, int C, int P,
                          int n_blocks, int32_t *counts_by_block, float *global_workload, float *o_weight,
                          int32_t *avail_num, int64_t *out, int32_t *physical_counts, int step_rule, int n_steps,
                          hipStream_t s, bool *done) {
  *done = false;
  const int L = P - D * C, n_fixed = L - D * C;
  const int n_logical = n_group * G * L, n_rep = n_group * G * C * D;
  if (!g_cooperative || n_elements <= 0 || n_blocks < 2)
    return LPLB_OK;
  int gm = 0, dm = 0;
  if (!plan_lp_shape(G, D, &gm, &dm) || n_group > kLpsPerWorkgroup * kMaxLpWorkgroups ||
      n_group * G * D > kMaxShares || global_workload == nullptr || n_logical > kMaxTotals ||
      n_group * G * P >= 65536 || n_elements > (INT32_MAX - 41) / 499)
    return LPLB_OK;
  const int n_lp_workgroups = (n_group + kLpsPerWorkgroup - 1) / kLpsPerWorkgroup;
  const int n_cus = current_device_cu_count();
  if (n_cus <= 0)
    return LPLB_OK;
  // Workgroup size: 16 waves where the LP's registers allow it, 8 where they do not, where
  // the LDS tables need it, and for batches so long that 16-wave workgroups (one per CU)
  // could not all be resident.
  int waves = plan_waves(gm, dm);
  // Slices of 1024 indices while kPreferredSlices of them cover the batch, else of 2048,
  // 4096, 8192 (the longest a workgroup holds in registers); at most n_blocks - 1 of them
  // (the caller's bound on parallelism; the last row of its table takes the totals).
  const int64_t longest = 8192;
  int64_t len = 1024;
  while (len < longest && (n_elements + len - 1) / len > kPreferredSlices)
    len *= 2;
  int64_t slices = (n_elements + len - 1) / len;
  if (slices > n_blocks - 1)
    slices = n_blocks - 1;
  const int64_t per = slice_len(n_elements, (int)slices);
  if (per > longest)
    return LPLB_OK;
  slices = (n_elements + per - 1) / per;   // (rounding the slice length up may have emptied the last ones)
  if (waves == 16 && (slices + n_lp_workgroups > n_cus / 2 ||
                      plan_lds_bytes(n_logical, n_rep, 16, chunks_per_wave(per, 16)) > (size_t)kPlanLdsLimit))
    waves = 8;
  int row_shift = 0;
  while ((1 << row_shift) < n_rep)
    ++row_shift;
  if ((slices << row_shift) > (int64_t)(n_blocks - 1) * n_logical)
    return LPLB_OK;   // the rows of the exchange live in the caller's table

  PlanArgs a{};   // every field the host does not set below is zero
  a.idx = idx; a.n = n_elements; a.per = per; a.n_slices = (int)slices; a.n_lp_workgroups = n_lp_workgroups;
  a.o2r = o2r; a.phy2log = phy2log; a.rows = counts_by_block; a.row_shift = row_shift;
  a.totals = counts_by_block + (int64_t)(n_blocks - 1) * n_logical; a.out = out;
  a.physical_counts = physical_counts; a.avail = avail_num;
  a.sh = RedirectShape{n_logical, n_group * G, G, D, C, L, P};
  a.n_rep = n_rep;
  a.magic_L = fast_div_magic((uint32_t)L); a.magic_cd = fast_div_magic((uint32_t)(C * D));
  a.magic_D = fast_div_magic((uint32_t)D); a.magic_G = fast_div_magic((uint32_t)G);
  a.local_counts = counts == nullptr;
  a.n_copies = 1;
  while (a.n_copies < kTotalCopies && a.n_copies * 16 < a.n_slices)
    a.n_copies *= 2;
  a.n_share_copies = 1;
  while (a.n_share_copies < kShareCopies && a.n_share_copies * 8 < a.n_slices)
    a.n_share_copies *= 2;
  a.n_arrival_copies = 1;
  while (a.n_arrival_copies < kArrivalCopies && a.n_arrival_copies * 32 < a.n_slices)
    a.n_arrival_copies *= 2;
  SolveArgs &sa = a.solve;
  sa.workload = counts; sa.gw_out = global_workload; sa.r2o = r2o; sa.phy2log = phy2log;
  sa.avail = avail_num; sa.result = o_weight; sa.n_group = n_group; sa.G = G; sa.D = D; sa.C = C;
  sa.n_fixed = n_fixed; sa.n_experts = n_logical; sa.step_rule = step_rule; sa.n_steps = n_steps;
  sa.n_units = n_group; sa.staged_stride = 0;
  sa.clocks = debug_clocks();

  int rc = LPLB_OK;
#define LPLB_PLAN_CASE_W(GM, DM, W)                                                            \
  if (gm == GM && dm == DM && waves == W)                                                      \
    rc = (G == GM && D == DM) ? launch_plan_shape<GM, DM, true, W>(a, s, done)                \
                              : launch_plan_shape<GM, DM, false, W>(a, s, done);
  LPLB_PLAN_CASE_W(8, 1, 16) LPLB_PLAN_CASE_W(8, 1, 8) LPLB_PLAN_CASE_W(8, 2, 16) LPLB_PLAN_CASE_W(8, 2, 8)
  LPLB_PLAN_CASE_W(8, 4, 8) LPLB_PLAN_CASE_W(16, 1, 8) LPLB_PLAN_CASE_W(16, 2, 8)
  LPLB_PLAN_CASE_W(32, 1, 8) LPLB_PLAN_CASE_W(32, 2, 8)
#undef LPLB_PLAN_CASE_W
  return rc;
}

} // namespace lplb

extern "C" int lplb_plan_set_cooperative(int enabled) {
  lplb::g_cooperative = enabled != 0;
  return LPLB_OK;
}

extern "C" int lplb_plan_forget_captured(lplb_stream_t stream) {
  using namespace lplb;
  PlanDevice *d = nullptr;
  const int rc = plan_device(&d);
  if (rc != LPLB_OK)
    return rc;
  std::lock_guard<std::mutex> lock(g_plan_guard);
  for (int i = 0; i < kSyncSlots; ++i) {
    PlanSlot &ps = d->slots[i];
    if (ps.used && ps.captured && ps.stream == static_cast<hipStream_t>(stream)) {
      // back to a slot whose stream has nothing pending: it may serve this stream again or pass to another
      ps.captured = ps.maybe_executing = false;
      ps.cost = 0.0f;
    }
  }
  return LPLB_OK;
}

extern "C" int lplb_plan_sync_timeouts(int *count) {
  using namespace lplb;
  LPLB_REQUIRE(count != nullptr, LPLB_EINVAL, "plan_sync_timeouts: null pointer");
  PlanDevice *d = nullptr;
  const int rc = plan_device(&d);
  if (rc != LPLB_OK)
    return rc;
  // Everything enqueued so far has ended after this, so a block that is switched off can be
  // cleared without a launch looking at it (the caller must not enqueue plans from other
  // threads meanwhile, as the header says).
  LPLB_HIP_TRY(hipDeviceSynchronize());
  *count = 0;
  for (int slot = 0; slot < kSyncSlots; ++slot) {
    int *block = d->sync + (size_t)slot * kSlotInts;
    int head[kTimeoutsAt + 1] = {};
    LPLB_HIP_TRY(hipMemcpy(head, block, sizeof(head), hipMemcpyDeviceToHost));
    *count += head[kTimeoutsAt];
    if (head[kPoisonAt] != 0) {
      // back to the state of a block that has never been used; the failures stay counted
      LPLB_HIP_TRY(hipMemset(block, 0, kTimeoutsAt * sizeof(int)));
      LPLB_HIP_TRY(hipMemset(block + kTimeoutsAt + 1, 0, (size_t)(kSlotInts - kTimeoutsAt - 1) * sizeof(int)));
    }
  }
  LPLB_HIP_TRY(hipDeviceSynchronize());
  {
    std::lock_guard<std::mutex> lock(g_plan_guard);   // nothing enqueued so far is still running
    for (int slot = 0; slot < kSyncSlots; ++slot)
      d->slots[slot].maybe_executing = false;
  }
  return LPLB_OK;
}

namespace lplb {
// dst[0] = waits that ran out on this device so far, dst[1] = blocks of counters switched off right now
__global__ void report_plan_health(const int *sync, int32_t *dst) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int timeouts = 0, off = 0;
    for (int slot = 0; slot < kSyncSlots; ++slot) {
      timeouts += agent_load(sync + (size_t)slot * kSlotInts + kTimeoutsAt);
      off += agent_load(sync + (size_t)slot * kSlotInts + kPoisonAt) != 0;
    }
    dst[0] = timeouts;
    dst[1] = off;
  }
}
} // namespace lplb

extern "C" int lplb_plan_poll_timeouts(int32_t *dst, lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(dst != nullptr, LPLB_EINVAL, "plan_poll_timeouts: null pointer");
  PlanDevice *d = nullptr;
  const int rc = plan_device(&d);
  if (rc != LPLB_OK)
    return rc;
  launch(report_plan_health, dim3(1), dim3(kWave), 0, static_cast<hipStream_t>(stream), d->sync, dst);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}

extern "C" int lplb_plan_one_launch_count(long long *count) {
  LPLB_REQUIRE(count != nullptr, LPLB_EINVAL, "plan_one_launch_count: null pointer");
  *count = lplb::g_one_launch_plans.load(std::memory_order_relaxed);
  return LPLB_OK;
}

extern "C" int lplb_plan_inject_fault(int extra_slices_expected, int max_polls) {
  LPLB_REQUIRE(extra_slices_expected >= 0 && max_polls >= 0, LPLB_EINVAL, "plan_inject_fault: negative argument");
  lplb::g_fault_extra_slices = extra_slices_expected;
  lplb::g_fault_max_polls = max_polls;
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

// Per device: the table's address (the array's name is only a host-side handle: looked up once, at the
// first call on the device) and who used the table last.  One table serves every stream, so a call from
// another stream is refused while the last user's kernels may still be running; `done` is recorded
// behind each call and is made, like the address, at that first call, which therefore has to happen
// outside a stream capture.  A call captured into a graph keeps the table for its stream for good.
struct ScratchUse {
  int32_t *table = nullptr;
  int *finished = nullptr;   // pinned host memory: the number of the last call whose kernels have all ended
  int seq = 0;               // number of the last call
  hipStream_t stream = nullptr;
  bool used = false, captured = false;
};
static ScratchUse g_scratch_use[64];
static std::mutex g_scratch_guard;

static int scratch_of_current_device(ScratchUse **use) {
  int dev = -1;
  LPLB_HIP_TRY(hipGetDevice(&dev));
  LPLB_REQUIRE(dev >= 0 && dev < 64, LPLB_EUNSUPPORTED, "plan_noalloc: device ordinal %d", dev);
  ScratchUse &u = g_scratch_use[dev];
  if (!u.table) {
    int32_t *p = nullptr;
    LPLB_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
    LPLB_REQUIRE(p != nullptr, LPLB_EHIP, "plan_noalloc: no device address for the slice table");
    LPLB_HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&u.finished), sizeof(int), hipHostMallocDefault));
    *u.finished = 0;
    u.table = p;
  }
  *use = &u;
  return LPLB_OK;
}

// The last kernel of a call: copies the batch's totals out (n may be 0) and says, in pinned host memory, that
// every kernel of call number `seq` has ended (kernels of one stream end in the order they were enqueued).
__global__ void copy_ints_and_report(const int32_t *__restrict__ src, int32_t *__restrict__ dst, int n, int *finished,
                                     int seq) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    dst[i] = src[i];
  if (i == 0 && finished)
    __hip_atomic_store(finished, seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
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
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capture) != hipSuccess)
    capture = hipStreamCaptureStatusNone;
  const bool capturing = capture == hipStreamCaptureStatusActive;
  std::lock_guard<std::mutex> lock(g_scratch_guard);   // held over the call: check, enqueue and record agree
  ScratchUse *use = nullptr;
  int rc = scratch_of_current_device(&use);
  if (rc != LPLB_OK)
    return rc;
  if (use->used && use->stream != s) {
    const bool busy = use->captured || __atomic_load_n(use->finished, __ATOMIC_ACQUIRE) != use->seq;
    LPLB_REQUIRE(!busy, LPLB_EBUSY,
                 "plan_noalloc: the built-in slice table is in use by a plan on another stream%s; wait for it, keep "
                 "such plans on one stream, or use lplb_plan with a workspace of your own",
                 use->captured ? " (captured into a graph, which keeps it)" : "");
  }
  int32_t *table = use->table;
  // Nothing in the table has to start at zero: every row is written (by the slice that
  // owns it) before anything reads it, and rows beyond n_blocks are never read.
  rc = plan_checked(idx, n_elements, global_counts, r2o, o2r, phy2log, n_group, group_size, dup_per_rank,
                    n_combined_experts, n_local_experts, n_blocks, table, global_workload, o_weight, avail_num, out,
                    physical_counts, step_rule, n_steps, stream);
  // Whatever was enqueued may touch the table, also when a later step of the chain failed: the call is
  // numbered and its last kernel reports the number (a captured call reports nothing: it keeps the table).
  use->used = true;
  use->stream = s;
  use->captured = use->captured || capturing;
  if (!capturing)
    use->seq = (use->seq + 1) & 0x3fffffff;
  const int n_copy = rc == LPLB_OK && local_counts != nullptr ? (int)n_logical : 0;
  launch(copy_ints_and_report, dim3((unsigned)((n_copy + 255) / 256 > 0 ? (n_copy + 255) / 256 : 1)), dim3(256), 0, s,
         table + (int64_t)(n_blocks - 1) * n_logical, local_counts, n_copy, capturing ? nullptr : use->finished, use->seq);
  if (hipGetLastError() != hipSuccess && rc == LPLB_OK)
    rc = fail(LPLB_EHIP, "plan_noalloc: launch failed");
  return rc;
}
