// Logical -> physical redirect of routing indices (streaming, HBM-bound:
// 8 bytes read + 8 bytes written per index).
//
// A token of an expert WITHOUT a replica goes to the expert's original slot: one
// table look-up.  A token of an expert WITH a replica needs its ordinal k among the
// tokens of the same expert, in index order, because the original/replica decision
// hashes k (minilp.cu:503-509).  The reference takes k from a shared-memory atomic
// (minilp.cu:504), which fixes the set of ordinals per block but not which token
// gets which.  Here k is canonical, and it is worked out only for the replicated
// sets (a few per rank), which keeps the ranking state small: one 16-byte slot per
// (wave, replicated set, chunk).
//
// A workgroup walks its slice in passes of n_waves * K consecutive 64-index chunks,
// K per wave; the loads of two passes are in flight.  Per pass:
//   A  every lane looks up its token's route; lanes with a replicated expert set
//      their bit in the 64-bit bitmap of (wave, set, chunk);
//   -- workgroup barrier --
//   B  lane (set, chunk) counts the bits of the same set and chunk in the waves
//      before it (popcounts) and of the chunks before it in its own wave, which gives
//      the ordinal of the chunk's first token of that set;
//   C  a token's ordinal is that start plus the number of lower lanes in the bitmap
//      (one 16-byte LDS read, two mbcnt); hash, compare, store.
// Nothing in C depends on another chunk, so the K chunks of a wave overlap.
// Bitmaps and running totals are double-buffered by pass parity, which leaves one
// workgroup barrier per pass.  Nothing depends on execution order.
#include "map_kernel.h"

namespace lplb {

struct MapArgs {
  const int64_t *idx;
  const float *o_weight;
  const int32_t *by_block;
  const int32_t *o2r;
  const int32_t *phy2log;
  int64_t n;
  int64_t per;
  int n_logical, n_ranks, n_rep, G, D, C, L, P, n_blocks;
  uint32_t magic_L, magic_cd, magic_D, magic_G;   // fast_div_magic of L, C * D, D, G
  int64_t *out;
  int32_t *physical_counts;   // [n_ranks * P] tokens per physical expert, or null
  const int32_t *prepared;    // table of lplb_prepare_mapping for this phy2log / o2r / shape, or null
  long long *clocks;   // debug builds: stamps of the first and the last workgroup (else null)
};
#define LPLB_MAP_STAMP(k)                                                                      \
  LPLB_STAMP_AT(blockIdx.x == 0 ? a.clocks + 32 : (blockIdx.x == gridDim.x - 1 ? a.clocks + 48 : nullptr), k)

__global__ void zero_ints(int32_t *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    p[i] = 0;
}

// ---- the tables every workgroup builds before its first token (minilp.cu:466-496) ----
// original slot of logical position e: rank e / L, place e % L
__device__ inline int slot_of(const MapArgs &a, int e) {
  return e + (int)fast_div((uint32_t)e, a.magic_L) * (a.P - a.L);
}
// replicated set i = (ep_rank, place): its slot index d and the group rank of ep_rank
struct SetOf {
  int ep_rank, place, d, group_rank;
};
__device__ inline SetOf set_of(const MapArgs &a, int i) {
  const int cd = a.C * a.D;
  SetOf s;
  s.ep_rank = (int)fast_div((uint32_t)i, a.magic_cd);
  s.place = i - s.ep_rank * cd;
  s.d = s.place - (int)fast_div((uint32_t)s.place, a.magic_D) * a.D;
  s.group_rank = s.ep_rank - (int)fast_div((uint32_t)s.ep_rank, a.magic_G) * a.G;
  return s;
}
// What a thread reads of the small tables before it issues its index loads.  All of them are
// unconditional loads from clamped addresses: a load inside a branch makes the compiler wait
// for it right there, before the index loads are issued.
struct TableLoads {
  int slot0, le0;                   // first (usually only) expert of this thread: its slot, who sits there
  int32_t total0, before0_raw;      // that expert's tokens in the whole array / before this slice
  bool set0;                        // first (usually only) replicated set of this thread
  SetOf s0;
  int rle0, host0;
  float share0;
};
__device__ inline TableLoads issue_table_loads(const MapArgs &a, int tid, const int32_t *last, const int32_t *prev) {
  const int nl = a.n_logical;
  TableLoads t;
  const int e0 = min(tid, nl - 1);
  t.slot0 = slot_of(a, e0);
  t.le0 = a.phy2log[t.slot0];
  // The counts are read per expert, not per replicated set, so that they do not have to
  // wait for phy2log (a load issued after the index loads returns after them).
  t.total0 = last[e0];
  t.before0_raw = (prev ? prev : last)[e0];
  t.set0 = tid < a.n_rep;
  t.s0 = set_of(a, t.set0 ? tid : 0);
  // (with no replicated set at all, R == 0, these read element 0 of each table)
  t.rle0 = a.phy2log[t.s0.ep_rank * a.P + t.s0.place];
  t.share0 = a.o_weight[t.s0.ep_rank * a.D + t.s0.d];
  t.host0 = a.o2r[t.s0.group_rank * a.D + t.s0.d];
  return t;
}
// First half, up to the workgroup barrier the caller places after it: empty routes, the
// stand-in set, the two rows of counts.
__device__ inline void tables_before_barrier(const MapArgs &a, const TableLoads &t, Route *route, RepEntry *reps,
                                             int32_t *staged, const int32_t *last, const int32_t *prev, int tid, int nt) {
  const int nl = a.n_logical, R = a.n_rep;
  for (int e = tid; e <= nl; e += nt)
    route[e] = Route{-1, R};
  if (tid == 0)
    reps[R] = RepEntry{1, 0xffffffffu, INT32_MAX, -1};   // "no replica": every token stays
  if (tid < nl) {
    staged[tid] = t.total0;
    staged[nl + tid] = prev ? t.before0_raw : 0;
  }
  for (int e = tid + nt; e < nl; e += nt) {
    staged[e] = last[e];
    staged[nl + e] = prev ? prev[e] : 0;
  }
}
// Second half: where every expert's original sits, and the constants of the replicated sets.
// A workgroup barrier has to follow before anything reads the tables.
__device__ inline void tables_after_barrier(const MapArgs &a, const TableLoads &t, Route *route, RepEntry *reps,
                                            int32_t *carry, const int32_t *staged, int tid, int nt) {
  const int nl = a.n_logical, R = a.n_rep, cd = a.C * a.D;
  if (tid < nl && t.le0 >= 0 && t.le0 < nl)
    route[t.le0].original = t.slot0;
  for (int e = tid + nt; e < nl; e += nt) {
    const int s = slot_of(a, e), le = a.phy2log[s];
    if (le >= 0 && le < nl)
      route[le].original = s;
  }
  // A set's key is R - 1 - i, so that of two sets that name the same expert the later one
  // wins (as a sequential pass over the sets would have it) with an atomic min.
  auto fill_set = [&](int i, const SetOf &s, int le, float share, int host) {
    const bool ok = le >= 0 && le < nl;
    const int32_t tokens = ok ? staged[le] : 0;
    const int32_t before = ok ? staged[nl + le] : 0;
    if (ok)
      atomicMin(&route[le].rep, R - 1 - i);
    RepEntry x;
    x.total = tokens;
    x.magic = tokens >= 1 ? 0xffffffffu / (uint32_t)tokens : 0u;
    x.expected = expected_on_original(share, tokens);
    x.replica = ((s.ep_rank - s.group_rank) + host + 1) * a.P - cd + s.place;
    reps[R - 1 - i] = x;
    carry[R - 1 - i] = before;
  };
  if (t.set0)
    fill_set(tid, t.s0, t.rle0, t.share0, t.host0);
  for (int i = tid + nt; i < R; i += nt) {
    const SetOf s = set_of(a, i);
    fill_set(i, s, a.phy2log[s.ep_rank * a.P + s.place], a.o_weight[s.ep_rank * a.D + s.d],
             a.o2r[s.group_rank * a.D + s.d]);
  }
}
// Tokens per physical expert (= bincount of the output) from the tables alone.
__device__ inline void physical_counts_from_tables(const MapArgs &a, const Route *route, const RepEntry *reps,
                                                   const int32_t *staged, int tid, int nt) {
  const int nl = a.n_logical, R = a.n_rep;
  for (int i = tid; i < a.n_ranks * a.P; i += nt) {
    const int le = a.phy2log[i];
    int32_t v = 0;
    if (le >= 0 && le < nl) {
      const Route rt = route[le];
      if (rt.rep >= R) {
        v = rt.original == i ? staged[le] : 0;
      } else {
        const RepEntry x = reps[rt.rep];
        const int32_t kept = kept_on_original(x.total, x.expected);
        v = rt.original == i ? kept : (x.replica == i ? x.total - kept : 0);
      }
    }
    a.physical_counts[i] = v;
  }
}

// LDS bytes for n_logical experts, n_rep replicated sets, w waves and K chunks per wave and pass.
static size_t map_lds_bytes(int n_logical, int n_rep, int w, int k) {
  return (size_t)(n_rep + 1) * sizeof(RepEntry) + (size_t)w * (n_rep + 1) * rank_record_bytes(k) +
         (size_t)(n_logical + 1) * sizeof(Route) + (size_t)2 * n_rep * sizeof(int32_t) +
         (size_t)2 * n_logical * sizeof(int32_t);
}

// TAIL: some wave's K chunks may reach past the end of its slice (loads and stores are
// then predicated per lane); without it every pass of every slice is whole, and the
// code from the first load to the first barrier has no branch, which lets the compiler
// count outstanding loads exactly: the tables are built from the small loads while the
// index loads issued after them are still in flight.
// SINGLE: a slice is at most one pass long (no second set of loads in flight, and the
// registers that saves let twice as many waves stay resident).
template <int K, bool WRAP, bool TAIL, bool SINGLE>
__global__ __launch_bounds__(kMaxWaves *kWave, SINGLE ? 8 : 4) void redirect_indices(MapArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  fetch_arguments_now(a.idx, a.o_weight, a.by_block, a.o2r, a.phy2log, a.n, a.per, a.n_logical, a.n_ranks, a.n_rep, a.G,
                      a.D, a.C, a.L, a.P, a.n_blocks, a.magic_L, a.magic_cd, a.magic_D, a.magic_G, a.out,
                      a.physical_counts);
  constexpr int kRec = rank_record_bytes(K);
  const int nl = a.n_logical, R = a.n_rep;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid % kWave, n_waves = nt / kWave;
  const int wave_s = __builtin_amdgcn_readfirstlane(tid / kWave);   // wave-uniform
  const int pid = blockIdx.x;
  const int64_t begin = slice_begin(a.n, a.per, pid);
  const int64_t end = slice_begin(a.n, a.per, pid + 1);
  const bool counts_wanted = pid == 0 && a.physical_counts != nullptr;
  if (begin >= end && !counts_wanted)
    return;

  RepEntry *reps = reinterpret_cast<RepEntry *>(smem_raw);                          // [R + 1]
  unsigned char *records = smem_raw + (size_t)(R + 1) * sizeof(RepEntry);          // [n_waves][R + 1][kRec]
  const int wave_stride = (R + 1) * kRec;
  Route *route = reinterpret_cast<Route *>(records + (size_t)n_waves * wave_stride);   // [nl + 1]
  int32_t *carry = reinterpret_cast<int32_t *>(route + nl + 1);                     // [2][R]
  int32_t *staged = carry + 2 * R;   // [2][nl] tokens per expert: in the whole array, before this slice
  unsigned char *my_records = records + (size_t)wave_s * wave_stride;
  const unsigned long long my_bit = 1ull << lane;
  const int32_t *last = a.by_block + (int64_t)(a.n_blocks - 1) * nl;
  const int32_t *prev = pid ? a.by_block + (int64_t)(pid - 1) * nl : nullptr;
  LPLB_MAP_STAMP(0);

  // ---- small global reads of the table build first (mostly L2 hits) ----
  const TableLoads tl = issue_table_loads(a, tid, last, prev);

  // ---- the index loads of the first two passes right behind them ----
  const int64_t pass_len = (int64_t)n_waves * K * kWave;
  const int64_t wave_off = (int64_t)wave_s * (K * kWave);
  auto issue_loads = [&](int64_t (&raw)[K], int64_t pass) {
    const int64_t w0 = pass + wave_off;                    // first index of this wave's K chunks (uniform)
    const int64_t *src = a.idx + w0 + lane;
    if (!TAIL || w0 + K * kWave <= end) {
#pragma unroll
      for (int c = 0; c < K; ++c)
        raw[c] = __builtin_nontemporal_load(src + c * kWave);
    } else {
#pragma unroll
      for (int c = 0; c < K; ++c)
        raw[c] = w0 + c * kWave + lane < end ? __builtin_nontemporal_load(src + c * kWave) : -1;
    }
  };
  int64_t raw0[K], raw1[SINGLE ? 1 : K];
  issue_loads(raw0, begin);
  // (without TAIL a slice of one pass loads that pass twice rather than branch here)
  if constexpr (!SINGLE)
    issue_loads(raw1, (TAIL || begin + pass_len < end) ? begin + pass_len : begin);

  // ---- tables ----
  {
    const i32x4 zero{0, 0, 0, 0};
    i32x4 *z = reinterpret_cast<i32x4 *>(records);
    for (int i = tid; i < n_waves * wave_stride / 16; i += nt)
      z[i] = zero;
  }
  tables_before_barrier(a, tl, route, reps, staged, last, prev, tid, nt);
  __syncthreads();
  tables_after_barrier(a, tl, route, reps, carry, staged, tid, nt);
  __syncthreads();
  LPLB_MAP_STAMP(1);
  if (counts_wanted)
    physical_counts_from_tables(a, route, reps, staged, tid, nt);

  // ---- one pass ----
  auto process = [&](auto parity_c, int64_t (&raw)[K], int64_t pass) {
    constexpr int PAR = decltype(parity_c)::value;
    int32_t original[K];
    int32_t set[K];
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const bool valid = (uint64_t)raw[c] < (uint64_t)nl;   // -1, other negatives and too large ids fail
      const Route rt = route[valid ? (int)raw[c] : nl];
      original[c] = rt.original;
      set[c] = rt.rep;
    }
    if constexpr (!SINGLE)
      if (pass + 2 * pass_len < end)
        issue_loads(raw, pass + 2 * pass_len);   // in flight during this pass and the next
    // Phase A.
    ChunkSlot *slot[K];
#pragma unroll
    for (int c = 0; c < K; ++c) {
      slot[c] = reinterpret_cast<ChunkSlot *>(my_records + __umul24((uint32_t)set[c], (uint32_t)kRec)) + (PAR * K + c);
      if (set[c] < R)
        atomicOr(reinterpret_cast<unsigned long long *>(slot[c]), my_bit);
    }
    LPLB_MAP_STAMP(2 + 4 * PAR);
    __syncthreads();
    LPLB_MAP_STAMP(3 + 4 * PAR);
    // Phase B: lane = (set, chunk), chunk fastest.  The rows of the waves before this
    // one are read four at a time (clamped addresses, masked values).
    if (R > 0) {
      const int c = lane % K;
      for (int p0 = 0; p0 < R * K; p0 += kWave) {
        const bool live = p0 + lane < R * K;
        const int q = live ? (p0 + lane) / K : R;   // lanes past the end read the stand-in record (zeros)
        unsigned char *first = records + __umul24((uint32_t)q, (uint32_t)kRec) + (PAR * K + c) * (int)sizeof(ChunkSlot);
        const int32_t carried = carry[PAR * R + (live ? q : 0)];
        const unsigned long long own_bits =
            *reinterpret_cast<const unsigned long long *>(first + wave_s * wave_stride);
        int earlier = 0;
        for (int w0 = 0; w0 < wave_s; w0 += 4) {
          unsigned long long bits[4];
#pragma unroll
          for (int u = 0; u < 4; ++u)
            bits[u] = *reinterpret_cast<const unsigned long long *>(first + min(w0 + u, wave_s) * wave_stride);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            earlier += w0 + u < wave_s ? __popcll(bits[u]) : 0;
        }
        const int own = __popcll(own_bits);
        const int in_earlier_waves = group_sum<K>(earlier);
        const int in_my_wave = group_sum<K>(own);
        const int in_earlier_chunks = group_exclusive_scan<K>(own, c);
        if (live) {
          const int32_t base = carried + in_earlier_waves;
          ChunkSlot *mine = reinterpret_cast<ChunkSlot *>(first + wave_s * wave_stride);
          mine->start = base + in_earlier_chunks;
          // the other parity's bitmap is free again: clear it for the pass after this one
          *reinterpret_cast<unsigned long long *>(mine + (PAR ? -K : K)) = 0ull;
          if (wave_s == n_waves - 1 && c == 0)
            carry[(PAR ^ 1) * R + q] = base + in_my_wave;
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
    LPLB_MAP_STAMP(4 + 4 * PAR);
    // Phase C: all LDS reads of the K chunks first, then the arithmetic, then the stores.
    const int64_t w0 = pass + wave_off;
    int64_t *dst = a.out + w0 + lane;
    i32x4 s[K], x[K];
#pragma unroll
    for (int c = 0; c < K; ++c) {
      s[c] = *reinterpret_cast<const i32x4 *>(slot[c]);         // bits_lo, bits_hi, start
      x[c] = *reinterpret_cast<const i32x4 *>(&reps[set[c]]);   // total, magic, expected, replica
    }
    int32_t o[K];
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const int32_t k = __builtin_amdgcn_mbcnt_hi((uint32_t)s[c].y,
                                                  __builtin_amdgcn_mbcnt_lo((uint32_t)s[c].x, (uint32_t)s[c].z));
      const int32_t h = ordinal_hash<WRAP>(k, x[c].x, (uint32_t)x[c].y);
      o[c] = h >= x[c].z ? x[c].w : original[c];
    }
    if (!TAIL || w0 + K * kWave <= end) {
#pragma unroll
      for (int c = 0; c < K; ++c)
        __builtin_nontemporal_store((int64_t)o[c], dst + c * kWave);
    } else {
#pragma unroll
      for (int c = 0; c < K; ++c)
        if (w0 + c * kWave + lane < end)
          __builtin_nontemporal_store((int64_t)o[c], dst + c * kWave);
    }
    LPLB_MAP_STAMP(5 + 4 * PAR);
  };

  if constexpr (SINGLE) {
    if (begin < end)
      process(std::integral_constant<int, 0>{}, raw0, begin);
  } else {
    for (int64_t pass = begin; pass < end; pass += 2 * pass_len) {
      process(std::integral_constant<int, 0>{}, raw0, pass);
      if (pass + pass_len >= end)
        break;
      process(std::integral_constant<int, 1>{}, raw1, pass + pass_len);
    }
  }

#ifdef LPLB_PHASE_CLOCKS
  __builtin_amdgcn_s_waitcnt(0);
#endif
  LPLB_MAP_STAMP(10);
}

// ---- slices of up to 8192 indices: two indices per lane and load, one pass ----
// At the sweep shape ([262144 x 8]: 16 MiB in, 16 MiB out) three things decide the redirect's
// time besides the memory system itself:
//   * how its accesses are shaped: a plain copy with 16 bytes per lane and instruction and a
//     workgroup's loads all landed before its stores start takes 6.1 us, with 8 bytes per lane
//     6.7 us;
//   * vector-ALU issue: a CU's 8192 tokens are 32 wave-instructions per SIMD for every
//     instruction spent on a token, 53 ns each, all of it between the arrival of the indices and
//     the first store (clock stamps: 2 us with the 60 instructions per token of the kernel above);
//   * LDS: lanes that update one word are served one after the other, and the hottest expert
//     has ten tokens per 64 at Zipf(1.0).
// So here a wave takes KP runs of 128 consecutive indices, lane l holding indices 2 l and 2 l + 1
// of each (one 16-byte load), a workgroup covers its whole slice in one pass, and a token costs
// about 19 vector instructions, two LDS reads and one LDS update.
//
// Everything a token needs to know about its expert is one 16-byte LDS entry (ExpertPlan), read
// once.  The entries come ready-made from a table the caller prepares once per mapping
// (lplb_prepare_mapping: they depend on phy2log, o2r and the shape only); per batch a workgroup
// copies them and patches the replicated experts' tokens, reciprocal and share.  Callers without
// such a table get the kernel above, which builds its tables from phy2log in every workgroup.
// Kernel arguments are fetched in one batch and the small table reads are issued only by the
// waves that have an element to fetch (each measured: a plain copy in this kernel's shape
// loses 1 us when all sixteen waves issue five small loads ahead of their index loads).
//
// Ranking state: per (wave, replicated set, run, quarter of the wave) one 32-bit word of
// bitmaps -- bit j: the first index of lane 16 quarter + j belongs to the set, bit 16 + j: its
// second one -- and next to it the ordinal of the quarter's first token of the set (8 bytes, one
// LDS read per token).  In index order a quarter's tokens go x0 y0 x1 y1 ..., so a token's
// ordinal is that start + popcount(word & lower lanes, both halves), the lane's own first index
// included for its second one.
typedef long long i64x2 __attribute__((ext_vector_type(2)));
constexpr int kPairRun = 2 * kWave;   // indices one 16-byte load per lane covers
constexpr int kMaxPairRuns = 4;       // runs per wave: a slice is at most 16 waves x 4 runs x 128 indices
constexpr int kQuarters = 4, kQuarterLanes = kWave / kQuarters;
constexpr int kPairMaxSets = 511;              // the set's index has 9 bits in an expert's entry
constexpr int kPairMaxTotal = (1 << 23) - 1;   // ... and an expert's tokens 23
constexpr int kPairMaxSlots = 32767;           // slots are kept as signed 16-bit numbers (-1 = none)

struct __attribute__((aligned(16))) ExpertPlan {
  uint32_t total_set;   // tokens of the expert in the whole array | index of its replicated set << 23 (n_rep: none)
  uint32_t magic;       // floor((2^32 - 1) / tokens)
  int32_t stay;         // a token whose hash is below this stays on the original
  uint32_t slots;       // original slot | replica slot << 16, each as int16 (-1: none)
};
__device__ inline ExpertPlan plan_of_nobody(int n_rep) {   // no replica, every token stays; masked tokens: slot -1
  return ExpertPlan{1u | (uint32_t)n_rep << 23, 0xffffffffu, INT32_MAX, 0xffffffffu};
}
// Words of the prepared table: the entries, per replicated set (in key order) its expert (-1:
// none, or another set has the expert) and the index of its share, then copies of phy2log and o2r.
__host__ __device__ inline int64_t prepared_sets_at(int n_logical) { return 4 * ((int64_t)n_logical + 1); }
__host__ __device__ inline int64_t prepared_phy2log_at(int n_logical, int n_rep) { return prepared_sets_at(n_logical) + 2 * (int64_t)n_rep; }
__host__ __device__ inline int64_t prepared_o2r_at(int n_logical, int n_rep, int n_physical) {
  return prepared_phy2log_at(n_logical, n_rep) + n_physical;
}
// bytes of the ranking words of one (wave, replicated set): KP runs x 4 quarters x {bitmaps, start},
// padded to an odd multiple of 16 bytes so that consecutive sets start in different LDS banks
constexpr int pair_record_bytes(int kp) { return kp * kQuarters * 8 + 16; }
static size_t pairs_lds_bytes(int n_logical, int n_rep, int w, int kp) {
  return (size_t)(n_logical + 1) * sizeof(ExpertPlan) + (size_t)w * (n_rep + 1) * pair_record_bytes(kp) +
         (size_t)(w + 2) * n_rep * sizeof(int32_t) + (size_t)2 * n_logical * sizeof(int32_t) + 64;
}

// Builds the entries from phy2log and o2r (the prepared table's kernel, one workgroup).  plan: LDS,
// n_logical + 1 entries; set_expert: LDS, n_rep ints, receives each set's expert (-1: none / lost
// to a later set).  Ends with a workgroup barrier.
__device__ inline void build_expert_plans(const MapArgs &a, ExpertPlan *plan, int32_t *set_expert, int tid, int nt) {
  const int nl = a.n_logical, R = a.n_rep;
  const ExpertPlan nobody = plan_of_nobody(R);
  for (int e = tid; e <= nl; e += nt)
    plan[e] = nobody;
  __syncthreads();
  // where every expert's original sits (minilp.cu:471-473)
  for (int e = tid; e < nl; e += nt) {
    const int slot = slot_of(a, e), le = a.phy2log[slot];
    if (le >= 0 && le < nl)
      reinterpret_cast<uint16_t *>(&plan[le].slots)[0] = (uint16_t)slot;
  }
  // the replicated sets (minilp.cu:478-495): key R - 1 - i, so that the later of two sets that name
  // one expert wins the min, as a sequential pass over the sets would have it
  for (int i = tid; i < R; i += nt) {
    const SetOf s = set_of(a, i);
    const int le = a.phy2log[s.ep_rank * a.P + s.place];
    if (le >= 0 && le < nl)
      atomicMin(&plan[le].total_set, 1u | (uint32_t)(R - 1 - i) << 23);
  }
  __syncthreads();
  for (int i = tid; i < R; i += nt) {
    const SetOf s = set_of(a, i);
    const int le = a.phy2log[s.ep_rank * a.P + s.place];
    const bool mine = le >= 0 && le < nl && (int)(plan[le].total_set >> 23) == R - 1 - i;
    if (mine) {
      const int host = a.o2r[s.group_rank * a.D + s.d];
      reinterpret_cast<uint16_t *>(&plan[le].slots)[1] =
          (uint16_t)(((s.ep_rank - s.group_rank) + host + 1) * a.P - a.C * a.D + s.place);
    }
    set_expert[R - 1 - i] = mine ? le : -1;
  }
  __syncthreads();
}

__global__ __launch_bounds__(1024) void prepare_mapping(MapArgs a, int32_t *prepared) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int nl = a.n_logical, R = a.n_rep, n_physical = a.n_ranks * a.P;
  const int tid = threadIdx.x, nt = blockDim.x;
  ExpertPlan *plan = reinterpret_cast<ExpertPlan *>(smem_raw);
  int32_t *set_expert = reinterpret_cast<int32_t *>(plan + nl + 1);
  build_expert_plans(a, plan, set_expert, tid, nt);
  for (int i = tid; i < 4 * (nl + 1); i += nt)
    prepared[i] = reinterpret_cast<const int32_t *>(plan)[i];
  int32_t *sets = prepared + prepared_sets_at(nl);
  for (int i = tid; i < R; i += nt) {   // i: position in the reference's order; the set's key is R - 1 - i
    const SetOf s = set_of(a, i);
    sets[2 * (R - 1 - i)] = set_expert[R - 1 - i];
    sets[2 * (R - 1 - i) + 1] = s.ep_rank * a.D + s.d;
  }
  for (int i = tid; i < n_physical; i += nt)
    prepared[prepared_phy2log_at(nl, R) + i] = a.phy2log[i];
  for (int i = tid; i < a.G * a.D; i += nt)
    prepared[prepared_o2r_at(nl, R, n_physical) + i] = a.o2r[i];
}

// TAIL: the slice (or the array) may end inside or before a wave's runs; loads and stores of
// such a wave are predicated per index.  a.prepared holds the prepared table.
template <int KP, bool TAIL>
__global__ __launch_bounds__(kMaxWaves *kWave, KP >= 4 ? 4 : 8) void redirect_pairs(MapArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  fetch_arguments_now(a.idx, a.o_weight, a.by_block, a.o2r, a.phy2log, a.n, a.per, a.n_logical, a.n_ranks, a.n_rep, a.G,
                      a.D, a.C, a.L, a.P, a.n_blocks, a.magic_L, a.magic_cd, a.magic_D, a.magic_G, a.out,
                      a.physical_counts, a.prepared);
  constexpr int kRec = pair_record_bytes(KP);
  const int nl = a.n_logical, R = a.n_rep;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid % kWave, n_waves = nt / kWave;
  const int wave_s = __builtin_amdgcn_readfirstlane(tid / kWave);   // wave-uniform
  const int pid = blockIdx.x;
  const int64_t begin = slice_begin(a.n, a.per, pid);
  const int64_t end = slice_begin(a.n, a.per, pid + 1);
  const bool counts_wanted = pid == 0 && a.physical_counts != nullptr;
  if (begin >= end && !counts_wanted)
    return;

  ExpertPlan *plan = reinterpret_cast<ExpertPlan *>(smem_raw);                      // [nl + 1]
  unsigned char *records = reinterpret_cast<unsigned char *>(plan + nl + 1);       // [n_waves][R + 1][kRec]
  const int wave_stride = (R + 1) * kRec;
  int32_t *wave_total = reinterpret_cast<int32_t *>(records + (size_t)n_waves * wave_stride);   // [n_waves][R]
  int32_t *carry = wave_total + n_waves * R;   // [R] tokens of each set before this slice
  float *shares = reinterpret_cast<float *>(carry + R);   // [R] every share of the batch (one per rank and replica slot)
  int32_t *staged = reinterpret_cast<int32_t *>(shares + R);   // [2][nl] tokens per expert: in the whole array, before this slice
  unsigned char *my_records = records + (size_t)wave_s * wave_stride;
  const int32_t *last = a.by_block + (int64_t)(a.n_blocks - 1) * nl;
  const int32_t *prev = pid ? a.by_block + (int64_t)(pid - 1) * nl : nullptr;
  LPLB_MAP_STAMP(0);

  // ---- small global reads first (from clamped addresses: no lane-dependent branch), the index loads
  // right behind them ----
  const int e0 = min(tid, nl - 1), q0 = min(tid, max(R, 1) - 1);
  int32_t total0 = 0, before0 = 0;
  i32x4 entry0{0, 0, 0, 0};
  int2 set0{-1, 0};
  float share0 = 0.0f;
  // (only the waves whose threads have a table element to fetch: a wave-uniform branch)
  if (wave_s * kWave <= max(nl, max(R, a.n_ranks * a.D))) {
    total0 = last[e0];
    before0 = (prev ? prev : last)[e0];
    entry0 = reinterpret_cast<const i32x4 *>(a.prepared)[min(tid, nl)];
    set0 = reinterpret_cast<const int2 *>(a.prepared + prepared_sets_at(nl))[R > 0 ? q0 : 0];   // (R == 0: a word of phy2log, unused)
    share0 = a.o_weight[min(tid, a.n_ranks * a.D - 1)];
  }
  const int64_t w0 = begin + (int64_t)wave_s * (KP * kPairRun);   // first index of this wave's runs (uniform)
  const bool whole = !TAIL || w0 + KP * kPairRun <= end;
  i64x2 raw[KP];
  if (whole) {
    const i64x2 *src = reinterpret_cast<const i64x2 *>(a.idx + w0) + lane;
#pragma unroll
    for (int c = 0; c < KP; ++c)
      raw[c] = __builtin_nontemporal_load(src + c * kWave);
  } else {
#pragma unroll
    for (int c = 0; c < KP; ++c) {
      const int64_t i = w0 + c * kPairRun + 2 * lane;
      raw[c].x = i < end ? __builtin_nontemporal_load(a.idx + i) : -1;
      raw[c].y = i + 1 < end ? __builtin_nontemporal_load(a.idx + i + 1) : -1;
    }
  }

  // ---- tables (minilp.cu:466-496) ----
  {
    const i32x4 zero{0, 0, 0, 0};
    i32x4 *z = reinterpret_cast<i32x4 *>(records);
    for (int i = tid; i < n_waves * wave_stride / 16; i += nt)
      z[i] = zero;
  }
  if (tid < nl) {
    staged[tid] = total0;
    staged[nl + tid] = prev ? before0 : 0;
  }
  for (int e = tid + nt; e < nl; e += nt) {
    staged[e] = last[e];
    staged[nl + e] = prev ? prev[e] : 0;
  }
  if (tid <= nl)
    reinterpret_cast<i32x4 *>(plan)[tid] = entry0;
  for (int e = tid + nt; e <= nl; e += nt)
    reinterpret_cast<i32x4 *>(plan)[e] = reinterpret_cast<const i32x4 *>(a.prepared)[e];
  for (int i = tid; i < a.n_ranks * a.D; i += nt)
    shares[i] = i == tid ? share0 : a.o_weight[i];
  __syncthreads();
  // the replicated experts' tokens, reciprocal and share; the sets' tokens before this slice
  for (int q = tid; q < R; q += nt) {
    const int2 set = q == tid ? set0 : reinterpret_cast<const int2 *>(a.prepared + prepared_sets_at(nl))[q];
    const int le = set.x;
    const float share = shares[set.y];
    int32_t before = 0;
    if (le >= 0) {
      const int32_t tokens = staged[le];
      before = staged[nl + le];
      ExpertPlan x = plan[le];
      x.total_set = ((uint32_t)tokens & (uint32_t)kPairMaxTotal) | (uint32_t)q << 23;
      x.magic = tokens >= 1 ? 0xffffffffu / (uint32_t)tokens : 0u;
      x.stay = expected_on_original(share, tokens);
      plan[le] = x;
    }
    carry[q] = before;
  }
  __syncthreads();
  LPLB_MAP_STAMP(1);
  // Tokens per physical expert (= bincount of the output) from the tables alone.
  if (counts_wanted) {
    const int32_t *p2l = a.prepared + prepared_phy2log_at(nl, R);
    for (int i = tid; i < a.n_ranks * a.P; i += nt) {
      const int le = p2l[i];
      int32_t v = 0;
      if (le >= 0 && le < nl) {
        const ExpertPlan x = plan[le];
        const bool has_set = (int)(x.total_set >> 23) < R;
        const int32_t tokens = staged[le];
        const int32_t kept = has_set ? kept_on_original(tokens, x.stay) : tokens;
        const int original = (int)(int16_t)(x.slots & 0xffffu), replica = (int)(int16_t)(x.slots >> 16);
        v = original == i ? kept : (has_set && replica == i ? tokens - kept : 0);
      }
      a.physical_counts[i] = v;
    }
  }

  // ---- A: my tokens' entries; tokens of replicated sets enter their quarter's bitmaps ----
  const int quarter = lane / kQuarterLanes, lane16 = lane % kQuarterLanes;
  const uint32_t bit_x = 1u << lane16, bit_y = 1u << (16 + lane16);
  const uint32_t below_x = (bit_x - 1u) * 0x10001u;   // lower lanes of my quarter, both indices
  const uint32_t below_y = below_x | bit_x;           // ... and my own first index
  const uint32_t my_words = (uint32_t)(wave_s * wave_stride + quarter * 8) +
                            (uint32_t)(reinterpret_cast<uintptr_t>(records) - reinterpret_cast<uintptr_t>(smem_raw));
  i32x4 ex[KP], ey[KP];       // total | set, magic, stay, slots
  uint32_t wx[KP], wy[KP];    // LDS offset of the token's ranking word
#pragma unroll
  for (int c = 0; c < KP; ++c) {
    const bool valid_x = (uint64_t)raw[c].x < (uint64_t)nl;   // -1, other negatives and too large ids fail
    const bool valid_y = (uint64_t)raw[c].y < (uint64_t)nl;
    ex[c] = *reinterpret_cast<const i32x4 *>(&plan[valid_x ? (int)raw[c].x : nl]);
    ey[c] = *reinterpret_cast<const i32x4 *>(&plan[valid_y ? (int)raw[c].y : nl]);
  }
  LPLB_MAP_STAMP(6);
#pragma unroll
  for (int c = 0; c < KP; ++c) {
    const uint32_t set_x = (uint32_t)ex[c].x >> 23, set_y = (uint32_t)ey[c].x >> 23;
    wx[c] = __umul24(set_x, (uint32_t)kRec) + (my_words + c * kQuarters * 8);
    wy[c] = __umul24(set_y, (uint32_t)kRec) + (my_words + c * kQuarters * 8);
    if (set_x < (uint32_t)R)
      atomicOr(reinterpret_cast<uint32_t *>(smem_raw + wx[c]), bit_x);
    if (set_y < (uint32_t)R)
      atomicOr(reinterpret_cast<uint32_t *>(smem_raw + wy[c]), bit_y);
  }
  LPLB_MAP_STAMP(7);
  // ---- B, inside the wave: lane = (set, run), run fastest, reads the four quarters' words of its
  // run: tokens of the set in the wave's earlier runs and quarters, and in the whole wave.  The
  // first 64 (set, run) pairs stay in registers across the barrier. ----
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int n_pairs = R * KP;
  struct RunWords {
    i32x4 lo, hi;         // {word, start} of quarters 0, 1 and 2, 3
    int32_t before[4];    // tokens of the set in the wave before each quarter of this run
  };
  auto read_run = [&](int p, bool write_total) {
    const bool live = p < n_pairs;
    const int q = live ? p / KP : R, c = p % KP;   // lanes past the end read the stand-in record (zeros)
    const unsigned char *at = my_records + __umul24((uint32_t)q, (uint32_t)kRec) + c * (kQuarters * 8);
    RunWords r;
    r.lo = reinterpret_cast<const i32x4 *>(at)[0];
    r.hi = reinterpret_cast<const i32x4 *>(at)[1];
    const int n0 = __popc((uint32_t)r.lo.x), n1 = __popc((uint32_t)r.lo.z), n2 = __popc((uint32_t)r.hi.x),
              n3 = __popc((uint32_t)r.hi.z);
    const int in_run = (n0 + n1) + (n2 + n3);
    const int earlier_runs = group_exclusive_scan<KP>(in_run, c);
    r.before[0] = earlier_runs;
    r.before[1] = earlier_runs + n0;
    r.before[2] = earlier_runs + n0 + n1;
    r.before[3] = earlier_runs + n0 + n1 + n2;
    const int in_my_wave = group_sum<KP>(in_run);
    if (write_total && live && c == 0)
      wave_total[wave_s * R + q] = in_my_wave;
    return r;
  };
  // ordinal of each quarter's first token of the set: what is before this slice and in the waves before
  auto write_starts = [&](int p, RunWords &r) {
    if (p < n_pairs) {
      const int q = p / KP, c = p % KP;
      int32_t base = carry[q];
      for (int w = 0; w < wave_s; ++w)
        base += wave_total[w * R + q];
      unsigned char *at = my_records + __umul24((uint32_t)q, (uint32_t)kRec) + c * (kQuarters * 8);
      r.lo.y = base + r.before[0];
      r.lo.w = base + r.before[1];
      r.hi.y = base + r.before[2];
      r.hi.w = base + r.before[3];
      reinterpret_cast<i32x4 *>(at)[0] = r.lo;
      reinterpret_cast<i32x4 *>(at)[1] = r.hi;
    }
  };
  RunWords first = read_run(lane, true);
  for (int p = kWave + lane; p < (n_pairs + kWave - 1) / kWave * kWave; p += kWave)
    (void)read_run(p, true);
  LPLB_MAP_STAMP(2);
  __syncthreads();
  LPLB_MAP_STAMP(3);
  write_starts(lane, first);
  for (int p = kWave + lane; p < (n_pairs + kWave - 1) / kWave * kWave; p += kWave) {
    RunWords r = read_run(p, false);
    write_starts(p, r);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  LPLB_MAP_STAMP(4);
  // ---- C: ordinals, hashes, choices; all LDS reads first ----
  int2 rx[KP], ry[KP];   // bitmaps, start
#pragma unroll
  for (int c = 0; c < KP; ++c) {
    rx[c] = *reinterpret_cast<const int2 *>(smem_raw + wx[c]);
    ry[c] = *reinterpret_cast<const int2 *>(smem_raw + wy[c]);
  }
  auto choose = [&](const i32x4 &e, int32_t k) {
    const int32_t h = ordinal_hash<false>(k, e.x & kPairMaxTotal, (uint32_t)e.y);
    const int32_t slot = __builtin_amdgcn_sbfe(e.w, h >= e.z ? 16 : 0, 16);   // int16 -> int32
    return (long long)slot;
  };
  i64x2 o[KP];
#pragma unroll
  for (int c = 0; c < KP; ++c) {
    o[c].x = choose(ex[c], rx[c].y + __popc((uint32_t)rx[c].x & below_x));
    o[c].y = choose(ey[c], ry[c].y + __popc((uint32_t)ry[c].x & below_y));
  }
  if (whole) {
    i64x2 *dst = reinterpret_cast<i64x2 *>(a.out + w0) + lane;
#pragma unroll
    for (int c = 0; c < KP; ++c)
      __builtin_nontemporal_store(o[c], dst + c * kWave);
  } else {
#pragma unroll
    for (int c = 0; c < KP; ++c) {
      const int64_t i = w0 + c * kPairRun + 2 * lane;
      if (i < end)
        __builtin_nontemporal_store((long long)o[c].x, a.out + i);
      if (i + 1 < end)
        __builtin_nontemporal_store((long long)o[c].y, a.out + i + 1);
    }
  }
  LPLB_MAP_STAMP(5);
#ifdef LPLB_PHASE_CLOCKS
  __builtin_amdgcn_s_waitcnt(0);
#endif
  LPLB_MAP_STAMP(10);
}


template <int K, bool WRAP, bool TAIL, bool SINGLE>
static hipError_t launch_redirect_variant(const MapArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  if (lds > 64 * 1024) {
    const hipError_t err = allow_dynamic_lds(&redirect_indices<K, WRAP, TAIL, SINGLE>, 160 * 1024);
    if (err != hipSuccess)
      return err;
  }
  launch(redirect_indices<K, WRAP, TAIL, SINGLE>, grid, block, lds, s, a);
  return hipGetLastError();
}
template <int K, bool WRAP>
static hipError_t launch_redirect(const MapArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  // every slice a whole number of passes?  (the last slice may be shorter than the others)
  const int64_t pass_len = (int64_t)block.x * K;
  const bool whole = a.per % pass_len == 0 && a.n % pass_len == 0;
  const bool single = a.per <= pass_len;
  if (single)
    return whole ? launch_redirect_variant<K, WRAP, false, true>(a, grid, block, lds, s)
                 : launch_redirect_variant<K, WRAP, true, true>(a, grid, block, lds, s);
  return whole ? launch_redirect_variant<K, WRAP, false, false>(a, grid, block, lds, s)
               : launch_redirect_variant<K, WRAP, true, false>(a, grid, block, lds, s);
}

template <int KP, bool TAIL>
static hipError_t launch_pairs_variant(const MapArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  if (lds > 64 * 1024) {
    const hipError_t err = allow_dynamic_lds(&redirect_pairs<KP, TAIL>, 160 * 1024);
    if (err != hipSuccess)
      return err;
  }
  launch(redirect_pairs<KP, TAIL>, grid, block, lds, s, a);
  return hipGetLastError();
}
template <int KP> static hipError_t launch_pairs_runs(const MapArgs &a, dim3 grid, dim3 block, size_t lds, bool whole, hipStream_t s) {
  return whole ? launch_pairs_variant<KP, false>(a, grid, block, lds, s) : launch_pairs_variant<KP, true>(a, grid, block, lds, s);
}
static hipError_t launch_pairs(const MapArgs &a, int n_waves, int kp, size_t lds, hipStream_t s) {
  const dim3 grid(a.n_blocks), block(n_waves * kWave);
  // every slice exactly the workgroup's n_waves x kp runs?
  const bool whole = a.per == (int64_t)n_waves * kp * kPairRun && a.n % a.per == 0;
  switch (kp) {
  case 1: return launch_pairs_runs<1>(a, grid, block, lds, whole, s);
  case 2: return launch_pairs_runs<2>(a, grid, block, lds, whole, s);
  default: return launch_pairs_runs<4>(a, grid, block, lds, whole, s);
  }
}

// Shape of a mapping, as every entry point takes it.
static int shape_args(MapArgs &a, const char *who, int n_group, int group_size, int dup_per_rank, int n_combined_experts,
                      int n_local_experts) {
  LPLB_REQUIRE(n_group > 0 && group_size > 0 && dup_per_rank > 0 && n_combined_experts >= 0, LPLB_EINVAL,
               "%s: n_group=%d group_size=%d dup_per_rank=%d n_combined=%d", who, n_group, group_size, dup_per_rank,
               n_combined_experts);
  const int L = n_local_experts - dup_per_rank * n_combined_experts;
  LPLB_REQUIRE(L > 0 && L >= dup_per_rank * n_combined_experts, LPLB_EINVAL,
               "%s: n_local_experts=%d leaves %d logical experts per rank for %d replicas", who, n_local_experts, L,
               dup_per_rank * n_combined_experts);
  LPLB_REQUIRE((int64_t)n_group * group_size * n_local_experts < 65536, LPLB_EUNSUPPORTED,
               "%s: %lld physical experts exceed the 65535 the tables index", who,
               (long long)n_group * group_size * n_local_experts);
  a.n_ranks = n_group * group_size; a.n_logical = a.n_ranks * L;
  a.n_rep = a.n_ranks * n_combined_experts * dup_per_rank;
  a.G = group_size; a.D = dup_per_rank; a.C = n_combined_experts; a.L = L; a.P = n_local_experts;
  a.magic_L = fast_div_magic((uint32_t)L);
  a.magic_cd = fast_div_magic((uint32_t)(n_combined_experts * dup_per_rank));
  a.magic_D = fast_div_magic((uint32_t)dup_per_rank);
  a.magic_G = fast_div_magic((uint32_t)group_size);
  return LPLB_OK;
}
static int64_t prepared_words(const MapArgs &a) {
  return prepared_o2r_at(a.n_logical, a.n_rep, a.n_ranks * a.P) + (int64_t)a.G * a.D;
}

// The body of lplb_map_idx and lplb_map_idx_prepared (prepared: device table or null).
static int map_checked(const int64_t *idx, const float *o_weight, const int32_t *counts_by_block, const int32_t *o2r,
                       const int32_t *phy2log, const int32_t *prepared, int64_t n_elements, int n_group,
                       int group_size, int dup_per_rank, int n_combined_experts, int n_local_experts, int n_blocks,
                       int64_t *out, int32_t *physical_counts, hipStream_t s) {
  LPLB_REQUIRE(n_elements >= 0 && n_elements <= INT32_MAX, LPLB_EINVAL,
               "map_idx: n_elements=%lld out of range", (long long)n_elements);
  LPLB_REQUIRE(n_blocks > 0, LPLB_EINVAL, "map_idx: n_blocks=%d", n_blocks);
  MapArgs a{};
  const int rc = shape_args(a, "map_idx", n_group, group_size, dup_per_rank, n_combined_experts, n_local_experts);
  if (rc != LPLB_OK)
    return rc;
  LPLB_REQUIRE(o_weight && counts_by_block && (prepared || (o2r && phy2log)) && (n_elements == 0 || (idx && out)),
               LPLB_EINVAL, "map_idx: null pointer");
  // 499 k + 41 stays below 2^31 for every ordinal k < n_elements
  const bool wrap = n_elements > (INT32_MAX - 41) / 499;
  LPLB_REQUIRE(!(wrap && physical_counts), LPLB_EUNSUPPORTED,
               "map_idx: physical_counts needs n_elements <= %d", (INT32_MAX - 41) / 499);
  if (n_elements == 0) {
    if (physical_counts) {   // a kernel, not a memset: memset nodes misbehave in replayed HIP graphs here
      const int n_physical = n_group * group_size * n_local_experts;
      launch(zero_ints, dim3((n_physical + 255) / 256), dim3(256), 0, s, physical_counts, n_physical);
      LPLB_HIP_TRY(hipGetLastError());
    }
    return LPLB_OK;
  }
  a.idx = idx; a.o_weight = o_weight; a.by_block = counts_by_block;
  a.prepared = prepared;
  // (the prepared table carries copies of both, for the kernels that read them)
  a.phy2log = phy2log ? phy2log : prepared + prepared_phy2log_at(a.n_logical, a.n_rep);
  a.o2r = o2r ? o2r : prepared + prepared_o2r_at(a.n_logical, a.n_rep, a.n_ranks * a.P);
  a.n = n_elements; a.per = slice_len(n_elements, n_blocks);
  a.n_blocks = n_blocks; a.out = out; a.physical_counts = physical_counts;
  LPLB_REQUIRE(a.n_logical < 65536, LPLB_EUNSUPPORTED, "map_idx: %d logical experts exceed the 65535 the tables index",
               a.n_logical);
#ifdef LPLB_PHASE_CLOCKS
  a.clocks = g_phase_clocks;
#else
  a.clocks = nullptr;
#endif

  constexpr size_t kLdsLimit = 160 * 1024;
  // With a prepared table, slices of up to 8192 indices whose ends are 16-byte aligned go through
  // the kernel that moves two indices per lane and instruction.
  {
    const int64_t runs = (a.per + kPairRun - 1) / kPairRun;
    bool pairs = prepared != nullptr && !wrap && runs <= (int64_t)kMaxWaves * kMaxPairRuns && a.n_rep <= kPairMaxSets &&
                 n_elements <= kPairMaxTotal && a.n_ranks * a.P <= kPairMaxSlots &&
                 ((reinterpret_cast<uintptr_t>(idx) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    // as many waves as the slice has runs, up to 16 (two such workgroups fill a CU's wave slots, and one's
    // ranking overlaps the other's loads and stores), then 2 and 4 runs per wave
    int kp = runs > 2 * kMaxWaves ? 4 : runs > kMaxWaves ? 2 : 1;
    int n_waves = (int)((runs + kp - 1) / kp);
    if (pairs && n_waves <= kMaxWaves && (int64_t)n_waves * kp >= runs &&
        pairs_lds_bytes(a.n_logical, a.n_rep, n_waves, kp) <= kLdsLimit) {
      LPLB_HIP_TRY(launch_pairs(a, n_waves, kp, pairs_lds_bytes(a.n_logical, a.n_rep, n_waves, kp), s));
      return LPLB_OK;
    }
  }

  // Waves per workgroup: one per 64-index chunk of the slice, at most 16 when there is
  // one workgroup per CU; with more workgroups than CUs smaller ones (8, then 4 waves)
  // share a CU.  A wave takes K chunks per pass; two passes are in flight, so that one
  // pass's ranking and stores overlap the next one's loads.
  const int64_t chunks = (a.per + kWave - 1) / kWave;
  const int n_cus = current_device_cu_count();
  int max_waves = kMaxWaves;
  while (max_waves > 4 && n_cus > 0 && (int64_t)n_blocks * max_waves > (int64_t)kMaxWaves * n_cus)
    max_waves >>= 1;
  int n_waves = chunks < max_waves ? (int)chunks : max_waves;
  const int64_t per_wave = (chunks + n_waves - 1) / n_waves;
  int k = per_wave >= 8 ? 4 : per_wave >= 3 ? 2 : 1;
  while (k > 1 && map_lds_bytes(a.n_logical, a.n_rep, n_waves, k) > kLdsLimit)
    k >>= 1;
  while (n_waves > 1 && map_lds_bytes(a.n_logical, a.n_rep, n_waves, k) > kLdsLimit)
    n_waves >>= 1;
  const size_t lds = map_lds_bytes(a.n_logical, a.n_rep, n_waves, k);
  LPLB_REQUIRE(lds <= kLdsLimit, LPLB_EUNSUPPORTED,
               "map_idx: %d logical experts with %d replicated sets do not fit the LDS tables", a.n_logical,
               a.n_rep);
  const dim3 grid(n_blocks), block(n_waves * kWave);
  hipError_t err;
#define LPLB_MAP_CASE(K)                                                                    \
  err = wrap ? launch_redirect<K, true>(a, grid, block, lds, s)                             \
             : launch_redirect<K, false>(a, grid, block, lds, s)
  if (k <= 1) {
    LPLB_MAP_CASE(1);
  } else if (k <= 2) {
    LPLB_MAP_CASE(2);
  } else {
    LPLB_MAP_CASE(4);
  }
#undef LPLB_MAP_CASE
  LPLB_HIP_TRY(err);
  return LPLB_OK;
}

} // namespace lplb


extern "C" int lplb_map_idx(const int64_t *idx, const float *o_weight,
                            const int32_t *counts_by_block, const int32_t *o2r,
                            const int32_t *phy2log, int64_t n_elements,
                            int n_group, int group_size, int dup_per_rank,
                            int n_combined_experts, int n_local_experts,
                            int n_blocks, int64_t *out, int32_t *physical_counts,
                            lplb_stream_t stream) {
  LPLB_REQUIRE(o2r && phy2log, LPLB_EINVAL, "map_idx: null pointer");
  return lplb::map_checked(idx, o_weight, counts_by_block, o2r, phy2log, nullptr, n_elements, n_group, group_size,
                           dup_per_rank, n_combined_experts, n_local_experts, n_blocks, out, physical_counts,
                           static_cast<hipStream_t>(stream));
}

extern "C" int64_t lplb_prepared_mapping_bytes(int n_group, int group_size, int dup_per_rank,
                                               int n_combined_experts, int n_local_experts) {
  using namespace lplb;
  MapArgs a{};
  if (shape_args(a, "prepared_mapping_bytes", n_group, group_size, dup_per_rank, n_combined_experts,
                 n_local_experts) != LPLB_OK)
    return -1;
  return prepared_words(a) * (int64_t)sizeof(int32_t);
}

extern "C" int lplb_prepare_mapping(const int32_t *o2r, const int32_t *phy2log, int n_group,
                                    int group_size, int dup_per_rank, int n_combined_experts,
                                    int n_local_experts, void *prepared, int64_t prepared_bytes,
                                    lplb_stream_t stream) {
  using namespace lplb;
  MapArgs a{};
  const int rc = shape_args(a, "prepare_mapping", n_group, group_size, dup_per_rank, n_combined_experts, n_local_experts);
  if (rc != LPLB_OK)
    return rc;
  LPLB_REQUIRE(o2r && phy2log && prepared, LPLB_EINVAL, "prepare_mapping: null pointer");
  LPLB_REQUIRE((reinterpret_cast<uintptr_t>(prepared) & 15) == 0, LPLB_EINVAL,
               "prepare_mapping: the table must be 16-byte aligned");
  LPLB_REQUIRE(prepared_bytes >= prepared_words(a) * (int64_t)sizeof(int32_t), LPLB_EINVAL,
               "prepare_mapping: the table needs %lld bytes, got %lld",
               (long long)(prepared_words(a) * (int64_t)sizeof(int32_t)), (long long)prepared_bytes);
  const size_t lds = (size_t)(a.n_logical + 1) * sizeof(ExpertPlan) + (size_t)a.n_rep * sizeof(int32_t) + 16;
  LPLB_REQUIRE(a.n_rep <= kPairMaxSets && a.n_ranks * a.P <= kPairMaxSlots && lds <= 160 * 1024, LPLB_EUNSUPPORTED,
               "prepare_mapping: %d logical experts / %d replicated sets / %d physical experts are more than a "
               "prepared table holds (%d sets, %d physical experts)", a.n_logical, a.n_rep, a.n_ranks * a.P,
               kPairMaxSets, kPairMaxSlots);
  a.o2r = o2r; a.phy2log = phy2log;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (lds > 64 * 1024)
    LPLB_HIP_TRY(allow_dynamic_lds(&prepare_mapping, 160 * 1024));
  launch(prepare_mapping, dim3(1), dim3(1024), lds, s, a, static_cast<int32_t *>(prepared));
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}

extern "C" int lplb_map_idx_prepared(const int64_t *idx, const float *o_weight,
                                     const int32_t *counts_by_block, const void *prepared,
                                     int64_t n_elements, int n_group, int group_size,
                                     int dup_per_rank, int n_combined_experts,
                                     int n_local_experts, int n_blocks, int64_t *out,
                                     int32_t *physical_counts, lplb_stream_t stream) {
  LPLB_REQUIRE(prepared != nullptr && (reinterpret_cast<uintptr_t>(prepared) & 15) == 0, LPLB_EINVAL,
               "map_idx_prepared: the prepared table is null or not 16-byte aligned");
  return lplb::map_checked(idx, o_weight, counts_by_block, nullptr, nullptr, static_cast<const int32_t *>(prepared),
                           n_elements, n_group, group_size, dup_per_rank, n_combined_experts, n_local_experts, n_blocks,
                           out, physical_counts, static_cast<hipStream_t>(stream));
}


extern "C" int lplb_map_idx_prepared_series(const int64_t *const *idx, const float *o_weight,
                                            const int32_t *const *counts_by_block, const void *prepared,
                                            int64_t n_elements, int n_group, int group_size,
                                            int dup_per_rank, int n_combined_experts,
                                            int n_local_experts, int n_blocks, int64_t *const *out,
                                            int n_launches, void *const *start_events,
                                            void *const *stop_events, lplb_stream_t stream) {
  LPLB_REQUIRE(idx && counts_by_block && out && n_launches >= 0, LPLB_EINVAL,
               "map_idx_prepared_series: null pointer or negative count");
  for (int r = 0; r < n_launches; ++r) {
    lplb_time_next_launch(start_events ? start_events[r] : nullptr, stop_events ? stop_events[r] : nullptr);
    const int rc = lplb_map_idx_prepared(idx[r], o_weight, counts_by_block[r], prepared, n_elements, n_group, group_size,
                                         dup_per_rank, n_combined_experts, n_local_experts, n_blocks, out[r], nullptr,
                                         stream);
    if (rc != LPLB_OK) {
      lplb_time_next_launch(nullptr, nullptr);   // (an entry point that fails before its launch leaves the pair armed)
      return rc;
    }
  }
  return LPLB_OK;
}
