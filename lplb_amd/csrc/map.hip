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
  long long *clocks;   // debug builds: stamps of the first and the last workgroup (else null)
};
#define LPLB_MAP_STAMP(k)                                                                      \
  LPLB_STAMP_AT(blockIdx.x == 0 ? a.clocks + 32 : (blockIdx.x == gridDim.x - 1 ? a.clocks + 48 : nullptr), k)

__global__ void zero_ints(int32_t *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    p[i] = 0;
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
  const int cd = a.C * a.D;
  LPLB_MAP_STAMP(0);

  // ---- small global reads of the table build first (mostly L2 hits), minilp.cu:466-496 ----
  // original slot of logical position e: rank e / L, place e % L
  auto slot_of = [&](int e) { return e + (int)fast_div((uint32_t)e, a.magic_L) * (a.P - a.L); };
  // replicated set i = (ep_rank, place): its expert, its share, the group rank that holds the copy
  struct SetOf {
    int ep_rank, place, d, group_rank;
  };
  auto set_of = [&](int i) {
    SetOf s;
    s.ep_rank = (int)fast_div((uint32_t)i, a.magic_cd);
    s.place = i - s.ep_rank * cd;
    s.d = s.place - (int)fast_div((uint32_t)s.place, a.magic_D) * a.D;
    s.group_rank = s.ep_rank - (int)fast_div((uint32_t)s.ep_rank, a.magic_G) * a.G;
    return s;
  };
  // All of them are unconditional loads from clamped addresses: a load inside a branch
  // makes the compiler wait for it right there, before the index loads are issued.
  const int e0 = min(tid, nl - 1);                          // first (usually only) expert of this thread
  const int slot0 = slot_of(e0);
  const int le0 = a.phy2log[slot0];
  // The counts are read per expert, not per replicated set, so that they do not have to
  // wait for phy2log (a load issued after the index loads returns after them).
  const int32_t total0 = last[e0];
  const int32_t before0_raw = (prev ? prev : last)[e0];
  const bool set0 = tid < R;                               // first (usually only) replicated set
  const SetOf s0 = set_of(set0 ? tid : 0);
  // (with no replicated set at all, R == 0, these read element 0 of each table)
  const int rle0 = a.phy2log[s0.ep_rank * a.P + s0.place];
  const float share0 = a.o_weight[s0.ep_rank * a.D + s0.d];
  const int host0 = a.o2r[s0.group_rank * a.D + s0.d];

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
  for (int e = tid; e <= nl; e += nt)
    route[e] = Route{-1, R};
  {
    const i32x4 zero{0, 0, 0, 0};
    i32x4 *z = reinterpret_cast<i32x4 *>(records);
    for (int i = tid; i < n_waves * wave_stride / 16; i += nt)
      z[i] = zero;
  }
  if (tid == 0)
    reps[R] = RepEntry{1, 0xffffffffu, INT32_MAX, -1};   // "no replica": every token stays
  if (tid < nl) {
    staged[tid] = total0;
    staged[nl + tid] = prev ? before0_raw : 0;
  }
  for (int e = tid + nt; e < nl; e += nt) {
    staged[e] = last[e];
    staged[nl + e] = prev ? prev[e] : 0;
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
  auto fill_set = [&](int i, const SetOf &s, int le, float share, int host) {
    const bool ok = le >= 0 && le < nl;
    const int32_t t = ok ? staged[le] : 0;
    const int32_t before = ok ? staged[nl + le] : 0;
    if (ok)
      atomicMin(&route[le].rep, R - 1 - i);
    RepEntry x;
    x.total = t;
    x.magic = t >= 1 ? 0xffffffffu / (uint32_t)t : 0u;
    x.expected = expected_on_original(share, t);
    x.replica = ((s.ep_rank - s.group_rank) + host + 1) * a.P - cd + s.place;
    reps[R - 1 - i] = x;
    carry[R - 1 - i] = before;
  };
  if (set0)
    fill_set(tid, s0, rle0, share0, host0);
  for (int i = tid + nt; i < R; i += nt) {
    const SetOf s = set_of(i);
    fill_set(i, s, a.phy2log[s.ep_rank * a.P + s.place], a.o_weight[s.ep_rank * a.D + s.d],
             a.o2r[s.group_rank * a.D + s.d]);
  }
  __syncthreads();
  LPLB_MAP_STAMP(1);
  // Tokens per physical expert (= bincount of the output) from the tables alone.
  if (counts_wanted)
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

#ifdef LPLB_TUNING
// Tuning builds only: force the launch shape of the redirect (0 = choose as usual).
int g_force_waves = 0, g_force_k = 0;
#endif

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

} // namespace lplb

#ifdef LPLB_TUNING
extern "C" void lplb_debug_force_redirect_shape(int waves, int k) {
  lplb::g_force_waves = waves;
  lplb::g_force_k = k;
}
#endif

extern "C" int lplb_map_idx(const int64_t *idx, const float *o_weight,
                            const int32_t *counts_by_block, const int32_t *o2r,
                            const int32_t *phy2log, int64_t n_elements,
                            int n_group, int group_size, int dup_per_rank,
                            int n_combined_experts, int n_local_experts,
                            int n_blocks, int64_t *out, int32_t *physical_counts,
                            lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(n_elements >= 0 && n_elements <= INT32_MAX, LPLB_EINVAL,
               "map_idx: n_elements=%lld out of range", (long long)n_elements);
  LPLB_REQUIRE(n_group > 0 && group_size > 0 && dup_per_rank > 0 && n_combined_experts >= 0 &&
                   n_blocks > 0,
               LPLB_EINVAL, "map_idx: n_group=%d group_size=%d dup_per_rank=%d n_combined=%d n_blocks=%d",
               n_group, group_size, dup_per_rank, n_combined_experts, n_blocks);
  const int L = n_local_experts - dup_per_rank * n_combined_experts;
  LPLB_REQUIRE(L > 0 && L >= dup_per_rank * n_combined_experts, LPLB_EINVAL,
               "map_idx: n_local_experts=%d leaves %d logical experts per rank for %d replicas",
               n_local_experts, L, dup_per_rank * n_combined_experts);
  LPLB_REQUIRE(o_weight && counts_by_block && o2r && phy2log && (n_elements == 0 || (idx && out)),
               LPLB_EINVAL, "map_idx: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
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

  MapArgs a{};
  a.idx = idx; a.o_weight = o_weight; a.by_block = counts_by_block; a.o2r = o2r;
  a.phy2log = phy2log; a.n = n_elements; a.per = slice_len(n_elements, n_blocks);
  a.n_ranks = n_group * group_size; a.n_logical = a.n_ranks * L;
  a.n_rep = a.n_ranks * n_combined_experts * dup_per_rank;
  a.G = group_size; a.D = dup_per_rank; a.C = n_combined_experts; a.L = L;
  a.P = n_local_experts; a.n_blocks = n_blocks; a.out = out; a.physical_counts = physical_counts;
  LPLB_REQUIRE(a.n_logical < 65536 && a.n_ranks * a.P < 65536, LPLB_EUNSUPPORTED,
               "map_idx: %d logical / %d physical experts exceed the 65535 the tables index", a.n_logical,
               a.n_ranks * a.P);
  a.magic_L = fast_div_magic((uint32_t)L);
  a.magic_cd = fast_div_magic((uint32_t)(n_combined_experts * dup_per_rank));
  a.magic_D = fast_div_magic((uint32_t)dup_per_rank);
  a.magic_G = fast_div_magic((uint32_t)group_size);
#ifdef LPLB_PHASE_CLOCKS
  a.clocks = g_phase_clocks;
#else
  a.clocks = nullptr;
#endif

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
#ifdef LPLB_TUNING
  if (g_force_waves > 0)
    n_waves = min(g_force_waves, kMaxWaves);
  if (g_force_k > 0)
    k = g_force_k;
#endif
  constexpr size_t kLdsLimit = 160 * 1024;
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
