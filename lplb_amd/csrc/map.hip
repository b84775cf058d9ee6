// Logical -> physical redirect of routing indices (streaming, HBM-bound:
// 8 bytes read + 8 bytes written per index).
//
// Each token needs its ordinal k among the tokens of the same expert, in index
// order, because the original/replica decision hashes k.  The reference takes k
// from a shared-memory atomic (minilp.cu:504), which fixes the set of ordinals
// per block but not which token gets which.  Here k is canonical.
//
// A workgroup walks its slice in passes of n_waves * K consecutive 64-index chunks,
// K per wave.  The loads of the first pass are issued up front (before the small
// table loads are used), those of every later pass while the pass before it is
// still being ranked and stored.  Per pass:
//   A  each wave histograms its K chunks into its own LDS counter row;
//   B  each wave turns the rows into its starting ordinals (running total of
//      earlier slices and passes + counts of the waves before it);
//   C  chunk by chunk, lanes holding the same expert find each other through a
//      per-wave 64-bit LDS bitmap (one OR, one 16-byte read); the rank among those
//      peers is a popcount of lower lanes and the last peer advances the counter.
// Counter rows and running totals are double-buffered by pass parity, which
// leaves one workgroup barrier per pass.  Nothing depends on execution order.
// The modulo of the hash uses a per-expert reciprocal prepared with the tables.
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
  int n_logical, n_ranks, G, D, C, L, P, n_blocks;
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

template <int K, bool WRAP>
__global__ __launch_bounds__(kMaxWaves *kWave) void redirect_indices(MapArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int nl = a.n_logical;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid % kWave, wave = tid / kWave, n_waves = nt / kWave;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);   // the same, but known to be wave-uniform
  const int pid = blockIdx.x;
  ExpertEntry *table = reinterpret_cast<ExpertEntry *>(smem_raw);                 // [nl]
  WaveSlot *slots = reinterpret_cast<WaveSlot *>(table + nl);                    // [n_waves][nl]
  int32_t *replica = reinterpret_cast<int32_t *>(slots + (size_t)n_waves * nl);  // [nl]
  int32_t *carry = replica + nl;                                                 // [2][nl]
  int32_t *counts = carry + 2 * nl;                                              // [2][n_waves][nl]
  const int32_t *last = a.by_block + (int64_t)(a.n_blocks - 1) * nl;
  const int32_t *prev = pid ? a.by_block + (int64_t)(pid - 1) * nl : nullptr;

  const int64_t begin = slice_begin(a.n, a.per, pid);
  const int64_t end = slice_begin(a.n, a.per, pid + 1);
  const int64_t pass_len = (int64_t)n_waves * K * kWave;
  WaveSlot *mine = slots + (size_t)wave * nl;
  const unsigned long long my_bit = 1ull << lane;
  LPLB_MAP_STAMP(0);

  // Global reads of the table build (small, mostly L2 hits) go out first, the
  // first pass's indices right behind them, so that the build does not wait for
  // the bulk data.  Tables, minilp.cu:466-496.
  const int cd = a.C * a.D;
  const int e0 = tid;                                   // first (usually only) expert of this thread
  const int32_t t0 = e0 < nl ? last[e0] : 0;
  const int32_t s0 = (e0 < nl && prev) ? prev[e0] : 0;
  const int le0 = e0 < nl ? a.phy2log[(e0 / a.L) * a.P + (e0 % a.L)] : -1;
  const bool rep0 = tid < a.n_ranks * cd;               // first replicated expert set of this thread
  const int rank0 = rep0 ? tid / cd : 0, local0 = rep0 ? tid % cd : 0;
  const int rle0 = rep0 ? a.phy2log[rank0 * a.P + local0] : -1;
  const float share0 = rep0 ? a.o_weight[rank0 * a.D + local0 % a.D] : 0.0f;
  const int host0 = rep0 ? a.o2r[(rank0 % a.G) * a.D + local0 % a.D] : 0;

  // One pass of indices, as loaded (raw) and as expert ids (ev: -1 for masked /
  // out-of-range / past the end).  The loads of the next pass are issued while the
  // current one is still being ranked and stored.
  int64_t raw[K];
  int32_t ev[K];
  auto issue_loads = [&](int64_t pass) {
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const int64_t i = pass + ((int64_t)wave * K + c) * kWave + lane;
      raw[c] = i < end ? __builtin_nontemporal_load(a.idx + i) : -1;
    }
  };
  auto take_loads = [&]() {
#pragma unroll
    for (int c = 0; c < K; ++c)
      ev[c] = (raw[c] >= 0 && raw[c] < nl) ? (int32_t)raw[c] : -1;
  };
  issue_loads(begin);

  const RedirectShape sh{nl, a.n_ranks, a.G, a.D, a.C, a.L, a.P};
  if (e0 < nl)
    init_entry(table, replica, carry, e0, t0, s0);
  for (int e = tid + nt; e < nl; e += nt)
    init_entry(table, replica, carry, e, last[e], prev ? prev[e] : 0);
  for (int i = tid; i < n_waves * nl; i += nt) {
    slots[i] = WaveSlot{0, 0, 0ull};
    counts[i] = 0;
    counts[n_waves * nl + i] = 0;
  }
  __syncthreads();
  if (e0 < nl)
    set_original(table, sh, e0, le0);
  for (int e = tid + nt; e < nl; e += nt)
    set_original(table, sh, e, a.phy2log[(e / a.L) * a.P + (e % a.L)]);
  if (rep0)
    set_replica(table, replica, sh, rank0, local0, rle0, share0, host0);
  for (int i = tid + nt; i < a.n_ranks * cd; i += nt) {
    const int ep_rank = i / cd, local = i % cd, d = local % a.D;
    set_replica(table, replica, sh, ep_rank, local, a.phy2log[ep_rank * a.P + local],
                a.o_weight[ep_rank * a.D + d], a.o2r[(ep_rank % a.G) * a.D + d]);
  }
  // (the barrier after the first phase A also publishes the tables)
  LPLB_MAP_STAMP(1);

  int parity = 0;   // which half of counts / carry the current pass uses
  for (int64_t pass = begin; pass < end; pass += pass_len) {
    take_loads();
    int32_t *my_counts = counts + ((size_t)parity * n_waves + wave) * nl;
    // Phase A: tokens per expert in this wave's chunks.
#pragma unroll
    for (int c = 0; c < K; ++c)
      if (ev[c] >= 0)
        atomicAdd(&my_counts[ev[c]], 1);
    if (pass + pass_len < end)
      issue_loads(pass + pass_len);   // in flight during the barrier, phases B and C
    LPLB_MAP_STAMP(2);
    __syncthreads();
    LPLB_MAP_STAMP(3);
    // Phase B: every wave derives its own starting ordinals: the running total
    // of earlier slices and passes plus the counts of the waves before it.  The
    // last wave writes the next pass's running total into the other half, and
    // every wave clears its row of the other half for the next pass.
    const int32_t *pass_counts = counts + (size_t)parity * n_waves * nl;
    int32_t *other_counts = counts + ((size_t)(parity ^ 1) * n_waves + wave) * nl;
    // The code is specialised by the number of earlier waves (wave-uniform), so that
    // the inner loop is straight-line: exactly that many reads, no branches.
    static_for<kMaxWaves>([&](auto wc) {
      constexpr int kEarlier = decltype(wc)::value;
      if (wave_s != kEarlier)
        return;
      for (int e = lane; e < nl; e += kWave) {
        // all reads in flight before the first add
        int32_t before[kEarlier + 1];
#pragma unroll
        for (int w = 0; w < kEarlier; ++w)
          before[w] = pass_counts[(size_t)w * nl + e];
        int32_t run = carry[parity * nl + e];
        const int32_t own = my_counts[e];
#pragma unroll
        for (int w = 0; w < kEarlier; ++w)
          run += before[w];
        mine[e].next = run;
        if (kEarlier == n_waves - 1)
          carry[(parity ^ 1) * nl + e] = run + own;
        other_counts[e] = 0;
      }
    });
    __builtin_amdgcn_wave_barrier();
    LPLB_MAP_STAMP(4);
    // Phase C.
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const int64_t o = redirect_token<WRAP>(ev[c], mine, table, replica, my_bit);
      const int64_t i = pass + ((int64_t)wave * K + c) * kWave + lane;
      if (i < end)
        __builtin_nontemporal_store(o, a.out + i);
      __builtin_amdgcn_wave_barrier();
    }
    LPLB_MAP_STAMP(5);
    parity ^= 1;
  }
  if (pid == 0 && a.physical_counts)   // the tables are complete since the first barrier
    emit_physical_counts(table, replica, sh, a.phy2log, a.physical_counts, tid, nt);
  __builtin_amdgcn_s_waitcnt(0);
  LPLB_MAP_STAMP(6);
}

// LDS bytes for n_logical experts and w waves.
static size_t map_lds_bytes(int n_logical, int w) {
  return (size_t)n_logical * (sizeof(ExpertEntry) + 4 + 8 + (size_t)w * (sizeof(WaveSlot) + 8));
}

template <int K, bool WRAP>
static hipError_t launch_redirect(const MapArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  if (lds > 64 * 1024) {
    const hipError_t err = allow_dynamic_lds(&redirect_indices<K, WRAP>, 160 * 1024);
    if (err != hipSuccess)
      return err;
  }
  launch(redirect_indices<K, WRAP>, grid, block, lds, s, a);
  return hipGetLastError();
}

} // namespace lplb

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
  a.G = group_size; a.D = dup_per_rank; a.C = n_combined_experts; a.L = L;
  a.P = n_local_experts; a.n_blocks = n_blocks; a.out = out; a.physical_counts = physical_counts;
#ifdef LPLB_PHASE_CLOCKS
  a.clocks = g_phase_clocks;
#else
  a.clocks = nullptr;
#endif

  // One wave per 64-index chunk of the slice, as LDS allows, then up to 8 chunks per
  // wave and pass.  At most 16 waves when there is one workgroup per CU; with more
  // workgroups than CUs smaller ones (8, then 4 waves) share a CU, and one's ranking
  // phases overlap another's loads and stores (measured at 512 MiB in + 512 MiB out:
  // 1024 slices of 4 waves 4.9 TB/s, 256 slices of 16 waves 4.1 TB/s).
  const int64_t chunks = (a.per + kWave - 1) / kWave;
  const int n_cus = current_device_cu_count();
  int max_waves = kMaxWaves;
  while (max_waves > 4 && n_cus > 0 && (int64_t)n_blocks * max_waves > (int64_t)kMaxWaves * n_cus)
    max_waves >>= 1;
  int n_waves = chunks < max_waves ? (int)chunks : max_waves;
  constexpr size_t kLdsLimit = 160 * 1024;
  while (n_waves > 1 && map_lds_bytes(a.n_logical, n_waves) > kLdsLimit)
    n_waves >>= 1;
  LPLB_REQUIRE(map_lds_bytes(a.n_logical, n_waves) <= kLdsLimit, LPLB_EUNSUPPORTED,
               "map_idx: %d logical experts do not fit the LDS tables", a.n_logical);
  const int64_t per_wave = (chunks + n_waves - 1) / n_waves;
  const size_t lds = map_lds_bytes(a.n_logical, n_waves);
  const dim3 grid(n_blocks), block(n_waves * kWave);
  hipError_t err;
#define LPLB_MAP_CASE(K)                                                                    \
  err = wrap ? launch_redirect<K, true>(a, grid, block, lds, s)                             \
             : launch_redirect<K, false>(a, grid, block, lds, s)
  // K chunks per wave and pass (K loads in flight per lane, K more prefetched).
  // Measured at [262144 x 8] on MI355X: a pass costs about 2.5 us of barrier skew
  // and counter traffic, so a pass is as long as registers allow (8 chunks per
  // wave); longer slices loop over passes.
  if (per_wave <= 1) {
    LPLB_MAP_CASE(1);
  } else if (per_wave <= 2) {
    LPLB_MAP_CASE(2);
  } else if (per_wave <= 4) {
    LPLB_MAP_CASE(4);
  } else {
    LPLB_MAP_CASE(8);
  }
#undef LPLB_MAP_CASE
  LPLB_HIP_TRY(err);
  return LPLB_OK;
}
