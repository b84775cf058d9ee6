// Logical -> physical redirect of routing indices (streaming, HBM-bound:
// 8 bytes read + 8 bytes written per index).
//
// Each token needs its ordinal k among the tokens of the same expert, in index
// order, because the original/replica decision hashes k.  The reference takes k
// from a shared-memory atomic (minilp.cu:504), which fixes the set of ordinals
// per block but not which token gets which.  Here k is canonical.  A workgroup
// walks its slice in rounds of n_waves * K * 64 indices; in a round every wave
// owns K consecutive 64-index chunks, loaded once into registers with all loads
// in flight together:
//   A  each wave histograms its chunks into its own LDS counter row;
//   B  the rows become exclusive starting ordinals (running total of earlier
//      slices and rounds + earlier waves of this round);
//   C  chunk by chunk, lanes holding the same expert find each other through a
//      per-wave 64-bit LDS bitmap (one OR, one read); the rank among those peers
//      is a popcount of lower lanes and the last peer advances the counter.
// Two workgroup barriers per round, nothing order-dependent.  The modulo of the
// hash uses a per-expert reciprocal prepared with the tables.
#include "common.h"

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
};

// Per-expert constants of the redirect, one 16-byte LDS read per token.
struct __attribute__((aligned(16))) ExpertEntry {
  int32_t total;     // tokens of this expert in the whole index array
  uint32_t magic;    // floor(2^32 / total) (all ones for total == 1)
  int32_t expected;  // tokens that stay on the original, trunc(o_weight * total)
  int32_t original;  // physical slot of the original
};

// |h| mod t with q = mulhi(|h|, magic): q is the true quotient or one less.
__device__ inline int32_t hashed_mod(int32_t h, const ExpertEntry &x) {
  if (x.total <= 0)
    return 0;
  const uint32_t a = h < 0 ? 0u - (uint32_t)h : (uint32_t)h;
  uint32_t r = a - __umulhi(a, x.magic) * (uint32_t)x.total;
  r = r >= (uint32_t)x.total ? r - (uint32_t)x.total : r;
  return h < 0 ? -(int32_t)r : (int32_t)r;   // C's truncating %
}

constexpr int kMaxWaves = 16;

template <int K>
__global__ __launch_bounds__(kMaxWaves *kWave) void redirect_indices(MapArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int nl = a.n_logical;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid % kWave, wave = tid / kWave, n_waves = nt / kWave;
  const int pid = blockIdx.x;
  ExpertEntry *table = reinterpret_cast<ExpertEntry *>(smem_raw);                 // [nl]
  unsigned long long *bitmap = reinterpret_cast<unsigned long long *>(table + nl); // [n_waves][nl]
  int32_t *replica = reinterpret_cast<int32_t *>(bitmap + (size_t)n_waves * nl);   // [nl]
  int32_t *carry = replica + nl;                                                   // [nl]
  int32_t *base = carry + nl;                                                      // [n_waves][nl]
  const int32_t *last = a.by_block + (int64_t)(a.n_blocks - 1) * nl;
  const int32_t *prev = pid ? a.by_block + (int64_t)(pid - 1) * nl : nullptr;

  const int64_t begin = slice_begin(a.n, a.per, pid);
  const int64_t end = slice_begin(a.n, a.per, pid + 1);
  const int64_t round_len = (int64_t)n_waves * K * kWave;
  int32_t *mine = base + wave * nl;
  unsigned long long *my_bits = bitmap + (size_t)wave * nl;
  const unsigned long long my_bit = 1ull << lane;

  // First round's indices: issued before anything else so that their latency
  // overlaps the table build.  ev = expert id, or -1 for masked / out-of-range /
  // past the end.
  int32_t ev[K];
  auto load_round = [&](int64_t round) {
    const int64_t wbeg = round + (int64_t)wave * K * kWave;
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const int64_t i = wbeg + c * kWave + lane;
      const int64_t v = i < end ? __builtin_nontemporal_load(a.idx + i) : -1;
      ev[c] = (v >= 0 && v < nl) ? (int32_t)v : -1;
    }
  };
  load_round(begin);

  // Tables, minilp.cu:466-496.  All global reads of the build are independent of
  // each other; the replicas' totals come back from LDS after the barrier.
  const int cd = a.C * a.D;
  for (int e = tid; e < nl; e += nt) {
    const int32_t t = last[e];
    const int32_t start = prev ? prev[e] : 0;
    table[e].total = t;
    table[e].magic = t > 1 ? (uint32_t)(0x100000000ull / (uint32_t)t) : 0xffffffffu;
    table[e].expected = t;
    table[e].original = -1;
    replica[e] = -1;
    carry[e] = start;
  }
  for (int i = tid; i < n_waves * nl; i += nt) {
    base[i] = 0;
    bitmap[i] = 0;
  }
  __syncthreads();
  for (int e = tid; e < nl; e += nt) {
    const int slot = (e / a.L) * a.P + (e % a.L);
    const int le = a.phy2log[slot];
    if (le >= 0 && le < nl)
      table[le].original = slot;
  }
  for (int i = tid; i < a.n_ranks * cd; i += nt) {
    const int ep_rank = i / cd, local = i % cd, d = local % a.D;
    const int le = a.phy2log[ep_rank * a.P + local];
    const float share = a.o_weight[ep_rank * a.D + d];
    const int host = a.o2r[(ep_rank % a.G) * a.D + d];
    if (le >= 0 && le < nl) {
      // fp32 product truncated toward zero (saturating, NaN -> 0)
      table[le].expected = __float2int_rz(share * (float)table[le].total);
      replica[le] = ((ep_rank / a.G) * a.G + host + 1) * a.P - cd + local;
    }
  }
  // (the barrier of phase A below also publishes the tables)

  for (int64_t round = begin; round < end; round += round_len) {
    const int64_t wbeg = round + (int64_t)wave * K * kWave;
    if (round != begin) {
      load_round(round);
      // counter rows still hold the previous round's ordinals
      __syncthreads();
      for (int i = tid; i < n_waves * nl; i += nt)
        base[i] = 0;
      __syncthreads();
    }
    // Phase A.
#pragma unroll
    for (int c = 0; c < K; ++c)
      if (ev[c] >= 0)
        atomicAdd(&mine[ev[c]], 1);
    __syncthreads();
    // Phase B: all rows of an expert are read before any is rewritten.
    for (int e = tid; e < nl; e += nt) {
      int32_t cnt[kMaxWaves];
#pragma unroll
      for (int w = 0; w < kMaxWaves; ++w)
        cnt[w] = w < n_waves ? base[w * nl + e] : 0;
      int32_t run = carry[e];
#pragma unroll
      for (int w = 0; w < kMaxWaves; ++w)
        if (w < n_waves) {
          base[w * nl + e] = run;
          run += cnt[w];
        }
      carry[e] = run;
    }
    __syncthreads();
    // Phase C.
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const int e = ev[c];
      const bool valid = e >= 0;
      if (valid)
        atomicOr(&my_bits[e], my_bit);
      int64_t o = -1;
      if (valid) {
        const unsigned long long peers =
            __hip_atomic_load(&my_bits[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        const int rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(peers >> 32),
                                                   __builtin_amdgcn_mbcnt_lo((uint32_t)peers, 0u));
        const int cnt = __popcll(peers);
        const int32_t k = mine[e] + rank;
        const ExpertEntry x = table[e];
        // (k * 499 + 41) % total in int32 arithmetic (minilp.cu:505)
        const int32_t h = hashed_mod((int32_t)((uint32_t)k * 499u + 41u), x);
        o = h >= x.expected ? replica[e] : x.original;
        if (rank == cnt - 1) {
          mine[e] = k + 1;
          my_bits[e] = 0;
        }
      }
      const int64_t i = wbeg + c * kWave + lane;
      if (i < end)
        __builtin_nontemporal_store(o, a.out + i);
      __builtin_amdgcn_wave_barrier();
    }
  }
}

// LDS bytes for n_logical experts and w waves.
static size_t map_lds_bytes(int n_logical, int w) {
  return (size_t)n_logical * (sizeof(ExpertEntry) + 8 + (size_t)w * 12);
}

} // namespace lplb

extern "C" int lplb_map_idx(const int64_t *idx, const float *o_weight,
                            const int32_t *counts_by_block, const int32_t *o2r,
                            const int32_t *phy2log, int64_t n_elements,
                            int n_group, int group_size, int dup_per_rank,
                            int n_combined_experts, int n_local_experts,
                            int n_blocks, int64_t *out, lplb_stream_t stream) {
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
  if (n_elements == 0)
    return LPLB_OK;

  MapArgs a;
  a.idx = idx; a.o_weight = o_weight; a.by_block = counts_by_block; a.o2r = o2r;
  a.phy2log = phy2log; a.n = n_elements; a.per = slice_len(n_elements, n_blocks);
  a.n_ranks = n_group * group_size; a.n_logical = a.n_ranks * L;
  a.G = group_size; a.D = dup_per_rank; a.C = n_combined_experts; a.L = L;
  a.P = n_local_experts; a.n_blocks = n_blocks; a.out = out;

  // One wave per 64-index chunk of the slice, up to 16 waves, as LDS allows;
  // then up to 8 chunks per wave and round.
  const int64_t chunks = (a.per + kWave - 1) / kWave;
  int n_waves = chunks < kMaxWaves ? (int)chunks : kMaxWaves;
  constexpr size_t kLdsLimit = 64 * 1024;
  while (n_waves > 1 && map_lds_bytes(a.n_logical, n_waves) > kLdsLimit)
    n_waves >>= 1;
  LPLB_REQUIRE(map_lds_bytes(a.n_logical, n_waves) <= kLdsLimit, LPLB_EUNSUPPORTED,
               "map_idx: %d logical experts do not fit the LDS tables", a.n_logical);
  const int64_t per_wave = (chunks + n_waves - 1) / n_waves;
  const size_t lds = map_lds_bytes(a.n_logical, n_waves);
  const dim3 grid(n_blocks), block(n_waves * kWave);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (per_wave <= 1)
    launch(redirect_indices<1>, grid, block, lds, s, a);
  else if (per_wave <= 2)
    launch(redirect_indices<2>, grid, block, lds, s, a);
  else if (per_wave <= 4)
    launch(redirect_indices<4>, grid, block, lds, s, a);
  else
    launch(redirect_indices<8>, grid, block, lds, s, a);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}
