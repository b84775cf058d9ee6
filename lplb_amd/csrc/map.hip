// Logical -> physical redirect of routing indices (streaming, HBM-bound:
// 8 bytes read + 8 bytes written per index).
//
// Each token needs its ordinal k among the tokens of the same expert, in index
// order, because the original/replica decision hashes k.  The reference takes k
// from a shared-memory atomic (minilp.cu:504), which fixes the set of ordinals
// per block but not which token gets which.  Here k is canonical:
//   * the slice of a workgroup is cut into contiguous sub-slices, one per wave;
//   * phase A histograms every sub-slice into the wave's own LDS counter row;
//   * phase B turns the rows into exclusive starting ordinals
//     (previous slices' prefix + earlier waves of this slice);
//   * phase C walks the sub-slice 64 indices at a time; lanes holding the same
//     expert find each other with one ballot per expert-id bit, their rank among
//     those peers is a popcount of lower lanes, and the last peer advances the
//     wave's counter.  No atomics and two workgroup barriers in total.
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
  int n_logical, n_ranks, G, D, C, L, P, n_blocks, id_bits;
  int64_t *out;
};

// Mask of the lanes whose (valid) key equals this lane's key.
__device__ inline uint64_t match_any(int key, bool valid, int bits) {
  uint64_t peers = __ballot(valid);
  for (int b = 0; b < bits; ++b) {
    const bool bit = (key >> b) & 1;
    const uint64_t m = __ballot(bit);
    peers &= bit ? m : ~m;
  }
  return peers;
}

__global__ __launch_bounds__(1024) void redirect_indices(MapArgs a) {
  extern __shared__ int32_t smem[];
  const int nl = a.n_logical;
  int32_t *total = smem;
  int32_t *expected = total + nl;
  int32_t *log2r = expected + nl;    // [nl][2]: original slot, replica slot
  int32_t *base = log2r + 2 * nl;    // [n_waves][nl]
  const int tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid % kWave, wave = tid / kWave, n_waves = nt / kWave;
  const int pid = blockIdx.x;
  const int32_t *last = a.by_block + (int64_t)(a.n_blocks - 1) * nl;
  const int32_t *prev = pid ? a.by_block + (int64_t)(pid - 1) * nl : nullptr;

  // Tables, minilp.cu:466-496.
  for (int e = tid; e < nl; e += nt) {
    total[e] = expected[e] = last[e];
    log2r[2 * e] = -1;
    log2r[2 * e + 1] = -1;
    for (int w = 0; w < n_waves; ++w)
      base[w * nl + e] = 0;
  }
  __syncthreads();
  for (int e = tid; e < nl; e += nt) {
    const int slot = (e / a.L) * a.P + (e % a.L);
    const int le = a.phy2log[slot];
    if (le >= 0 && le < nl)
      log2r[2 * le] = slot;
  }
  const int cd = a.C * a.D;
  for (int i = tid; i < a.n_ranks * cd; i += nt) {
    const int ep_rank = i / cd, local = i % cd, d = local % a.D;
    const int le = a.phy2log[ep_rank * a.P + local];
    if (le >= 0 && le < nl) {
      // fp32 product truncated toward zero (saturating, NaN -> 0)
      expected[le] = __float2int_rz(a.o_weight[ep_rank * a.D + d] * (float)last[le]);
      const int group = ep_rank / a.G, group_rank = ep_rank % a.G;
      log2r[2 * le + 1] = (group * a.G + a.o2r[group_rank * a.D + d] + 1) * a.P - cd + local;
    }
  }

  // Sub-slice of this wave: whole 64-index chunks.
  const int64_t begin = slice_begin(a.n, a.per, pid);
  const int64_t end = slice_begin(a.n, a.per, pid + 1);
  const int64_t chunks = (end - begin + kWave - 1) / kWave;
  const int64_t chunks_per_wave = (chunks + n_waves - 1) / n_waves;
  int64_t wbeg = begin + wave * chunks_per_wave * kWave;
  if (wbeg > end)
    wbeg = end;
  int64_t wend = wbeg + chunks_per_wave * kWave;
  if (wend > end)
    wend = end;
  int32_t *mine = base + wave * nl;

  // Phase A (base rows were zeroed before the first barrier).
  for (int64_t i = wbeg + lane; i < wend; i += kWave) {
    const int64_t v = a.idx[i];
    if (v >= 0 && v < nl)
      atomicAdd(&mine[v], 1);
  }
  __syncthreads();
  // Phase B.
  for (int e = tid; e < nl; e += nt) {
    int32_t run = prev ? prev[e] : 0;
    for (int w = 0; w < n_waves; ++w) {
      const int32_t t = base[w * nl + e];
      base[w * nl + e] = run;
      run += t;
    }
  }
  __syncthreads();
  // Phase C.
  for (int64_t pos = wbeg; pos < wend; pos += kWave) {
    const int64_t i = pos + lane;
    const bool in = i < wend;
    const int64_t v = in ? a.idx[i] : -1;
    const bool valid = v >= 0 && v < nl;
    const int e = valid ? (int)v : 0;
    const uint64_t peers = match_any(e, valid, a.id_bits);
    int64_t o = -1;
    if (valid) {
      const int rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(peers >> 32),
                                                 __builtin_amdgcn_mbcnt_lo((uint32_t)peers, 0u));
      const int cnt = __popcll(peers);
      const int32_t k = mine[e] + rank;
      // (k * 499 + 41) % total in int32 arithmetic (minilp.cu:505)
      int32_t h = (int32_t)((uint32_t)k * 499u + 41u);
      const int32_t t = total[e];
      h = t > 0 ? h % t : 0;
      o = log2r[2 * e + (h >= expected[e] ? 1 : 0)];
      if (rank == cnt - 1)
        mine[e] = k + 1;
    }
    if (in)
      a.out[i] = o;
    __builtin_amdgcn_wave_barrier();
  }
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
  a.id_bits = 0;
  while ((1 << a.id_bits) < a.n_logical)
    ++a.id_bits;

  // One wave per 64-index chunk of the slice, up to 16 waves, as LDS allows.
  int n_waves = (int)((a.per + kWave - 1) / kWave);
  if (n_waves > 16)
    n_waves = 16;
  auto lds_bytes = [&](int w) { return sizeof(int32_t) * (size_t)a.n_logical * (4 + w); };
  while (n_waves > 1 && lds_bytes(n_waves) > 64 * 1024)
    n_waves >>= 1;
  LPLB_REQUIRE(lds_bytes(n_waves) <= 64 * 1024, LPLB_EUNSUPPORTED,
               "map_idx: %d logical experts do not fit the LDS tables", a.n_logical);
  hipLaunchKernelGGL(redirect_indices, dim3(n_blocks), dim3(n_waves * kWave), lds_bytes(n_waves),
                     static_cast<hipStream_t>(stream), a);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}
