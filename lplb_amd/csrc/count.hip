// Per-expert token histogram with an inclusive prefix over slices.
//
// Two launches on the caller's stream:
//   1. slice_histogram: one workgroup per slice, LDS histogram fed by coalesced
//      16-byte index loads, row p of the output = counts of slice p;
//   2. prefix_over_slices: turns the rows into running sums down the slice
//      axis.  A workgroup owns 64 experts (one per lane) and splits the slice
//      axis over its waves, so the scan costs two short passes instead of the
//      serial walk over all slices the reference does after its grid barrier
//      (minilp.cu:439-442).
// HBM-bound: 8 bytes read per index; the [n_blocks, n_experts] table is small.
#include "common.h"

namespace lplb {

constexpr int kCountThreads = 256;

__global__ __launch_bounds__(kCountThreads) void slice_histogram(
    const int64_t *__restrict__ idx, int64_t n, int n_experts, int64_t per,
    int32_t *__restrict__ counts) {
  extern __shared__ int32_t hist[];
  const int tid = threadIdx.x;
  const int p = blockIdx.x;
  for (int e = tid; e < n_experts; e += kCountThreads)
    hist[e] = 0;
  __syncthreads();

  const int64_t begin = slice_begin(n, per, p);
  const int64_t end = slice_begin(n, per, p + 1);
  // Slices start on multiples of 256 indices, so pairs are 16-byte aligned.
  const int64_t n_pairs = (end - begin) >> 1;
  const longlong2 *pairs = reinterpret_cast<const longlong2 *>(idx + begin);
  for (int64_t i = tid; i < n_pairs; i += kCountThreads) {
    longlong2 v = pairs[i];
    if (v.x >= 0 && v.x < n_experts)
      atomicAdd(&hist[v.x], 1);
    if (v.y >= 0 && v.y < n_experts)
      atomicAdd(&hist[v.y], 1);
  }
  if (tid == 0 && ((end - begin) & 1)) {
    int64_t v = idx[end - 1];
    if (v >= 0 && v < n_experts)
      atomicAdd(&hist[v], 1);
  }
  __syncthreads();
  int32_t *row = counts + (int64_t)p * n_experts;
  for (int e = tid; e < n_experts; e += kCountThreads)
    row[e] = hist[e];
}

constexpr int kScanWaves = 16;

// counts[p][e] <- sum_{p' <= p} counts[p'][e].
__global__ __launch_bounds__(kScanWaves *kWave) void prefix_over_slices(
    int32_t *__restrict__ counts, int n_blocks, int n_experts) {
  __shared__ int32_t part[kScanWaves][kWave];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int e = blockIdx.x * kWave + lane;
  const int rows_per_wave = (n_blocks + kScanWaves - 1) / kScanWaves;
  const int r0 = min(n_blocks, wave * rows_per_wave);
  const int r1 = min(n_blocks, r0 + rows_per_wave);
  int32_t sum = 0;
  if (e < n_experts)
    for (int r = r0; r < r1; ++r)
      sum += counts[(int64_t)r * n_experts + e];
  part[wave][lane] = sum;
  __syncthreads();
  int32_t run = 0;
  for (int w = 0; w < wave; ++w)
    run += part[w][lane];
  if (e < n_experts)
    for (int r = r0; r < r1; ++r) {
      run += counts[(int64_t)r * n_experts + e];
      counts[(int64_t)r * n_experts + e] = run;
    }
}

} // namespace lplb

extern "C" int lplb_count_idx(const int64_t *idx, int64_t n_elements,
                              int n_experts, int n_blocks,
                              int32_t *counts_by_block, lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(n_elements >= 0 && n_elements <= INT32_MAX, LPLB_EINVAL,
               "count_idx: n_elements=%lld out of range", (long long)n_elements);
  LPLB_REQUIRE(n_experts > 0 && n_blocks > 0, LPLB_EINVAL,
               "count_idx: n_experts=%d n_blocks=%d must be positive", n_experts, n_blocks);
  LPLB_REQUIRE(counts_by_block != nullptr && (idx != nullptr || n_elements == 0), LPLB_EINVAL,
               "count_idx: null pointer");
  LPLB_REQUIRE((reinterpret_cast<uintptr_t>(idx) & 15) == 0, LPLB_EINVAL,
               "count_idx: idx must be 16-byte aligned");
  const size_t lds = sizeof(int32_t) * (size_t)n_experts;
  LPLB_REQUIRE(lds <= 160 * 1024, LPLB_EUNSUPPORTED,
               "count_idx: n_experts=%d does not fit the LDS histogram", n_experts);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t per = slice_len(n_elements, n_blocks);
  hipLaunchKernelGGL(slice_histogram, dim3(n_blocks), dim3(kCountThreads), lds, s, idx,
                     n_elements, n_experts, per, counts_by_block);
  LPLB_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(prefix_over_slices, dim3((n_experts + kWave - 1) / kWave),
                     dim3(kScanWaves * kWave), 0, s, counts_by_block, n_blocks, n_experts);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}
