// Per-expert token histogram with an inclusive prefix over slices.
//
// Two launches on the caller's stream:
//   1. slice_histogram: one workgroup per slice, LDS histogram (eight copies, chosen by lane)
//      fed by coalesced 16-byte index loads, row p of the output = counts of slice p;
//   2. prefix_over_slices: turns the rows into running sums down the slice axis,
//      16 experts per workgroup and 16 row bands per expert, instead of the serial
//      walk over all slices the reference does after its grid barrier
//      (minilp.cu:439-442).
// (Doing the scan inside the first kernel, by the last workgroup to finish, was
// measured and rejected: one CU sustains too few outstanding misses to pull the
// 256 KB table, 20 us against 3 us for this kernel.)
// HBM-bound: 8 bytes read per index; the [n_blocks, n_experts] table is small.
// Callers that need only the totals of a short batch get them in one launch: slice_histogram with
// TOTALS (slices add their counts to one vector) or expert_totals (every workgroup owns four experts).
#include "common.h"

namespace lplb {

constexpr int kLoadsInFlight = 4;   // 16-byte loads a thread issues before it consumes them

// COPIES histograms side by side, lane l counts into copy l % COPIES: lanes of one instruction that
// hold the same expert are served one after the other by the LDS, and at Zipf(1.0) the hottest expert
// has ten of a wave's 64 tokens.  The copies start 4 banks apart (a stride of 4 modulo the 32 banks),
// so that the counters of one expert sit in eight different banks.  (Measured at [262144 x 8] in 256
// slices, kernel alone: one copy 5.3 us, two 5.1, four 4.9, eight 4.8, eight in different banks 4.6;
// a copy per wave instead of per lane: no gain.)
constexpr int kHistogramCopies = 8;
__host__ __device__ constexpr int histogram_stride(int n_experts, int copies) {
  return copies > 1 ? ((n_experts + 31) & ~31) + 4 : n_experts;
}

// TOTALS: instead of writing its row, a slice adds its counts to the one vector `counts` [n_experts]
// (device-wide atomic adds, none for an expert the slice has no token of), and the launch sets the
// vector `clear` (if given) to zero -- a caller that takes two vectors in turn never has to zero one.
template <int COPIES, bool TOTALS>
__global__ __launch_bounds__(1024) void slice_histogram(
    const int64_t *__restrict__ idx, int64_t n, int n_experts, int64_t per,
    int32_t *__restrict__ counts, int32_t *__restrict__ clear) {
  extern __shared__ int32_t hist[];
  fetch_arguments_now(idx, n, n_experts, per, counts, clear);
  const int tid = threadIdx.x, nt = blockDim.x;
  const int p = blockIdx.x;
  const int stride = histogram_stride(n_experts, COPIES);
  int32_t *mine = hist + (tid % COPIES) * stride;
  auto count = [&](int64_t v) {
    if ((uint64_t)v < (uint64_t)n_experts)
      atomicAdd(&mine[(int)v], 1);
  };
  const int64_t begin = slice_begin(n, per, p);
  const int64_t end = slice_begin(n, per, p + 1);
  // Pairs are loaded 16 bytes at a time.  Slices start on multiples of 256 indices,
  // so a slice starts on a 16-byte boundary unless the array itself sits at an odd
  // multiple of 8 bytes (a view that starts inside a tensor); then its first index
  // is counted alone.
  const int64_t head = (begin < end && (reinterpret_cast<uintptr_t>(idx + begin) & 8)) ? 1 : 0;
  const int64_t n_pairs = (end - begin - head) >> 1;
  typedef long long i64x2 __attribute__((ext_vector_type(2)));
  const i64x2 *pairs = reinterpret_cast<const i64x2 *>(idx + begin + head);
  // the first batch of loads is on its way while the histogram is cleared
  i64x2 first[kLoadsInFlight];
#pragma unroll
  for (int u = 0; u < kLoadsInFlight; ++u) {
    const int64_t i = tid + (int64_t)u * nt;
    first[u] = i < n_pairs ? __builtin_nontemporal_load(pairs + i) : i64x2{-1, -1};
  }
  for (int e = tid; e < COPIES * stride; e += nt)
    hist[e] = 0;
  if constexpr (TOTALS)
    if (clear)
      for (int64_t e = (int64_t)p * nt + tid; e < n_experts; e += (int64_t)gridDim.x * nt)
        clear[e] = 0;
  __syncthreads();
#pragma unroll
  for (int u = 0; u < kLoadsInFlight; ++u) {
    count(first[u].x);
    count(first[u].y);
  }
  for (int64_t i0 = tid + (int64_t)nt * kLoadsInFlight; i0 < n_pairs; i0 += (int64_t)nt * kLoadsInFlight) {
    i64x2 v[kLoadsInFlight];
#pragma unroll
    for (int u = 0; u < kLoadsInFlight; ++u) {
      const int64_t i = i0 + (int64_t)u * nt;
      v[u] = i < n_pairs ? __builtin_nontemporal_load(pairs + i) : i64x2{-1, -1};
    }
#pragma unroll
    for (int u = 0; u < kLoadsInFlight; ++u) {
      count(v[u].x);
      count(v[u].y);
    }
  }
  if (tid == 0 && head)
    count(idx[begin]);
  if (tid == 0 && ((end - begin - head) & 1))
    count(idx[end - 1]);
  __syncthreads();
  int32_t *row = TOTALS ? counts : counts + (int64_t)p * n_experts;
  if constexpr (!TOTALS) {
    for (int e = tid; e < n_experts; e += nt) {
      int32_t sum = 0;
#pragma unroll
      for (int k = 0; k < COPIES; ++k)
        sum += hist[k * stride + e];
      row[e] = sum;
    }
  } else {
    // Two counters per atomic add: updates of one 64-byte line of memory are served one after the other
    // (about 14 ns each), and every slice updates every line, so the number of updates is what this
    // costs.  A counter stays below 2^31, so the low half never carries into the high one.
    unsigned long long *both = reinterpret_cast<unsigned long long *>(row);
    for (int e2 = tid; 2 * e2 < n_experts; e2 += nt) {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int k = 0; k < COPIES; ++k) {
        lo += (uint32_t)hist[k * stride + 2 * e2];
        hi += 2 * e2 + 1 < n_experts ? (uint32_t)hist[k * stride + 2 * e2 + 1] : 0u;
      }
      if (2 * e2 + 1 < n_experts) {
        if ((lo | hi) != 0)
          __hip_atomic_fetch_add(both + e2, ((unsigned long long)hi << 32) | lo, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
      } else if (lo != 0) {
        __hip_atomic_fetch_add(row + 2 * e2, (int32_t)lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

// The launch all callers share: eight copies while they fit the 64 KiB of LDS a kernel gets unasked
// (up to 2016 experts), else one.  TOTALS as in the kernel.
template <bool TOTALS>
static int launch_slice_histogram(const int64_t *idx, int64_t n_elements, int n_experts, int n_blocks, int32_t *counts,
                                  int32_t *clear, hipStream_t s, unsigned flags) {
  const size_t one = sizeof(int32_t) * (size_t)n_experts;
  LPLB_REQUIRE(one <= 64 * 1024, LPLB_EUNSUPPORTED, "n_experts=%d does not fit the LDS histogram", n_experts);
  const int64_t per = slice_len(n_elements, n_blocks);
  // one 16-byte load per thread covers 2 indices; a thread has kLoadsInFlight of them under
  // way, so a slice gets as many threads as cover it in one such batch, up to 1024
  const int64_t batches = (per / 2 + kLoadsInFlight - 1) / kLoadsInFlight;
  const int threads = batches <= 256 ? 256 : batches <= 512 ? 512 : 1024;
  const size_t copies = sizeof(int32_t) * (size_t)kHistogramCopies * histogram_stride(n_experts, kHistogramCopies);
  if (copies <= 64 * 1024)
    launch_with_flags(slice_histogram<kHistogramCopies, TOTALS>, dim3(n_blocks), dim3(threads), copies, s, flags, idx,
                      n_elements, n_experts, per, counts, clear);
  else
    launch_with_flags(slice_histogram<1, TOTALS>, dim3(n_blocks), dim3(threads), one, s, flags, idx, n_elements,
                      n_experts, per, counts, clear);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}

constexpr int kScanBands = 16;      // bands of rows, one per group of kScanCols lanes
constexpr int kScanRows = 16;       // rows of a band a thread keeps in registers
constexpr int kScanCols = 16;       // experts per workgroup: many small workgroups pull the
                                    // table through many CUs (one CU sustains few misses)

// counts[p][e] <- sum_{p' <= p} counts[p'][e].  A workgroup owns kScanCols experts;
// thread = (band of rows, expert).  All loads of a band are in flight at once
// (clamped addresses, masked values); band sums meet in LDS; tables with more than
// 256 slices take several sweeps with a running carry.
__global__ __launch_bounds__(kScanBands *kScanCols) void prefix_over_slices(
    int32_t *__restrict__ counts, int n_blocks, int n_experts) {
  __shared__ int32_t part[kScanBands][kScanCols];
  __shared__ int32_t carry[kScanCols];
  fetch_arguments_now(counts, n_blocks, n_experts);
  const int col = threadIdx.x % kScanCols, band = threadIdx.x / kScanCols;
  const int e = blockIdx.x * kScanCols + col;
  const bool live = e < n_experts;
  int32_t *column = counts + (live ? e : 0);
  if (band == 0)
    carry[col] = 0;
  __syncthreads();
  for (int row0 = 0; row0 < n_blocks; row0 += kScanBands * kScanRows) {
    const int r0 = row0 + band * kScanRows;
    int32_t v[kScanRows];
#pragma unroll
    for (int k = 0; k < kScanRows; ++k)
      v[k] = column[(int64_t)min(r0 + k, n_blocks - 1) * n_experts];
#pragma unroll
    for (int k = 0; k < kScanRows; ++k)
      v[k] = (live && r0 + k < n_blocks) ? v[k] : 0;
#pragma unroll
    for (int k = 1; k < kScanRows; ++k)
      v[k] += v[k - 1];
    part[band][col] = v[kScanRows - 1];
    __syncthreads();
    int32_t offset = carry[col];
#pragma unroll
    for (int b = 0; b < kScanBands; ++b)
      offset += b < band ? part[b][col] : 0;
#pragma unroll
    for (int k = 0; k < kScanRows; ++k)
      if (live && r0 + k < n_blocks)
        column[(int64_t)(r0 + k) * n_experts] = v[k] + offset;
    __syncthreads();
    if (band == kScanBands - 1)
      carry[col] = offset + v[kScanRows - 1];
    __syncthreads();
  }
}

// ---- totals only, for short batches: one launch, nothing shared between workgroups ----
// A workgroup owns kOwned experts and reads the whole batch; what it counts is final, so there is no
// second kernel, no atomic between workgroups and nothing to clear.  Every workgroup pulls all n indices
// through its CU (64 bytes per clock), which bounds the batch this pays for: 65536 indices take about as
// long as the launch itself, against two launches for histogram and scan.  A lane keeps four counters;
// the values of a batch of loads are first added up in one register, a byte per owned expert.
constexpr int kOwned = 4;
constexpr int64_t kTotalsMaxIndices = LPLB_COUNT_TOTALS_MAX_INDICES;   // per call; beyond, the two-kernel form is faster
constexpr int kTotalsMaxExperts = LPLB_COUNT_TOTALS_MAX_EXPERTS;

__global__ __launch_bounds__(1024) void expert_totals(const int64_t *__restrict__ idx, int64_t n, int n_experts,
                                                      int32_t *__restrict__ totals) {
  __shared__ int32_t per_wave[16][kOwned];
  fetch_arguments_now(idx, n, n_experts, totals);
  typedef long long i64x2 __attribute__((ext_vector_type(2)));
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t base = (int64_t)blockIdx.x * kOwned;
  // one byte per owned expert: 1 << (8 * (v - base)) for a value this workgroup owns, else 0
  auto key = [&](int64_t v) -> uint32_t {
    const uint64_t rel = (uint64_t)(v - base);
    return rel < (uint64_t)kOwned && v < n_experts ? 1u << (8 * (uint32_t)rel) : 0u;
  };
  const int64_t head = (n > 0 && (reinterpret_cast<uintptr_t>(idx) & 8)) ? 1 : 0;   // (see slice_histogram)
  const int64_t n_pairs = (n - head) >> 1;
  const i64x2 *pairs = reinterpret_cast<const i64x2 *>(idx + head);
  uint32_t mine[kOwned] = {};
  for (int64_t i0 = tid; i0 < n_pairs; i0 += (int64_t)nt * kLoadsInFlight) {
    i64x2 v[kLoadsInFlight];
#pragma unroll
    for (int u = 0; u < kLoadsInFlight; ++u) {
      const int64_t i = i0 + (int64_t)u * nt;
      v[u] = i < n_pairs ? pairs[i] : i64x2{-1, -1};
    }
    uint32_t packed = 0;   // at most 2 * kLoadsInFlight per byte
#pragma unroll
    for (int u = 0; u < kLoadsInFlight; ++u)
      packed += key(v[u].x) + key(v[u].y);
#pragma unroll
    for (int k = 0; k < kOwned; ++k)
      mine[k] += (packed >> (8 * k)) & 0xffu;
  }
  if (tid == 0) {
    uint32_t packed = head ? key(idx[0]) : 0u;
    if ((n - head) & 1)
      packed += key(idx[n - 1]);
#pragma unroll
    for (int k = 0; k < kOwned; ++k)
      mine[k] += (packed >> (8 * k)) & 0xffu;
  }
  // butterfly over the wave, the four counters side by side
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    uint32_t other[kOwned];
#pragma unroll
    for (int k = 0; k < kOwned; ++k)
      other[k] = bpermute(mine[k], lane_id() ^ off);
#pragma unroll
    for (int k = 0; k < kOwned; ++k)
      mine[k] += other[k];
  }
  if (tid % kWave == 0)
#pragma unroll
    for (int k = 0; k < kOwned; ++k)
      per_wave[tid / kWave][k] = (int32_t)mine[k];
  __syncthreads();
  if (tid < kOwned && base + tid < n_experts) {
    int32_t sum = 0;
    for (int w = 0; w < nt / kWave; ++w)
      sum += per_wave[w][tid];
    totals[base + tid] = sum;
  }
}

// Enqueues histogram and prefix.  any_order: the histogram launch does not wait for
// the kernel enqueued just before it on the stream (it still starts after everything
// that kernel waited for); the prefix launch is ordered after both.
int enqueue_count(const int64_t *idx, int64_t n_elements, int n_experts, int n_blocks,
                  int32_t *counts_by_block, hipStream_t s, bool any_order) {
  const int rc = launch_slice_histogram<false>(idx, n_elements, n_experts, n_blocks, counts_by_block, nullptr, s,
                                               any_order ? hipExtAnyOrderLaunch : 0u);
  if (rc != LPLB_OK)
    return rc;
  launch(prefix_over_slices, dim3((n_experts + kScanCols - 1) / kScanCols), dim3(kScanBands * kScanCols), 0, s,
         counts_by_block, n_blocks, n_experts);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
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
  LPLB_REQUIRE((reinterpret_cast<uintptr_t>(idx) & 7) == 0, LPLB_EINVAL,
               "count_idx: idx must be 8-byte aligned");
  return enqueue_count(idx, n_elements, n_experts, n_blocks, counts_by_block,
                       static_cast<hipStream_t>(stream), /*any_order=*/false);
}

extern "C" int lplb_count_totals(const int64_t *idx, int64_t n_elements, int n_experts, int32_t *totals,
                                 lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(n_elements >= 0 && n_experts > 0, LPLB_EINVAL, "count_totals: n_elements=%lld n_experts=%d",
               (long long)n_elements, n_experts);
  LPLB_REQUIRE(totals != nullptr && (idx != nullptr || n_elements == 0), LPLB_EINVAL, "count_totals: null pointer");
  LPLB_REQUIRE((reinterpret_cast<uintptr_t>(idx) & 7) == 0, LPLB_EINVAL, "count_totals: idx must be 8-byte aligned");
  LPLB_REQUIRE(n_elements <= kTotalsMaxIndices && n_experts <= kTotalsMaxExperts, LPLB_EUNSUPPORTED,
               "count_totals: serves up to %lld indices and %d experts (use lplb_count_idx beyond)",
               (long long)kTotalsMaxIndices, kTotalsMaxExperts);
  launch(expert_totals, dim3((n_experts + kOwned - 1) / kOwned), dim3(1024), 0, static_cast<hipStream_t>(stream), idx,
         n_elements, n_experts, totals);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}

extern "C" int lplb_count_totals_add(const int64_t *idx, int64_t n_elements, int n_experts, int32_t *totals,
                                     int32_t *clear, lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(n_elements >= 0 && n_elements <= INT32_MAX && n_experts > 0, LPLB_EINVAL,
               "count_totals_add: n_elements=%lld n_experts=%d", (long long)n_elements, n_experts);
  LPLB_REQUIRE(totals != nullptr && (idx != nullptr || n_elements == 0), LPLB_EINVAL, "count_totals_add: null pointer");
  LPLB_REQUIRE(totals != clear, LPLB_EINVAL, "count_totals_add: totals and clear are the same vector");
  LPLB_REQUIRE(((reinterpret_cast<uintptr_t>(idx) | reinterpret_cast<uintptr_t>(totals)) & 7) == 0, LPLB_EINVAL,
               "count_totals_add: idx and totals must be 8-byte aligned");
  LPLB_REQUIRE(n_elements <= kTotalsMaxIndices, LPLB_EUNSUPPORTED,
               "count_totals_add: serves up to %lld indices (use lplb_count_idx beyond)", (long long)kTotalsMaxIndices);
  // Slices of 8192 indices (1024 threads with four 16-byte loads each): at most 16 of them, because every
  // slice updates every line of the totals and those updates queue up.
  const int64_t wanted = (n_elements + 8191) / 8192;
  const int n_blocks = (int)(wanted < 1 ? 1 : wanted);
  return launch_slice_histogram<true>(idx, n_elements, n_experts, n_blocks, totals, clear,
                                      static_cast<hipStream_t>(stream), 0u);
}

// Measurement aid: the histogram kernel alone (no scan behind it), n_launches times, launch r on idx[r] and
// counts_by_block[r], each recording its own begin and end into start_events[r] / stop_events[r].
extern "C" int lplb_slice_histogram_series(const int64_t *const *idx, int64_t n_elements, int n_experts, int n_blocks,
                                           int32_t *const *counts_by_block, int n_launches, void *const *start_events,
                                           void *const *stop_events, lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(idx && counts_by_block && n_launches >= 0, LPLB_EINVAL, "slice_histogram_series: null pointer or negative count");
  LPLB_REQUIRE(n_elements > 0 && n_elements <= INT32_MAX && n_experts > 0 && n_blocks > 0 &&
                   sizeof(int32_t) * (size_t)n_experts <= 64 * 1024,
               LPLB_EINVAL, "slice_histogram_series: n_elements=%lld n_experts=%d n_blocks=%d", (long long)n_elements,
               n_experts, n_blocks);
  for (int r = 0; r < n_launches; ++r) {
    LPLB_REQUIRE(idx[r] && counts_by_block[r] && (reinterpret_cast<uintptr_t>(idx[r]) & 7) == 0, LPLB_EINVAL,
                 "slice_histogram_series: bad pointer in launch %d", r);
    lplb_time_next_launch(start_events ? start_events[r] : nullptr, stop_events ? stop_events[r] : nullptr);
    const int rc = launch_slice_histogram<false>(idx[r], n_elements, n_experts, n_blocks, counts_by_block[r], nullptr,
                                                 static_cast<hipStream_t>(stream), 0u);
    if (rc != LPLB_OK) {
      lplb_time_next_launch(nullptr, nullptr);
      return rc;
    }
  }
  return LPLB_OK;
}
