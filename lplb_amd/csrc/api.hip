// Error reporting and version query of the C ABI.
#include <atomic>
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace lplb {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

// Plain streaming copy: the yardstick the redirect's bandwidth and the profiler's byte counters
// are compared with, in the fastest shape found for 16 MiB in + 16 MiB out on this GPU: eight
// 16-byte loads per lane, 512 threads per workgroup -- one workgroup of eight waves per CU covers
// the array in one trip -- and a workgroup barrier between the loads and the stores.  Measured
// (kernel's own begin/end, 16 buffer pairs in turn, lplb_copy_shape_series below): 5.7 us; four
// loads per lane and 1024 threads (also one workgroup per CU) 5.9 us; two loads and 1024 threads
// (two workgroups per CU) 6.7 us; one load per lane 6.6-6.8 us in any workgroup size; eight loads
// and 1024 threads without the barrier 7.9 us (reads and writes of a workgroup mix in time), with
// it 6.4 us.
typedef long long i64x2 __attribute__((ext_vector_type(2)));
constexpr int kCopyThreads = 512, kCopyLoads = 8;
// WHOLE: the grid covers the array exactly, one tile per workgroup (no loop, no bounds).
template <bool WHOLE>
__global__ __launch_bounds__(kCopyThreads) void copy_calibration(const i64x2 *__restrict__ src,
                                                                    i64x2 *__restrict__ dst, int64_t n_pairs) {
  constexpr int64_t tile = (int64_t)kCopyThreads * kCopyLoads;
  if constexpr (WHOLE) {
    const int64_t t0 = (int64_t)blockIdx.x * tile + threadIdx.x;
    i64x2 v[kCopyLoads];
#pragma unroll
    for (int u = 0; u < kCopyLoads; ++u)
      v[u] = __builtin_nontemporal_load(src + t0 + u * kCopyThreads);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kCopyLoads; ++u)
      __builtin_nontemporal_store(v[u], dst + t0 + u * kCopyThreads);
    return;
  }
  for (int64_t t0 = (int64_t)blockIdx.x * tile; t0 < n_pairs; t0 += (int64_t)gridDim.x * tile) {
    i64x2 v[kCopyLoads];
#pragma unroll
    for (int u = 0; u < kCopyLoads; ++u) {
      const int64_t i = t0 + u * kCopyThreads + threadIdx.x;
      v[u] = i < n_pairs ? __builtin_nontemporal_load(src + i) : i64x2{0, 0};
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kCopyLoads; ++u) {
      const int64_t i = t0 + u * kCopyThreads + threadIdx.x;
      if (i < n_pairs)
        __builtin_nontemporal_store(v[u], dst + i);
    }
  }
}

#ifdef LPLB_PHASE_CLOCKS
long long *g_phase_clocks = nullptr;
#endif

static thread_local LaunchEvents g_launch_events;

int current_device_cu_count() {
  static std::atomic<int> cus_of[64];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    return 0;
  int n = cus_of[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      return 0;
    cus_of[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

LaunchEvents take_launch_events() {
  const LaunchEvents ev = g_launch_events;
  g_launch_events = LaunchEvents{};
  return ev;
}

} // namespace lplb

extern "C" void lplb_time_next_launch(void *start_event, void *stop_event) {
  lplb::g_launch_events.start = static_cast<hipEvent_t>(start_event);
  lplb::g_launch_events.stop = static_cast<hipEvent_t>(stop_event);
}

#ifdef LPLB_PHASE_CLOCKS
// Debug builds only: device buffer of int64 that receives the stamps.
extern "C" void lplb_debug_set_phase_clocks(long long *device_buffer) {
  lplb::g_phase_clocks = device_buffer;
}
#endif

extern "C" const char *lplb_last_error(void) { return lplb::g_last_error; }

extern "C" int lplb_abi_version(void) { return LPLB_ABI_VERSION; }

extern "C" int lplb_copy_calibration(const int64_t *src, int64_t *dst, int64_t n_elements,
                                     lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(src && dst && n_elements > 0 && n_elements % 2 == 0, LPLB_EINVAL,
               "copy_calibration: need an even, positive element count and non-null pointers");
  LPLB_REQUIRE(((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0, LPLB_EINVAL,
               "copy_calibration: src and dst must be 16-byte aligned");
  const int64_t n_pairs = n_elements / 2, tile = (int64_t)kCopyThreads * kCopyLoads;
  const int n_cus = current_device_cu_count();
  const int64_t resident = 4 * (int64_t)(n_cus > 0 ? n_cus : 256);   // workgroups the GPU holds at once (8 waves each)
  const int64_t tiles = (n_pairs + tile - 1) / tile;
  if (n_pairs % tile == 0 && tiles <= resident)
    launch(copy_calibration<true>, dim3((unsigned)tiles), dim3(kCopyThreads), 0, static_cast<hipStream_t>(stream),
           reinterpret_cast<const i64x2 *>(src), reinterpret_cast<i64x2 *>(dst), n_pairs);
  else
    launch(copy_calibration<false>, dim3((unsigned)(tiles < resident ? tiles : resident)), dim3(kCopyThreads), 0,
           static_cast<hipStream_t>(stream), reinterpret_cast<const i64x2 *>(src), reinterpret_cast<i64x2 *>(dst), n_pairs);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}

namespace lplb {
// The same copy in other shapes, for the comparison behind the choice above: LOADS 16-byte loads per
// lane, any workgroup size, with or without the barrier between loads and stores, cached or streaming
// accesses.  Whole tiles only.
template <int LOADS, bool BARRIER, bool STREAMING>
__global__ __launch_bounds__(1024) void copy_shape(const i64x2 *__restrict__ src, i64x2 *__restrict__ dst) {
  const int64_t t0 = (int64_t)blockIdx.x * blockDim.x * LOADS + threadIdx.x;
  i64x2 v[LOADS];
#pragma unroll
  for (int u = 0; u < LOADS; ++u)
    v[u] = STREAMING ? __builtin_nontemporal_load(src + t0 + u * blockDim.x) : src[t0 + u * blockDim.x];
  if constexpr (BARRIER)
    __syncthreads();
#pragma unroll
  for (int u = 0; u < LOADS; ++u) {
    if constexpr (STREAMING)
      __builtin_nontemporal_store(v[u], dst + t0 + u * blockDim.x);
    else
      dst[t0 + u * blockDim.x] = v[u];
  }
}
template <int LOADS> static void launch_copy_shape(int barrier, int streaming, dim3 grid, dim3 block, hipStream_t s,
                                                   const i64x2 *src, i64x2 *dst) {
  if (barrier && streaming) launch(copy_shape<LOADS, true, true>, grid, block, 0, s, src, dst);
  else if (barrier) launch(copy_shape<LOADS, true, false>, grid, block, 0, s, src, dst);
  else if (streaming) launch(copy_shape<LOADS, false, true>, grid, block, 0, s, src, dst);
  else launch(copy_shape<LOADS, false, false>, grid, block, 0, s, src, dst);
}
} // namespace lplb

extern "C" int lplb_copy_shape_series(const int64_t *const *src, int64_t *const *dst, int64_t n_elements,
                                      int n_launches, int loads_per_lane, int threads, int barrier, int streaming,
                                      void *const *start_events, void *const *stop_events, lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(src && dst && n_launches >= 0, LPLB_EINVAL, "copy_shape_series: null pointer or negative count");
  LPLB_REQUIRE((loads_per_lane == 1 || loads_per_lane == 2 || loads_per_lane == 4 || loads_per_lane == 8) &&
                   (threads == 256 || threads == 512 || threads == 1024),
               LPLB_EINVAL, "copy_shape_series: loads_per_lane in {1, 2, 4, 8}, threads in {256, 512, 1024}");
  const int64_t tile = (int64_t)threads * loads_per_lane * 2;
  LPLB_REQUIRE(n_elements > 0 && n_elements % tile == 0, LPLB_EINVAL,
               "copy_shape_series: n_elements must be a multiple of %lld", (long long)tile);
  const dim3 grid((unsigned)(n_elements / tile)), block(threads);
  for (int r = 0; r < n_launches; ++r) {
    LPLB_REQUIRE(((reinterpret_cast<uintptr_t>(src[r]) | reinterpret_cast<uintptr_t>(dst[r])) & 15) == 0, LPLB_EINVAL,
                 "copy_shape_series: src and dst must be 16-byte aligned");
    lplb_time_next_launch(start_events ? start_events[r] : nullptr, stop_events ? stop_events[r] : nullptr);
    const i64x2 *in = reinterpret_cast<const i64x2 *>(src[r]);
    i64x2 *out = reinterpret_cast<i64x2 *>(dst[r]);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (loads_per_lane) {
    case 1: launch_copy_shape<1>(barrier, streaming, grid, block, s, in, out); break;
    case 2: launch_copy_shape<2>(barrier, streaming, grid, block, s, in, out); break;
    case 4: launch_copy_shape<4>(barrier, streaming, grid, block, s, in, out); break;
    default: launch_copy_shape<8>(barrier, streaming, grid, block, s, in, out); break;
    }
    LPLB_HIP_TRY(hipGetLastError());
  }
  return LPLB_OK;
}

extern "C" int lplb_copy_calibration_series(const int64_t *const *src, int64_t *const *dst, int64_t n_elements,
                                            int n_launches, void *const *start_events, void *const *stop_events,
                                            lplb_stream_t stream) {
  LPLB_REQUIRE(src && dst && n_launches >= 0, LPLB_EINVAL, "copy_calibration_series: null pointer or negative count");
  for (int r = 0; r < n_launches; ++r) {
    lplb_time_next_launch(start_events ? start_events[r] : nullptr, stop_events ? stop_events[r] : nullptr);
    const int rc = lplb_copy_calibration(src[r], dst[r], n_elements, stream);
    if (rc != LPLB_OK) {
      lplb_time_next_launch(nullptr, nullptr);
      return rc;
    }
  }
  return LPLB_OK;
}
