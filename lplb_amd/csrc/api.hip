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
// are compared with, in the fastest shape found for 16 MiB in + 16 MiB out on this GPU: two
// 16-byte loads per lane, 1024 threads per workgroup, so that 512 workgroups (all resident at
// once, eight waves per SIMD) cover the array in one trip, and a workgroup barrier between the
// loads and the stores.  Measured (kernel's own begin/end, 18 buffer pairs in turn): 5.8 us;
// without the barrier 6.8 us (reads and writes of a workgroup mix in time); one load per lane
// in twice as many workgroups, which then run in two rounds, 7.3 us; four loads per lane in
// half as many waves 6.3 us, eight 8.5 us.
typedef long long i64x2 __attribute__((ext_vector_type(2)));
constexpr int kCopyThreads = 1024, kCopyLoads = 2;
// WHOLE: the grid covers the array exactly, one tile per workgroup (no loop, no bounds).
template <bool WHOLE>
__global__ __launch_bounds__(kCopyThreads, 8) void copy_calibration(const i64x2 *__restrict__ src,
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
  const int64_t resident = 2 * (int64_t)(n_cus > 0 ? n_cus : 256);   // workgroups the GPU holds at once
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
