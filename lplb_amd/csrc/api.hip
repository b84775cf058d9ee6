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

// Plain streaming copy, 16 bytes per lane and trip: the yardstick the redirect's
// bandwidth and the profiler's byte counters are compared with.
typedef long long i64x2 __attribute__((ext_vector_type(2)));
__global__ __launch_bounds__(1024) void copy_calibration(const i64x2 *__restrict__ src,
                                                         i64x2 *__restrict__ dst, int64_t n_pairs) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_pairs; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
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
  const int64_t n_pairs = n_elements / 2;
  const int blocks = (int)((n_pairs + 1023) / 1024 < 2048 ? (n_pairs + 1023) / 1024 : 2048);
  launch(copy_calibration, dim3(blocks), dim3(1024), 0, static_cast<hipStream_t>(stream),
         reinterpret_cast<const i64x2 *>(src), reinterpret_cast<i64x2 *>(dst), n_pairs);
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}
