// Shared host/device helpers of the planning kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>
#include <utility>

#include "../../include/lplb_hip.h"

namespace lplb {

constexpr int kWave = 64;
// Slice boundaries are aligned to this many indices whatever the workgroup
// size is; it is part of the observable slice partition (minilp.cu:404-408
// is called with the reference's fixed block size of 256).
constexpr int kSliceAlign = 256;

// Records a message for lplb_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define LPLB_REQUIRE(cond, code, ...)                                          \
  do {                                                                         \
    if (!(cond))                                                               \
      return ::lplb::fail((code), __VA_ARGS__);                                \
  } while (0)

#define LPLB_HIP_TRY(expr)                                                     \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess)                                                      \
      return ::lplb::fail(LPLB_EHIP, "%s failed: %s", #expr,                   \
                          hipGetErrorString(e_));                              \
  } while (0)

// Events handed to lplb_time_next_launch() by this thread, cleared by the call.
struct LaunchEvents {
  hipEvent_t start = nullptr, stop = nullptr;
};
LaunchEvents take_launch_events();

// Compute units of the current device (looked up once per device); 0 if the query fails.
int current_device_cu_count();

// Lets `kernel` use up to `bytes` of dynamic LDS (above the 64 KiB default the
// runtime has to be told, once per kernel and device).
template <typename Kernel> hipError_t allow_dynamic_lds(Kernel kernel, int bytes) {
  static std::atomic<bool> told[64];
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess)
    return err;
  if (dev < 0 || dev >= 64 || !told[dev].load(std::memory_order_acquire)) {
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (err == hipSuccess && dev >= 0 && dev < 64)
      told[dev].store(true, std::memory_order_release);
  }
  return err;
}

// Every kernel of the library is launched through here.  If the calling thread
// armed a pair of events, the launch records the kernel's own begin and end
// timestamps into them (not the time the launch was enqueued).
template <typename Kernel, typename... Args>
inline void launch_with_flags(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                              unsigned flags, Args... args) {
  const LaunchEvents ev = take_launch_events();
  if (ev.start || ev.stop || flags)
    hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, ev.start, ev.stop, flags, args...);
  else
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
}
template <typename Kernel, typename... Args>
inline void launch(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, Args... args) {
  launch_with_flags(kernel, grid, block, lds, stream, 0u, args...);
}

// count.hip: histogram + scan; any_order lets it overlap the kernel enqueued just before it.
int enqueue_count(const int64_t *idx, int64_t n_elements, int n_experts, int n_blocks,
                  int32_t *counts_by_block, hipStream_t s, bool any_order);

#ifdef LPLB_PHASE_CLOCKS
// Debug builds only (-DLPLB_PHASE_CLOCKS): device buffer that receives the 100 MHz
// wall clock at phase boundaries of selected waves; set with
// lplb_debug_set_phase_clocks().  Product builds compile the stamps away.
extern long long *g_phase_clocks;
#define LPLB_STAMP_AT(ptr, k)                                                  \
  do {                                                                         \
    if ((ptr) && threadIdx.x == 0)                                             \
      (ptr)[k] = wall_clock64();                                               \
  } while (0)
inline long long *debug_clocks() { return g_phase_clocks; }
#else
#define LPLB_STAMP_AT(ptr, k) do { } while (0)
inline long long *debug_clocks() { return nullptr; }
#endif

// Length of one slice: ceil(n / parts) rounded up to kSliceAlign.
__host__ __device__ inline int64_t slice_len(int64_t n, int parts) {
  int64_t per = (n + parts - 1) / parts;
  return (per + kSliceAlign - 1) / kSliceAlign * kSliceAlign;
}

__host__ __device__ inline int64_t slice_begin(int64_t n, int64_t per, int p) {
  int64_t v = per * p;
  return v < n ? v : n;
}

// Calls f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N - 1>):
// a loop whose index is a constant expression.
template <typename F, int... I> __device__ inline void static_for_impl(F &f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ inline void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Kernel arguments are fetched from memory by scalar loads, and the compiler issues each load
// where its value is first needed: behind an early exit, inside a branch.  Every such place is one
// more round trip to memory in front of the kernel's real work (0.7 us each, measured: the
// arguments were written by the host a moment ago and are in no cache).  Naming the arguments here,
// at the top of a kernel, makes the compiler fetch them all in one batch.  For the streaming kernels,
// whose workgroups all need everything; the LP's lone wave is faster with its first loads issued as
// soon as their own arguments are there (measured: 0.5 us per plan).
template <typename T> __device__ inline void fetch_argument_now(T v) { asm volatile("" ::"s"(v)); }
template <typename... T> __device__ inline void fetch_arguments_now(T... v) { (fetch_argument_now(v), ...); }

// ---- wave64 primitives -----------------------------------------------------

__device__ inline int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

template <typename T> __device__ inline T bpermute(T v, int src_lane) {
  static_assert(sizeof(T) == 4, "32-bit values only");
  int r = __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, v));
  return __builtin_bit_cast(T, r);
}

// Value of `v` in lane `src` (wave-uniform, compile-time or scalar `src`).
__device__ inline float readlane(float v, int src) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src));
}
__device__ inline double readlane(double v, int src) {
  int2 p = __builtin_bit_cast(int2, v);
  p.x = __builtin_amdgcn_readlane(p.x, src);
  p.y = __builtin_amdgcn_readlane(p.y, src);
  return __builtin_bit_cast(double, p);
}

// Butterfly reductions; every lane ends with the result.
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1)
    v += bpermute(v, lane_id() ^ off);
  return v;
}
// fmaxf semantics: a NaN operand is ignored unless both are NaN.
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1)
    v = fmaxf(v, bpermute(v, lane_id() ^ off));
  return v;
}

} // namespace lplb
