// LP solver entry points: batches of LPs, one per wave or four per wave.
// The device code and the description of the method are in solve_kernel.h.
#include "solve_kernel.h"

namespace lplb {

// One wave per workgroup; ROWS LPs per wave.
//
// Feasibility counter: updates of one address queue up behind each other in memory
// (about 10 ns each: 2048 waves that each add their result take 20 us longer than
// the arithmetic).  So the first thread of the grid counts every LP of the launch as
// feasible with one add, and a wave takes back the LPs of its own that failed -- rare,
// and the sum is the same.
template <int GM, int DM, bool EXACT, int ROWS, int EPL>
__global__ __launch_bounds__(kWave) void solve_groups(SolveArgs a) {
  extern __shared__ float staged_all[];   // a.staged_stride floats per LP of this wave
  __shared__ int rep_of_edge[EPL * kWave];
  __shared__ __attribute__((aligned(16))) double pivot_rows[2 * kWave];
  __shared__ __attribute__((aligned(16))) float tile[assembly_tile_floats<GM, EPL>()];
  if (blockIdx.x == 0 && threadIdx.x == 0)
    atomicAdd(a.avail, a.n_units);
  const int first_unit = blockIdx.x * ROWS;
  const int n_ok = solve_lp<GM, DM, EXACT, ROWS, EPL>(a, first_unit, staged_all, rep_of_edge, pivot_rows, tile);
  const int n_mine = min(max(a.n_units - first_unit, 0), ROWS);
  if (threadIdx.x == 0 && n_ok < n_mine)
    atomicAdd(a.avail, n_ok - n_mine);
}

// One LP per wave has the lowest latency (8 us at (8, 2)) and is the fastest form
// until the waves outnumber the SIMDs; from kPackFrom LPs on, shapes with G <= 16 and
// G * D <= 16 put four LPs into each wave (10.4 us per wave, a quarter of the waves).
// Measured at (8, 2): 1024 LPs 8.8 us unpacked; 2048 LPs 12.9 us unpacked, 11.4 us
// packed; 16384 LPs 73 us unpacked, 31 us packed.
constexpr int kPackFrom = 1536;
constexpr int kLdsLimit = 64 * 1024 - 2048;

template <int GM, int DM, bool EXACT, int ROWS, int EPL = 1>
static void launch_variant(SolveArgs a, hipStream_t s) {
  const size_t lds = (size_t)ROWS * a.n_experts * sizeof(float);
  a.staged_stride = lds <= kLdsLimit ? a.n_experts : 0;
  launch(solve_groups<GM, DM, EXACT, ROWS, EPL>, dim3((a.n_units + ROWS - 1) / ROWS), dim3(kWave),
         a.staged_stride ? lds : 0, s, a);
}

template <int GM, int DM, bool EXACT> static void launch_exactness(const SolveArgs &a, hipStream_t s) {
  if constexpr (GM <= kRowLanes && GM * DM <= kRowLanes) {
    if (a.n_units >= kPackFrom)
      return launch_variant<GM, DM, EXACT, 4>(a, s);
  }
  launch_variant<GM, DM, EXACT, 1>(a, s);
}

// A group that fills an instantiation exactly gets the variant whose loop bounds are all
// compile-time constants.  Instantiations with more than 64 edges (16 x 8, 32 x 4) exist only
// for the padded groups inside them (say 10 x 5 or 20 x 3): a group that filled them would
// have more edges than a wave has lanes and has been refused by then.
template <int GM, int DM> static void launch_solver(const SolveArgs &a, hipStream_t s) {
  if constexpr (GM * DM <= kWave) {
    if (a.G == GM && a.D == DM)
      return launch_exactness<GM, DM, true>(a, s);
  }
  launch_exactness<GM, DM, false>(a, s);
}

static int dispatch(const SolveArgs &a, hipStream_t s) {
  const int G = a.G, D = a.D;
  // 65 to 128 replica edges, or more than 8 slots per rank: two edges per lane, always the padded form (these shapes are rare, and one
  // kernel per row of this list serves every (G, D) inside it).
  if (G * D > kWave || D > 8) {
#define LPLB_WIDE_CASE(GM, DM)                                                 \
    if (G <= GM && D <= DM) {                                                  \
      launch_variant<GM, DM, false, 1, 2>(a, s);                               \
      return LPLB_OK;                                                          \
    }
    LPLB_WIDE_CASE(8, 16) LPLB_WIDE_CASE(16, 8) LPLB_WIDE_CASE(16, 16) LPLB_WIDE_CASE(32, 4) LPLB_WIDE_CASE(32, 8)
    LPLB_WIDE_CASE(64, 2) LPLB_WIDE_CASE(64, 4)
#undef LPLB_WIDE_CASE
    return fail(LPLB_EUNSUPPORTED, "solve: group_size=%d dup_per_rank=%d has no kernel", G, D);
  }
#define LPLB_CASE(GM, DM)                                                      \
  if (G <= GM && D <= DM) {                                                    \
    launch_solver<GM, DM>(a, s);                                               \
    return LPLB_OK;                                                            \
  }
  LPLB_CASE(8, 1) LPLB_CASE(8, 2) LPLB_CASE(8, 4) LPLB_CASE(8, 8)
  LPLB_CASE(16, 1) LPLB_CASE(16, 2) LPLB_CASE(16, 4) LPLB_CASE(16, 8)
  LPLB_CASE(32, 1) LPLB_CASE(32, 2) LPLB_CASE(32, 4)
  LPLB_CASE(64, 1)
#undef LPLB_CASE
  return fail(LPLB_EUNSUPPORTED, "solve: group_size=%d dup_per_rank=%d has no kernel", G, D);
}

} // namespace lplb

extern "C" int lplb_solve_batched(const int32_t *workloads, float *global_workloads,
                                  const int32_t *r2o, const int32_t *phy2log,
                                  int n_instances, int n_group, int group_size,
                                  int dup_per_rank, int n_experts_per_var,
                                  int n_experts_fixed, int32_t *avail_num,
                                  float *results, int step_rule, int n_steps,
                                  lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(workloads && r2o && phy2log && avail_num && results, LPLB_EINVAL,
               "solve: null pointer");
  LPLB_REQUIRE(n_instances > 0 && n_group > 0 && group_size > 0 && dup_per_rank > 0 &&
                   n_experts_per_var >= 0 && n_experts_fixed >= 0 && n_steps >= 0,
               LPLB_EINVAL,
               "solve: n_instances=%d n_group=%d group_size=%d dup_per_rank=%d per_var=%d fixed=%d n_steps=%d",
               n_instances, n_group, group_size, dup_per_rank, n_experts_per_var, n_experts_fixed,
               n_steps);
  LPLB_REQUIRE(step_rule == LPLB_STEP_REFERENCE_WINDOW || step_rule == LPLB_STEP_FULL_MAX,
               LPLB_EINVAL, "solve: unknown step_rule %d", step_rule);
  LPLB_REQUIRE(group_size * dup_per_rank <= 2 * kWave && group_size <= kWave && dup_per_rank <= 16, LPLB_EUNSUPPORTED,
               "solve: group_size=%d dup_per_rank=%d: at most 128 replica edges (two per lane of a wave), 64 ranks, "
               "16 slots per rank", group_size, dup_per_rank);
  const int64_t L = (int64_t)dup_per_rank * n_experts_per_var + n_experts_fixed;
  const int64_t n_experts = (int64_t)n_group * group_size * L;
  LPLB_REQUIRE(n_experts > 0 && n_experts <= (1 << 24) && (int64_t)n_instances * n_group <= INT32_MAX,
               LPLB_EINVAL, "solve: %lld experts x %d instances out of range",
               (long long)n_experts, n_instances);
  SolveArgs a{};
  a.workload = workloads; a.gw_out = global_workloads; a.r2o = r2o; a.phy2log = phy2log;
  a.avail = avail_num; a.result = results; a.n_group = n_group; a.G = group_size;
  a.D = dup_per_rank; a.C = n_experts_per_var; a.n_fixed = n_experts_fixed;
  a.n_experts = (int)n_experts; a.step_rule = step_rule; a.n_steps = n_steps; a.tagged_result = nullptr; a.tag_valid = 0; a.tagged_copies = 0; a.tagged_stride = 0; a.counts_ready = nullptr;
#ifdef LPLB_PHASE_CLOCKS
  a.clocks = g_phase_clocks;
#else
  a.clocks = nullptr;
#endif
  a.n_units = n_instances * n_group;
  int rc = dispatch(a, static_cast<hipStream_t>(stream));
  if (rc != LPLB_OK)
    return rc;
  LPLB_HIP_TRY(hipGetLastError());
  return LPLB_OK;
}

extern "C" int lplb_solve(const int32_t *workload, float *global_workload,
                          const int32_t *r2o, const int32_t *phy2log, int n_group,
                          int group_size, int dup_per_rank, int n_experts_per_var,
                          int n_experts_fixed, int32_t *avail_num, float *result,
                          int step_rule, int n_steps, lplb_stream_t stream) {
  LPLB_REQUIRE(global_workload != nullptr, LPLB_EINVAL, "solve: null global_workload");
  return lplb_solve_batched(workload, global_workload, r2o, phy2log, 1, n_group, group_size,
                            dup_per_rank, n_experts_per_var, n_experts_fixed, avail_num, result,
                            step_rule, n_steps, stream);
}
