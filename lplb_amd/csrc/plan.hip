// Whole plan in one call: histogram -> LP solve -> redirect on one stream.
// With the global counts supplied the LP does not depend on this GPU's histogram:
// it is enqueued first and the histogram launch does not wait for it (it still
// starts after everything the LP launch waited for); prefix and redirect are ordered
// after both.  Running the LP as a parallel branch of a captured HIP graph (side
// stream + events) was measured and rejected: 24.6 us per plan against 20.0 us for
// the plain chain in the graph.
#include "common.h"

extern "C" int lplb_plan(const int64_t *idx, int64_t n_elements,
                         const int32_t *global_counts, const int32_t *r2o,
                         const int32_t *o2r, const int32_t *phy2log, int n_group,
                         int group_size, int dup_per_rank, int n_combined_experts,
                         int n_local_experts, int n_blocks, int32_t *counts_by_block,
                         float *global_workload, float *o_weight, int32_t *avail_num,
                         int64_t *out, int step_rule, int n_steps,
                         lplb_stream_t stream) {
  using namespace lplb;
  LPLB_REQUIRE(n_group > 0 && group_size > 0 && dup_per_rank > 0 && n_blocks > 0, LPLB_EINVAL,
               "plan: n_group=%d group_size=%d dup_per_rank=%d n_blocks=%d must be positive",
               n_group, group_size, dup_per_rank, n_blocks);
  const int L = n_local_experts - dup_per_rank * n_combined_experts;
  const int n_fixed = L - dup_per_rank * n_combined_experts;
  LPLB_REQUIRE(L > 0 && n_fixed >= 0 && n_combined_experts >= 0, LPLB_EINVAL,
               "plan: n_local_experts=%d does not fit %d x %d replicas", n_local_experts,
               dup_per_rank, n_combined_experts);
  LPLB_REQUIRE(counts_by_block != nullptr, LPLB_EINVAL, "plan: null counts_by_block");
  const int n_logical = n_group * group_size * L;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc;
  if (global_counts) {
    LPLB_REQUIRE(n_elements >= 0 && n_elements <= INT32_MAX && (idx || n_elements == 0), LPLB_EINVAL,
                 "plan: bad idx / n_elements=%lld", (long long)n_elements);
    LPLB_REQUIRE((reinterpret_cast<uintptr_t>(idx) & 15) == 0, LPLB_EINVAL, "plan: idx must be 16-byte aligned");
    rc = lplb_solve(global_counts, global_workload, r2o, phy2log, n_group, group_size, dup_per_rank,
                    n_combined_experts, n_fixed, avail_num, o_weight, step_rule, n_steps, stream);
    if (rc != LPLB_OK)
      return rc;
    rc = enqueue_count(idx, n_elements, n_logical, n_blocks, counts_by_block, s, /*any_order=*/true);
    if (rc != LPLB_OK)
      return rc;
  } else {
    rc = lplb_count_idx(idx, n_elements, n_logical, n_blocks, counts_by_block, stream);
    if (rc != LPLB_OK)
      return rc;
    rc = lplb_solve(counts_by_block + (int64_t)(n_blocks - 1) * n_logical, global_workload, r2o, phy2log,
                    n_group, group_size, dup_per_rank, n_combined_experts, n_fixed, avail_num, o_weight,
                    step_rule, n_steps, stream);
    if (rc != LPLB_OK)
      return rc;
  }
  return lplb_map_idx(idx, o_weight, counts_by_block, o2r, phy2log, n_elements, n_group,
                      group_size, dup_per_rank, n_combined_experts, n_local_experts, n_blocks, out,
                      stream);
}
