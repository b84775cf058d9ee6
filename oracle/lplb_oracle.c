/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement (plain C, scalar, one thread) of
 * the reference's per-batch planning path: histogram + prefix, LP build +
 * fixed-step affine-scaling solve, logical->physical redirect.  Only tests, the
 * smoke check and the benchmark's cpu_baseline leg may load this library, and
 * only as the checker; the product path never calls it.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference checkout).
 *
 * Parity status
 *   split_and_align, count_idx   pinned: closed form (per-slice bincount +
 *                                cumulative sum), the reference test's
 *                                scatter_add histogram and sum invariant.
 *   map_idx                      pinned: brute force on tiny inputs, exact split
 *                                counts when 499 does not divide the total, the
 *                                reference test's membership / -1 / 5e-2 ratio
 *                                properties.  Ordinals are assigned in flat
 *                                index order (one valid schedule of the
 *                                reference's shared-memory atomics, whose
 *                                order inside a block is otherwise unspecified).
 *   build_lp                     pinned: A.1 = b, column non-zero pattern,
 *                                hand-checked 2-rank case.
 *   solve (algorithm)            pinned: A.x = b kept by every iterate,
 *                                HiGHS lower bound, symmetry, the reference
 *                                test suite's balance thresholds.
 *   solve (rounding)             PARITY UNPINNED at bit level: the reference's
 *                                products and Cholesky come from closed-source
 *                                cuBLASDx / cuSolverDx; see solve_core.inc.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define REAL float
#define SUFFIX _f32
#define FMAX fmaxf
#define FABS fabsf
#define FSQRT sqrtf
#include "solve_core.inc"
#undef REAL
#undef SUFFIX
#undef FMAX
#undef FABS
#undef FSQRT

#define REAL double
#define SUFFIX _f64
#define FMAX fmax
#define FABS fabs
#define FSQRT sqrt
#include "solve_core.inc"
#undef REAL
#undef SUFFIX
#undef FMAX
#undef FABS
#undef FSQRT

/* minilp.cu:404-408.  The reference computes in int; 64-bit intermediates give
 * the same values wherever that does not overflow and stay defined up to
 * n = INT_MAX. */
int lplb_oracle_split_and_align(int n, int par_rank, int par_size, int align) {
  long long per = ((long long)n + par_size - 1) / par_size;
  per = (per + align - 1) / align * align;
  long long v = per * par_rank;
  return v < n ? (int)v : n;
}

/* minilp.cu:410-443 (launched by csrc/plugin.cpp:580-600).
 * counts is [n_prog][n_experts]; on return row p holds the number of
 * occurrences of each expert in slices 0..p (inclusive prefix over slices).
 * -1 entries are dropped (the reference parks them in smem_counts[-1]). */
void lplb_oracle_count_idx(const int64_t *idx, int n_elements, int n_experts,
                           int n_prog, int block_size, int32_t *counts) {
  memset(counts, 0, sizeof(int32_t) * (size_t)n_prog * n_experts);
  for (int p = 0; p < n_prog; ++p) {
    int start = lplb_oracle_split_and_align(n_elements, p, n_prog, block_size);
    int end = lplb_oracle_split_and_align(n_elements, p + 1, n_prog, block_size);
    for (int i = start; i < end; ++i)
      if (idx[i] >= 0 && idx[i] < n_experts)
        counts[(size_t)p * n_experts + idx[i]] += 1;
  }
  for (int e = 0; e < n_experts; ++e)
    for (int p = 1; p < n_prog; ++p)
      counts[(size_t)p * n_experts + e] += counts[(size_t)(p - 1) * n_experts + e];
}

/* minilp.cu:181-189: divide every count by the maximum over ALL experts of
 * ALL groups, in fp32 (an all-zero input gives 0/0 = NaN, as there). */
void lplb_oracle_normalise(const int32_t *workload, int n_experts, float *gw) {
  float wmax = 0.0f;
  for (int i = 0; i < n_experts; ++i)
    wmax = fmaxf(wmax, (float)workload[i]);
  for (int i = 0; i < n_experts; ++i)
    gw[i] = (float)workload[i] / wmax;
}

/* Exposes the dense LP of one group for inspection (fp32).
 * a is [NC][NV], b [NC], c [NV], dupw [G*D]. */
void lplb_oracle_build_lp(const int32_t *workload, const int32_t *r2o,
                          const int32_t *phy2log, int n_group, int group, int G,
                          int D, int n_per_var, int n_fixed, float *dupw,
                          float *b, float *a, float *c) {
  const int L = D * n_per_var + n_fixed, P = L + D * n_per_var;
  const int n_experts = n_group * G * L;
  float *gw = (float *)malloc(sizeof(float) * n_experts);
  lplb_oracle_normalise(workload, n_experts, gw);
  build_lp_f32(gw, r2o, phy2log + (size_t)group * G * P, G, D, n_per_var,
               n_fixed, dupw, b, a, c);
  free(gw);
}

/* kernel_solve, minilp.cu:83-402 without the NVSHMEM branch, as launched by
 * csrc/plugin.cpp:491-578 (grid = n_group).  precision 32 or 64 selects the
 * arithmetic of the LP build and iteration; normalisation is always fp32.
 * x_out ([n_group][NV], as float or double per precision), trace
 * ([n_group][n_steps][4]) and resid ([n_group]) may be NULL. */
void lplb_oracle_solve(const int32_t *workload, float *global_workload,
                       const int32_t *r2o, const int32_t *phy2log, int n_group,
                       int G, int D, int n_per_var, int n_fixed,
                       int32_t *avail_num, float *result, int step_rule,
                       int n_steps, int precision, void *x_out, void *trace,
                       void *resid) {
  const int L = D * n_per_var + n_fixed, P = L + D * n_per_var;
  const int n_experts = n_group * G * L;
  const int NV = 2 * G * D + G + 2;
  lplb_oracle_normalise(workload, n_experts, global_workload);
  for (int g = 0; g < n_group; ++g) {
    const int32_t *p2l = phy2log + (size_t)g * G * P;
    float *res = result + (size_t)g * G * D;
    int flag;
    if (precision == 64)
      flag = solve_group_f64(
          global_workload, r2o, p2l, G, D, n_per_var, n_fixed, step_rule,
          n_steps, res, x_out ? (double *)x_out + (size_t)g * NV : NULL,
          trace ? (double *)trace + (size_t)g * n_steps * 4 : NULL,
          resid ? (double *)resid + g : NULL);
    else
      flag = solve_group_f32(
          global_workload, r2o, p2l, G, D, n_per_var, n_fixed, step_rule,
          n_steps, res, x_out ? (float *)x_out + (size_t)g * NV : NULL,
          trace ? (float *)trace + (size_t)g * n_steps * 4 : NULL,
          resid ? (float *)resid + g : NULL);
    *avail_num += flag; /* minilp.cu:383 */
  }
}

/* (int)(float) with the GPU's conversion semantics (round toward zero,
 * saturating, NaN -> 0) instead of x86's "integer indefinite". */
static int32_t f2i_rz_sat(float v) {
  if (v != v)
    return 0;
  if (v >= 2147483648.0f)
    return INT32_MAX;
  if (v <= -2147483648.0f)
    return INT32_MIN;
  return (int32_t)v;
}

/* kernel_map_idx, minilp.cu:445-515 (launched by csrc/plugin.cpp:602-660).
 * by_sm is count_idx's output [n_prog][n_logical].  Each slice p starts its
 * per-expert running ordinal at by_sm[p-1][e]; inside a slice ordinals follow
 * flat index order.  Because slice p covers exactly the indices counted in row
 * p, the ordinal of a token is the number of earlier tokens of the same expert
 * in the whole array, whatever n_prog is. */
void lplb_oracle_map_idx(const int64_t *idx, const float *o_weight,
                         const int32_t *by_sm, const int32_t *o2r,
                         const int32_t *phy2log, int n_elements, int n_group,
                         int G, int D, int n_combined, int n_local, int n_prog,
                         int block_size, int64_t *out) {
  const int L = n_local - D * n_combined; /* logical experts per rank */
  const int n_logical = n_group * G * L;
  int32_t *total = (int32_t *)malloc(sizeof(int32_t) * 5 * (size_t)n_logical);
  int32_t *expected = total + n_logical;
  int32_t *current = expected + n_logical;
  int32_t *log2r = current + n_logical;
  const int32_t *last = by_sm + (size_t)(n_prog - 1) * n_logical;

  for (int p = 0; p < n_prog; ++p) {
    /* :466-475 */
    for (int i = 0; i < n_logical; ++i) {
      total[i] = expected[i] = last[i];
      current[i] = p == 0 ? 0 : by_sm[(size_t)(p - 1) * n_logical + i];
    }
    for (int i = 0; i < n_logical; ++i)
      log2r[2 * i + 1] = -1;
    for (int i = 0; i < n_logical; ++i) {
      int slot = (i / L) * n_local + (i % L);
      log2r[2 * phy2log[slot]] = slot;
    }
    /* :478-495 */
    for (int i = 0; i < n_group * G * n_combined * D; ++i) {
      int ep_rank = i / (n_combined * D);
      int local = i % (n_combined * D);
      int e = phy2log[ep_rank * n_local + local];
      expected[e] = f2i_rz_sat(o_weight[ep_rank * D + local % D] * (float)last[e]);
      int i_group = ep_rank / G, group_rank = ep_rank % G;
      log2r[2 * e + 1] = (i_group * G + o2r[group_rank * D + local % D] + 1) * n_local -
                         n_combined * D + local;
    }
    /* :498-513 */
    int start = lplb_oracle_split_and_align(n_elements, p, n_prog, block_size);
    int end = lplb_oracle_split_and_align(n_elements, p + 1, n_prog, block_size);
    for (int i = start; i < end; ++i) {
      int64_t e = idx[i];
      int64_t o = -1;
      if (e >= 0 && e < n_logical) {
        int32_t k = current[e]++;
        /* int32 arithmetic; written with unsigned wrap to stay defined */
        int32_t h = (int32_t)((uint32_t)k * 499u + 41u);
        /* a zero total cannot occur with a consistent by_sm; keep it defined */
        h = total[e] > 0 ? h % total[e] : 0;
        o = log2r[2 * e + (h >= expected[e])];
      }
      out[i] = o;
    }
  }
  free(total);
}
