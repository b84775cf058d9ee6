/*
 * C ABI of the MI355X planning library (liblplb_hip.so).
 *
 * Each entry point replaces one method of the reference's pybind11 class
 * `lplb._cpp.CompiledSolver` (csrc/plugin.cpp:663-679 of the reference) and
 * takes what that method's host code hands to its kernel: raw device pointers,
 * sizes and the stream.  All pointers are device pointers on the current HIP
 * device unless stated otherwise.  Inputs are borrowed, outputs are caller
 * allocated; the library owns no user-visible memory.  Calls only enqueue work
 * on `stream` (a hipStream_t passed as void*, NULL = the default stream) and
 * never synchronise.
 *
 * Every function returns 0 on success or an LPLB_E* code; the message of the
 * calling thread's last failure is available from lplb_last_error().  No C++
 * exception crosses this boundary.  An LP that fails the feasibility test is
 * not an error: its group gets the neutral split 0.5 and the feasible-solution
 * counter is left unchanged, as in the reference (minilp.cu:379-400).
 */
#ifndef LPLB_HIP_H
#define LPLB_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LPLB_ABI_VERSION 7

#define LPLB_OK 0
#define LPLB_EINVAL 1      /* bad argument (null pointer, negative size, ...) */
#define LPLB_EUNSUPPORTED 2 /* shape outside what the kernels are built for */
#define LPLB_EHIP 3        /* a HIP runtime call failed */
#define LPLB_EBUSY 4       /* a resource inside the library is in use by work on another stream */

/* Step-length rules of the affine-scaling iteration. */
#define LPLB_STEP_REFERENCE_WINDOW 0 /* max over the last 32 columns, as minilp.cu:355-359 does */
#define LPLB_STEP_FULL_MAX 1         /* max over all columns (and 0) */

typedef void *lplb_stream_t;

int lplb_abi_version(void);

/* Message of this thread's most recent failing call ("" if none). Host pointer. */
const char *lplb_last_error(void);

/*
 * Profiling aid, no counterpart in the reference.  The next kernel this thread
 * launches through the library records its own begin and end timestamps into
 * the two hipEvent_t (either may be NULL); hipEventElapsedTime(start, stop)
 * then gives that kernel's execution time, the figure a kernel trace reports,
 * without the launch overhead an event pair around the call would include.
 * The pair is consumed by that one launch.
 */
void lplb_time_next_launch(void *start_event, void *stop_event);

/*
 * Measurement aid, no counterpart in the reference: a plain streaming copy of
 * n_elements int64 (even count, 16-byte aligned) from src to dst.  Its achieved bandwidth is the
 * practical ceiling the redirect kernel is compared with, and its known traffic
 * (8 bytes read + 8 written per element) calibrates the profiler's byte counters.
 */
int lplb_copy_calibration(const int64_t *src, int64_t *dst, int64_t n_elements,
                          lplb_stream_t stream);

/*
 * Measurement aids, no counterpart in the reference: n_launches calls of
 * lplb_copy_calibration / lplb_map_idx_prepared issued from one tight loop, launch r on
 * src[r], dst[r] / idx[r], counts_by_block[r], out[r] (host arrays of n_launches device
 * pointers; the other arguments as for the single call, physical_counts not written), the
 * kernel of launch r recording its own begin and end into start_events[r] and
 * stop_events[r] (hipEvent_t, as for lplb_time_next_launch; either array may be NULL).
 * For benchmarks written in an interpreted language: per-launch durations taken from a
 * Python loop showed a tail (one launch in ten 4 us longer) that the same launches issued
 * from compiled code do not have.
 */
int lplb_copy_calibration_series(const int64_t *const *src, int64_t *const *dst,
                                 int64_t n_elements, int n_launches,
                                 void *const *start_events, void *const *stop_events,
                                 lplb_stream_t stream);
/*
 * Measurement aid, no counterpart in the reference: the copy of lplb_copy_calibration in
 * another shape (loads_per_lane 16-byte loads per lane: 1, 2, 4 or 8; threads per
 * workgroup: 256, 512 or 1024; with or without a workgroup barrier between loads and
 * stores; streaming or cached accesses), n_launches times as in the series above.
 * n_elements must be a multiple of 2 * threads * loads_per_lane.  This is what the choice
 * of lplb_copy_calibration's own shape rests on (bench.py --copy-sweep prints the table).
 */
int lplb_copy_shape_series(const int64_t *const *src, int64_t *const *dst, int64_t n_elements,
                           int n_launches, int loads_per_lane, int threads, int barrier,
                           int streaming, void *const *start_events, void *const *stop_events,
                           lplb_stream_t stream);
/*
 * Measurement aid, no counterpart in the reference: the first of lplb_count_idx's two kernels
 * (the histogram per slice, rows not yet summed over the slices) alone, n_launches times as in
 * the series above.  A kernel that is followed at once by another one on the stream reads
 * 1.3-1.6 us longer by its own events than in a series of its own; this gives the latter.
 */
int lplb_slice_histogram_series(const int64_t *const *idx, int64_t n_elements, int n_experts,
                                int n_blocks, int32_t *const *counts_by_block, int n_launches,
                                void *const *start_events, void *const *stop_events,
                                lplb_stream_t stream);
int lplb_map_idx_prepared_series(const int64_t *const *idx, const float *o_weight,
                                 const int32_t *const *counts_by_block, const void *prepared,
                                 int64_t n_elements, int n_group, int group_size,
                                 int dup_per_rank, int n_combined_experts, int n_local_experts,
                                 int n_blocks, int64_t *const *out, int n_launches,
                                 void *const *start_events, void *const *stop_events,
                                 lplb_stream_t stream);

/*
 * Per-expert token histogram with an inclusive prefix over slices.
 * Replaces CompiledSolver.count_idx (csrc/plugin.cpp:580-600, kernel
 * minilp.cu:410-443).
 *
 *   idx              int64 [n_elements], values in [-1, n_experts); -1 (and any
 *                    other out-of-range value) is not counted
 *   n_blocks         number of slices (the reference's n_sms).  Slice p covers
 *                    [min(n, per*p), min(n, per*(p+1))) with
 *                    per = roundup(ceil(n / n_blocks), 256)  (minilp.cu:404-408)
 *   counts_by_block  int32 [n_blocks, n_experts], out: row p = occurrences in
 *                    slices 0..p.  The last row is the full histogram.
 */
int lplb_count_idx(const int64_t *idx, int64_t n_elements, int n_experts,
                   int n_blocks, int32_t *counts_by_block, lplb_stream_t stream);

/*
 * This GPU's tokens per expert and nothing else (the last row of lplb_count_idx's
 * table), in one kernel launch.  No counterpart in the reference: it serves
 * Planner.run with a process group, which needs the counts for the all-reduce
 * ahead of the plan and no table (lplb/planner.py:209-216 gets them from count_idx).
 * Every workgroup reads the whole batch, so this is for short batches:
 * n_elements <= LPLB_COUNT_TOTALS_MAX_INDICES and n_experts <=
 * LPLB_COUNT_TOTALS_MAX_EXPERTS, LPLB_EUNSUPPORTED beyond (callers then use
 * lplb_count_idx).
 *
 *   totals           int32 [n_experts], out
 */
#define LPLB_COUNT_TOTALS_MAX_INDICES 131072
#define LPLB_COUNT_TOTALS_MAX_EXPERTS 1024
int lplb_count_totals(const int64_t *idx, int64_t n_elements, int n_experts,
                      int32_t *totals, lplb_stream_t stream);

/*
 * The same counts, ADDED to what `totals` holds, in one kernel launch of a few
 * workgroups: slices of 8192 indices count into LDS and add what they found with
 * device-wide atomic adds (n_elements <= LPLB_COUNT_TOTALS_MAX_INDICES: every
 * slice updates every counter, and updates of one line of memory queue up).
 * No counterpart in the reference.  The caller hands
 * in a vector that is zero (or holds counts to add to); so that it never has
 * to zero one itself, the launch also sets `clear` to zero if that is given:
 * a caller keeps two vectors and swaps them from call to call (Planner.run with
 * a process group does; a call that is captured into a graph must not rely on
 * that, since a replay starts with the vectors as the last replay left them).
 * n_experts * 4 bytes must fit 64 KiB of LDS (LPLB_EUNSUPPORTED beyond).
 *
 *   totals           int32 [n_experts], in/out, 8-byte aligned
 *   clear            int32 [n_experts], out (all zero), or NULL; not `totals`
 */
int lplb_count_totals_add(const int64_t *idx, int64_t n_elements, int n_experts,
                          int32_t *totals, int32_t *clear, lplb_stream_t stream);

/*
 * Builds and solves one LP per EP group: minimise the maximum per-rank load by
 * moving tokens along replica edges.  Replaces CompiledSolver.solve
 * (csrc/plugin.cpp:491-578, kernel minilp.cu:83-402 without its NVSHMEM branch).
 *
 *   workload         int32 [n_group, group_size, L], global per-expert counts,
 *                    L = dup_per_rank * n_experts_per_var + n_experts_fixed
 *   global_workload  fp32 [n_group, group_size, L], out: counts / max count
 *   r2o              int32 [group_size, dup_per_rank] replica topology
 *   phy2log          int32 [n_group * group_size * P], P = L + dup_per_rank *
 *                    n_experts_per_var; per rank: replicated originals (slot =
 *                    c * dup_per_rank + d), other originals, replicas
 *   avail_num        int32 [1], in/out: incremented once per group whose LP
 *                    passed the feasibility test (never reset here)
 *   result           fp32 [n_group, group_size, dup_per_rank], out: share of
 *                    each replicated expert set that stays on its original rank
 *   step_rule        LPLB_STEP_*; 0 reproduces the reference
 *   n_steps          number of affine-scaling steps; the reference uses 5
 *
 * Requires group_size * dup_per_rank <= 128, group_size <= 64 and
 * dup_per_rank <= 16 (LPLB_EUNSUPPORTED otherwise).  Up to 64 replica edges
 * and 8 slots per rank a lane of the wave holds one edge; beyond that, two.
 */
int lplb_solve(const int32_t *workload, float *global_workload,
               const int32_t *r2o, const int32_t *phy2log, int n_group,
               int group_size, int dup_per_rank, int n_experts_per_var,
               int n_experts_fixed, int32_t *avail_num, float *result,
               int step_rule, int n_steps, lplb_stream_t stream);

/*
 * n_instances independent lplb_solve problems that share r2o and phy2log, one
 * wavefront per (instance, group), in a single launch.  No counterpart in the
 * reference (it solves one batch per launch); workloads / global_workloads /
 * results carry a leading [n_instances] dimension.  global_workloads may be
 * NULL.  avail_num is incremented once per feasible (instance, group).
 */
int lplb_solve_batched(const int32_t *workloads, float *global_workloads,
                       const int32_t *r2o, const int32_t *phy2log,
                       int n_instances, int n_group, int group_size,
                       int dup_per_rank, int n_experts_per_var,
                       int n_experts_fixed, int32_t *avail_num, float *results,
                       int step_rule, int n_steps, lplb_stream_t stream);

/*
 * Logical -> physical redirect of routing indices.  Replaces
 * CompiledSolver.map_idx (csrc/plugin.cpp:602-660, kernel minilp.cu:445-515).
 *
 *   idx              int64 [n_elements] logical expert ids, -1 = masked
 *   o_weight         fp32 [n_group, group_size, dup_per_rank] from lplb_solve
 *   counts_by_block  int32 [n_blocks, n_logical] from lplb_count_idx on the
 *                    same idx and n_blocks
 *   o2r              int32 [group_size, dup_per_rank], column-wise inverse of r2o
 *   phy2log          as for lplb_solve
 *   n_combined_experts  replicated expert sets per replica slot (C)
 *   n_local_experts  physical experts per rank (P)
 *   out              int64 [n_elements]: -1 stays -1; token number k (counting
 *                    earlier occurrences of the same expert in index order) of
 *                    expert e goes to e's original slot if
 *                    (499 k + 41) mod total[e] < trunc(o_weight * total[e]),
 *                    else to its replica (minilp.cu:484-486, 503-509)
 *
 * The reference takes each token's k from a shared-memory atomic, so which
 * token of a block gets which k is unspecified there; here k always follows
 * index order, which makes the output deterministic and independent of
 * n_blocks.  Values outside [-1, n_logical) map to -1.
 *
 *   physical_counts  int32 [n_group * group_size * n_local_experts] or NULL, out:
 *                    tokens per physical expert, i.e. the bincount of `out` that the
 *                    reference's test computes afterwards
 *                    (tests/test_idx_processing.py:100-101) and a dispatch needs.
 *                    It comes from the kernel's tables (the hash is a bijection on
 *                    [0, total) unless 499 divides total, which has its own closed
 *                    form), not from another pass over the tokens.  Needs
 *                    n_elements <= 4303557 (499 k + 41 must not wrap).
 */
int lplb_map_idx(const int64_t *idx, const float *o_weight,
                 const int32_t *counts_by_block, const int32_t *o2r,
                 const int32_t *phy2log, int64_t n_elements, int n_group,
                 int group_size, int dup_per_rank, int n_combined_experts,
                 int n_local_experts, int n_blocks, int64_t *out,
                 int32_t *physical_counts, lplb_stream_t stream);

/*
 * The part of the redirect's tables that depends on the mapping only, built once per
 * mapping instead of by every workgroup of every batch.  The reference rebuilds these
 * tables (where each logical expert's original and replica sit) in every block of every
 * launch, minilp.cu:466-496; they change only when phy2log does
 * (lplb/planner.py:115-182, update_redundancy_mapping).
 *
 * lplb_prepared_mapping_bytes   size of the table for a shape (-1: bad shape)
 * lplb_prepare_mapping          fills `prepared` (device memory of the caller's, 16-byte
 *                               aligned, at least that many bytes) from o2r and phy2log;
 *                               one small kernel on `stream`.  The table is opaque; it
 *                               stays valid until phy2log, o2r or the shape change.
 *                               LPLB_EUNSUPPORTED beyond 511 replicated expert sets or
 *                               32767 physical experts.
 * lplb_map_idx_prepared         lplb_map_idx with the table in place of o2r and phy2log:
 *                               same arguments otherwise, same results bit for bit.
 */
int64_t lplb_prepared_mapping_bytes(int n_group, int group_size, int dup_per_rank,
                                    int n_combined_experts, int n_local_experts);
int lplb_prepare_mapping(const int32_t *o2r, const int32_t *phy2log, int n_group,
                         int group_size, int dup_per_rank, int n_combined_experts,
                         int n_local_experts, void *prepared, int64_t prepared_bytes,
                         lplb_stream_t stream);
int lplb_map_idx_prepared(const int64_t *idx, const float *o_weight,
                          const int32_t *counts_by_block, const void *prepared,
                          int64_t n_elements, int n_group, int group_size,
                          int dup_per_rank, int n_combined_experts, int n_local_experts,
                          int n_blocks, int64_t *out, int32_t *physical_counts,
                          lplb_stream_t stream);

/*
 * One batch's whole plan in a single call: what Planner.run does with three
 * extension calls (lplb/planner.py:245-266), with the same results as
 * lplb_count_idx, lplb_solve and lplb_map_idx chained on `stream`.  Batches of up
 * to about two million indices (slices of at most 8192 indices, as many of them as
 * fit the GPU together) with LP shapes up to 32 x 2, up to 32 EP groups and up to 1024
 * logical experts run as ONE kernel launch in which the workgroups exchange their
 * counts and the LP's result through memory; everything else runs as the chain of
 * the three entry points' kernels.
 *
 *   global_counts    int32 [n_logical] or NULL.  NULL: the LP is fed this GPU's
 *                    own histogram, as Planner.run does without a process
 *                    group.  Otherwise the counts already summed over all EP
 *                    ranks (what the all-reduce at lplb/planner.py:214-216
 *                    yields).
 *   n_blocks         upper bound on the workgroups used, at least 1
 *   counts_by_block  int32 [n_blocks, n_logical]: workspace; on return its last
 *                    row holds this GPU's tokens per expert (the rows above it
 *                    are unspecified)
 *   global_workload  fp32 [n_logical], out (see lplb_solve)
 *   o_weight         fp32 [n_group, group_size, dup_per_rank], out
 *   out              int64 [n_elements], out (see lplb_map_idx)
 *   physical_counts  int32 [n_physical] or NULL, out (see lplb_map_idx)
 *
 * The one-launch form: its workgroups wait for each other, so the whole grid has to be
 * resident on the GPU.  The library admits a launch only if the grid fits (worked out
 * from the kernel's registers and LDS) beside the one-launch plans that are still executing, of which it keeps
 * track per stream (eight streams per device at a time; every launch writes its number
 * into pinned host memory once all its workgroups have arrived, and the library looks at
 * those words: it never waits and never hands a stream of the caller's to the runtime
 * after the call that brought it); otherwise the call runs the
 * chain, with identical results.  A plan captured into a graph keeps its share of the GPU reserved
 * from then on (its replays are invisible to the library; see lplb_plan_forget_captured).  Launches on one stream never overlap; the exception the
 * library cannot see is a graph captured on one stream and replayed concurrently on
 * several (see lplb_plan_set_cooperative).  Every wait inside the kernel is bounded; if one
 * runs out, the launch still completes, with a valid but unbalanced result: the tokens of
 * the slices whose wait ran out go to their experts' original slots (so every entry of
 * `out` still names a slot that holds the token's expert).  avail_num does not vouch for
 * such a batch: the reference's callers read "avail_num grew by n_group" as "this batch was
 * balanced" (tests/test_solve.py:58), so the first workgroup that gives up takes the
 * launch's feasible LPs back out of avail_num and LPs that finish later do not add
 * themselves; the same holds for every later plan on a block of counters that is switched
 * off.  The failure is also counted (lplb_plan_poll_timeouts reports the count without
 * waiting, lplb_plan_sync_timeouts reports it and switches the one-launch form on again).
 * What else such a call returns: physical_counts is filled with -1 when the workgroup that
 * writes it is among those that gave up (always the case when the counts of the batch never
 * became complete) and may otherwise not match `out`; the last row of counts_by_block may
 * not have been written.
 */
int lplb_plan(const int64_t *idx, int64_t n_elements,
              const int32_t *global_counts, const int32_t *r2o,
              const int32_t *o2r, const int32_t *phy2log, int n_group,
              int group_size, int dup_per_rank, int n_combined_experts,
              int n_local_experts, int n_blocks, int32_t *counts_by_block,
              float *global_workload, float *o_weight, int32_t *avail_num,
              int64_t *out, int32_t *physical_counts, int step_rule, int n_steps,
              lplb_stream_t stream);

/*
 * lplb_plan for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in
 * the reference (its extension allocates its outputs with at::empty on every call,
 * csrc/plugin.cpp:504-505, 532-534, 586-587, 630).
 *
 * Same arguments, results and error codes as lplb_plan, except that the slice table
 * (lplb_plan's counts_by_block workspace) is not passed in: it lives in a fixed
 * 1 MiB array inside the library, one copy per GPU, held until the process ends.
 * The call and everything it enqueues allocates and frees nothing.
 *
 *   local_counts     int32 [n_logical] or NULL, out: this GPU's tokens per logical
 *                    expert (what the last row of lplb_plan's counts_by_block holds)
 *
 * Limit: n_blocks * n_logical <= 262144 counters (LPLB_EUNSUPPORTED beyond; e.g. 256
 * slices of 1024 logical experts, 1024 slices of 256).  Every call on a GPU uses that
 * GPU's one table, whatever the stream.  Calls on one stream are ordered and safe; a call
 * on another stream is refused with LPLB_EBUSY while the previous caller's kernels may
 * still be running (the last kernel of every call reports its end in a word of pinned host
 * memory, which the next call looks at; nothing waits), and for good once a call has been
 * captured into a graph, whose replays the library cannot see.  Calls replayed from graphs
 * captured on different streams are the caller's to keep apart.  The table keeps the
 * previous call's contents; nothing in it needs clearing, every row is written before it
 * is read.  The first call on a device looks the table's address up, sets that word up and
 * reads the kernels' attributes: it has to happen outside a stream capture.
 */
int lplb_plan_noalloc(const int64_t *idx, int64_t n_elements,
                      const int32_t *global_counts, const int32_t *r2o,
                      const int32_t *o2r, const int32_t *phy2log, int n_group,
                      int group_size, int dup_per_rank, int n_combined_experts,
                      int n_local_experts, int n_blocks, int32_t *local_counts,
                      float *global_workload, float *o_weight, int32_t *avail_num,
                      int64_t *out, int32_t *physical_counts, int step_rule, int n_steps,
                      lplb_stream_t stream);

/*
 * No counterpart in the reference.  enabled = 0 makes lplb_plan always run the
 * chain of kernels (for callers that replay captured plans concurrently on
 * several streams, that let four or more plans execute at once, or that keep the
 * GPU full of kernels which themselves wait for a plan); 1 (the default) lets it use the one-launch form where that applies.
 * Process-wide.
 */
int lplb_plan_set_cooperative(int enabled);

/*
 * No counterpart in the reference.  A one-launch plan that was captured into a
 * graph keeps its share of the GPU reserved, because a replay may come at any
 * time (see lplb_plan).  A caller who has destroyed every graph that holds a plan
 * captured on `stream` (on the current device), and whose replays have all ended,
 * says so here: the share is given back and the stream's block of counters may
 * pass to another stream.  Not needed where all graphs are captured on one
 * stream (they share one reservation, the largest).
 */
int lplb_plan_forget_captured(lplb_stream_t stream);

/*
 * No counterpart in the reference.  The workgroups of the one-launch plan wait
 * for each other with a bounded number of polls; *count receives how many waits
 * ran out on the current device since the library was loaded (0 in a healthy
 * run; what a plan with such a wait returns is described at lplb_plan), and the
 * one-launch form is switched on again for the streams on which a wait had run out.
 * Synchronous: waits for everything enqueued on the device, then copies a few ints.  Not
 * to be called while a stream is being captured or while other threads enqueue plans.
 */
int lplb_plan_sync_timeouts(int *count);

/*
 * No counterpart in the reference.  The same health report without waiting: a one-thread
 * kernel on `stream` writes dst[0] = waits that ran out on the current device since the
 * library was loaded and dst[1] = blocks of counters that are switched off right now.
 * dst: two int32 in device memory or in pinned host memory (which the caller reads once
 * work enqueued after this call has completed, or simply at its next look).  Nothing is
 * cleared or switched on again; that takes lplb_plan_sync_timeouts.
 */
int lplb_plan_poll_timeouts(int32_t *dst, lplb_stream_t stream);

/*
 * No counterpart in the reference.  *count receives how many lplb_plan /
 * lplb_plan_noalloc calls of this process ran as one kernel launch (the others ran
 * the chain of kernels).  For callers and tests that want to know which form they got.
 */
int lplb_plan_one_launch_count(long long *count);

/*
 * Test hook, no counterpart in the reference.  The next plan that runs as one launch
 * waits for extra_slices_expected more slices than its grid has (so the wait cannot be
 * met) and gives up after max_polls polls instead of millions (0 = the default bound).
 * Every kernel still ends normally; the call exists to exercise the give-up path.
 */
int lplb_plan_inject_fault(int extra_slices_expected, int max_polls);

#ifdef __cplusplus
}
#endif
#endif /* LPLB_HIP_H */
