// LP solver: one wave64 per EP group, no workgroup barriers.
//
// Problem (reference: minilp.cu:199-293).  For a group of G ranks with D replica
// slots each, n = G*D replica edges.  Edge j = (k, d) carries the normalised
// token count w_j of rank k's d-th replicated expert set; a copy lives on the
// rank i with r2o[i][d] == k.  Variables: x_o[j] (share kept on k), x_r[j] (share
// sent to the copy), slack s_i per rank, the maximum load t and a Big-M
// artificial x_M.  Constraints: per rank i,
//     sum_{j on i} w_j x_o[j] + sum_{j copied to i} w_j x_r[j] + s_i - t + m_i x_M = b_i,
// per edge x_o[j] + x_r[j] - x_M = 1; minimise t + 1000 x_M.  m makes x = 1 feasible.
//
// Method (reference: minilp.cu:331-400): a fixed number of primal affine-scaling
// steps x <- x (1 - alpha d), d = x (c - A^T w), (A X^2 A^T) w = A X^2 c,
// alpha = 0.999 / d_max, then a feasibility test; same iteration count, step
// rule, thresholds and fallback as the reference.
//
// What is different is how (A X^2 A^T) w = A X^2 c is solved.  The reference
// forms the dense (G+n) x (G+n) matrix and calls a block Cholesky.  A has two
// structural non-zeros per edge column, so eliminating the n edge rows by hand
// (they are diagonal plus a rank-one term) leaves a G x G system
//     S = sum_j lambda_j (e_k - e_i)(e_k - e_i)^T + diag(s^2) + t^2 11^T + kappa v v^T
// -- a weighted graph Laplacian of the replica topology plus a diagonal and two
// rank-one terms -- with right-hand side -t^2 1 + 1000 kappa v, where
//     E_j = x_o^2 + x_r^2, u_j = 1/E_j, lambda_j = w_j^2 x_o^2 x_r^2 u_j,
//     kappa = x_M^2 / (1 + x_M^2 sum u), q = B u, v = m + q.
// Lane i of the wave owns rank i and row i of S, lane j owns edge j.  S is
// assembled, factorised (right-looking Cholesky, pivots broadcast with
// v_readlane) and solved in fp64: it is tiny, and fp64 here removes the
// 1e-4..1e-3 rounding scatter a 32-bit factorisation shows on nearly balanced
// loads.  Everything else is fp32.  The factor is transposed through LDS once per
// step so that the backward substitution is also a column sweep.
#include "common.h"

namespace lplb {

struct SolveArgs {
  const int32_t *workload;   // [n_inst][n_experts]
  float *gw_out;             // [n_inst][n_experts] or null
  const int32_t *r2o;        // [G][D]
  const int32_t *phy2log;    // [n_group][G][P]
  int32_t *avail;
  float *result;             // [n_inst][n_group][G][D]
  int n_group, G, D, C, n_fixed, n_experts, step_rule, n_steps;
};

template <int CTRL> __device__ inline float dpp(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
constexpr int kQuadSwap1 = 0xB1;    // quad_perm [1,0,3,2]
constexpr int kQuadSwap2 = 0x4E;    // quad_perm [2,3,0,1]
constexpr int kHalfMirror = 0x141;  // reverse within 8 lanes
constexpr int kRowMirror = 0x140;   // reverse within 16 lanes

// Sum over the 64 lanes; every lane gets the same bits.
__device__ inline float reduce_sum(float v) {
  v += dpp<kQuadSwap1>(v);
  v += dpp<kQuadSwap2>(v);
  v += dpp<kHalfMirror>(v);
  v += dpp<kRowMirror>(v);
  return (readlane(v, 0) + readlane(v, 16)) + (readlane(v, 32) + readlane(v, 48));
}
// Max with fmaxf semantics (NaN ignored unless everything is NaN).
__device__ inline float reduce_max(float v) {
  v = fmaxf(v, dpp<kQuadSwap1>(v));
  v = fmaxf(v, dpp<kQuadSwap2>(v));
  v = fmaxf(v, dpp<kHalfMirror>(v));
  v = fmaxf(v, dpp<kRowMirror>(v));
  return fmaxf(fmaxf(readlane(v, 0), readlane(v, 16)), fmaxf(readlane(v, 32), readlane(v, 48)));
}

// 1/sqrt(a) in fp64: hardware estimate + two Newton steps.
__device__ inline double rsqrt_f64(double a) {
  double r = __builtin_amdgcn_rsq(a);
  r = r * (1.5 - 0.5 * a * r * r);
  r = r * (1.5 - 0.5 * a * r * r);
  return r;
}

template <int GM, int DM>
__global__ __launch_bounds__(kWave) void solve_groups(SolveArgs a) {
  // GM and DM only size the register arrays; the host checks G*D <= 64 edges.
  constexpr int T = kWave / GM;      // lanes that share the work of one rank's b_i
  constexpr int LS = GM + 1;         // padded row stride of the transpose buffer
  __shared__ double lt_buf[GM * LS];

  const int lane = threadIdx.x;
  const int G = a.G, D = a.D, C = a.C, n = G * D;
  const int L = D * C + a.n_fixed, P = L + D * C;
  const int grp = blockIdx.x % a.n_group, inst = blockIdx.x / a.n_group;
  const int32_t *wl = a.workload + (int64_t)inst * a.n_experts;
  const int32_t *p2l = a.phy2log + (int64_t)grp * G * P;

  // Normalisation by the maximum over all experts of all groups (minilp.cu:181-189).
  float wmax = 0.0f;
  for (int i = lane; i < a.n_experts; i += kWave)
    wmax = fmaxf(wmax, (float)wl[i]);
  wmax = reduce_max(wmax);
  if (a.gw_out) {
    float *gw = a.gw_out + (int64_t)inst * a.n_experts;
    for (int i = grp * G * L + lane; i < (grp + 1) * G * L; i += kWave)
      gw[i] = (float)wl[i] / wmax;
  }
  auto norm_count = [&](int e) -> float {
    return (e >= 0 && e < a.n_experts) ? (float)wl[e] / wmax : 0.0f;
  };

  // ---- per-edge constants (lane j < n) ----
  const bool is_edge = lane < n;
  const int ek = is_edge ? lane / D : 0;   // original rank of my edge
  const int ed = is_edge ? lane % D : 0;   // its replica slot
  float w = 0.0f;                          // minilp.cu:203-221
  if (is_edge)
    for (int c = 0; c < C; ++c)
      w += norm_count(p2l[ek * P + c * D + ed]);
  int erep = ek;                           // rank holding the copy of my edge
  if (is_edge)
    for (int i = 0; i < G; ++i)
      if (a.r2o[i * D + ed] == ek)
        erep = i;

  // ---- per-rank constants (lane i < G) ----
  const bool is_rank = lane < G;
  int src_o[DM], src_r[DM], oth_o[DM], oth_r[DM];
  float w_o[DM], w_r[DM];
#pragma unroll
  for (int d = 0; d < DM; ++d) {
    const bool on = is_rank && d < D;
    int k = on ? a.r2o[lane * D + d] : 0;
    k = k < 0 ? 0 : (k >= G ? G - 1 : k);
    src_o[d] = on ? lane * D + d : 0;      // my d-th own edge
    src_r[d] = on ? k * D + d : 0;         // the edge whose copy sits in my slot d
    oth_r[d] = k;
    // Cross-lane reads stay outside any lane-dependent condition: a lane that
    // is masked off would otherwise read as zero.
    const int other = bpermute(erep, src_o[d]);
    const float mine_w = bpermute(w, src_o[d]), copy_w = bpermute(w, src_r[d]);
    oth_o[d] = on ? other : -1;
    oth_r[d] = on ? k : -1;
    w_o[d] = on ? mine_w : 0.0f;
    w_r[d] = on ? copy_w : 0.0f;
  }
  // b_i = -(load of the experts that cannot move), minilp.cu:223-234; T lanes per rank.
  float part = 0.0f;
  {
    const int r = lane / T, sub = lane % T;
    if (r < G)
      for (int j = sub; j < a.n_fixed; j += T)
        part += norm_count(p2l[r * P + D * C + j]);
    if (T >= 2) part += dpp<kQuadSwap1>(part);
    if (T >= 4) part += dpp<kQuadSwap2>(part);
    if (T >= 8) part += dpp<kHalfMirror>(part);
  }
  const float part_of_rank = bpermute(part, (lane * T) & (kWave - 1));
  const float b = is_rank ? -part_of_rank : 0.0f;
  // Big-M column, minilp.cu:275-281: b_i minus the other entries of row i.
  float m = b;
#pragma unroll
  for (int d = 0; d < DM; ++d)
    m -= w_o[d];
#pragma unroll
  for (int d = 0; d < DM; ++d)
    m -= w_r[d];
  m = (m - 1.0f) + 1.0f;
  if (!is_rank)
    m = 0.0f;

  // ---- affine scaling ----
  float xo = 1.0f, xr = 1.0f, xs = 1.0f, xt = 1.0f, xM = 1.0f;
  float d_max = 0.0f;
  const int NV = 2 * n + G + 2;
  const int win_lo = a.step_rule == LPLB_STEP_REFERENCE_WINDOW ? (NV > 32 ? NV - 32 : 0) : 0;
  const bool with_zero = a.step_rule != LPLB_STEP_REFERENCE_WINDOW || NV < 32;

  for (int step = 0; step < a.n_steps; ++step) {
    const float so = xo * xo, sr = xr * xr, ss = xs * xs, st = xt * xt, sM = xM * xM;
    const float u = is_edge ? 1.0f / (so + sr) : 0.0f;
    const float lam = w * w * so * sr * u;
    const float ao = w * so * u, ar = w * sr * u;
    const float sigma = reduce_sum(u);
    const float kappa = sM / (1.0f + sM * sigma);

    float q = 0.0f;
    double diag = (double)ss;
    double lam_o[DM], lam_r[DM];
#pragma unroll
    for (int d = 0; d < DM; ++d) {
      const float qo = bpermute(ao, src_o[d]), qr = bpermute(ar, src_r[d]);
      const float lo = bpermute(lam, src_o[d]), lr = bpermute(lam, src_r[d]);
      const bool on = oth_o[d] >= 0;
      q += on ? qo + qr : 0.0f;
      lam_o[d] = on ? (double)lo : 0.0;
      lam_r[d] = on ? (double)lr : 0.0;
      diag += lam_o[d] + lam_r[d];
    }
    const float v = is_rank ? m + q : 0.0f;

    // Row `lane` of S and its right-hand side, fp64.
    double S[GM];
    const double dk = (double)kappa, dv = (double)v, dst = (double)st;
#pragma unroll
    for (int c = 0; c < GM; ++c) {
      double s = dst + dk * dv * (double)readlane(v, c);
#pragma unroll
      for (int d = 0; d < DM; ++d) {
        s -= (oth_o[d] == c) ? lam_o[d] : 0.0;
        s -= (oth_r[d] == c) ? lam_r[d] : 0.0;
      }
      s += (lane == c) ? diag : 0.0;
      S[c] = s;
    }
    double rhs = 1000.0 * dk * dv - dst;

    // Cholesky S = L L^T with the forward substitution folded in.
    double fwd = 0.0, my_rinv = 0.0;
#pragma unroll
    for (int c = 0; c < GM; ++c) {
      if (c < G) {
        const double rinv = rsqrt_f64(readlane(S[c], c));
        const double lc = S[c] * rinv;           // L[lane][c]
        if (lane < GM)
          lt_buf[c * LS + lane] = lc;
        const double fc = readlane(rhs, c) * rinv;
        if (lane == c) {
          fwd = fc;
          my_rinv = rinv;
        }
        rhs -= lc * fc;
#pragma unroll
        for (int c2 = c + 1; c2 < GM; ++c2)
          if (c2 < G)
            S[c2] -= lc * readlane(lc, c2);
      }
    }
    __builtin_amdgcn_wave_barrier();
    // Lane c now takes column c of L.
    double LT[GM];
#pragma unroll
    for (int i = 0; i < GM; ++i)
      LT[i] = (lane < GM) ? lt_buf[lane * LS + i] : 0.0;
    __builtin_amdgcn_wave_barrier();
    double acc = fwd, yd = 0.0;
#pragma unroll
    for (int i = GM - 1; i >= 0; --i) {
      if (i < G) {
        const double yi = readlane(acc * my_rinv, i);
        if (lane == i)
          yd = yi;
        acc -= LT[i] * yi;
      }
    }
    const float y = is_rank ? (float)yd : 0.0f;

    // r = A^T w and the direction d = x (c - r); the edge part of w is
    // z = u (h - kappa u.h + kappa (m.y - 1000)), h = -B^T y.
    const float yk = bpermute(y, ek), yrep = bpermute(y, erep);
    const float hp = -w * (so * yk + sr * yrep);
    const float my = reduce_sum(m * y);
    const float sumy = reduce_sum(y);
    const float uh = reduce_sum(u * hp);
    const float z = u * (hp - kappa * uh + kappa * (my - 1000.0f));
    const float sumz = reduce_sum(z);
    const float d_o = -xo * (w * yk + z);
    const float d_r = -xr * (w * yrep + z);
    const float d_s = -xs * y;
    const float d_t = xt * (1.0f + sumy);
    const float d_M = xM * (1000.0f - (my - sumz));

    // Step length, minilp.cu:354-362.  NaN marks "not in the window".
    float cand = __builtin_nanf("");
    if (is_edge && lane >= win_lo)
      cand = fmaxf(cand, d_o);
    if (is_edge && n + lane >= win_lo)
      cand = fmaxf(cand, d_r);
    if (is_rank && 2 * n + lane >= win_lo)
      cand = fmaxf(cand, d_s);
    if (lane == 0)
      cand = fmaxf(fmaxf(cand, d_t), d_M);
    d_max = reduce_max(cand);
    if (with_zero)
      d_max = fmaxf(d_max, 0.0f);
    const float alpha = (float)(0.999 / (double)d_max);
    xo *= 1.0f - alpha * d_o;
    xr *= 1.0f - alpha * d_r;
    xs *= 1.0f - alpha * d_s;
    xt *= 1.0f - alpha * d_t;
    xM *= 1.0f - alpha * d_M;
  }

  // Feasibility, minilp.cu:369-385.
  float res = 0.0f;
  {
    float row = xs - xt + m * xM - b;
#pragma unroll
    for (int d = 0; d < DM; ++d) {
      const float a_o = bpermute(xo, src_o[d]), a_r = bpermute(xr, src_r[d]);
      row += w_o[d] * a_o + w_r[d] * a_r;
    }
    if (is_rank)
      res = fmaxf(res, fabsf(row));
    if (is_edge)
      res = fmaxf(res, fabsf(xo + xr - xM - 1.0f));
    res = reduce_max(res);
  }
  const bool ok = (double)d_max < 0.1 && 0.0 <= (double)xM && (double)xM < 1e-4 &&
                  (double)res < 0.05;
  if (lane == 0 && ok)
    atomicAdd(a.avail, 1);
  if (is_edge)
    a.result[(int64_t)blockIdx.x * n + lane] = ok ? xo : 0.5f;
}

template <int GM, int DM> static void launch(const SolveArgs &a, int n_waves, hipStream_t s) {
  hipLaunchKernelGGL((solve_groups<GM, DM>), dim3(n_waves), dim3(kWave), 0, s, a);
}

static int dispatch(const SolveArgs &a, int n_waves, hipStream_t s) {
  const int G = a.G, D = a.D;
#define LPLB_CASE(GM, DM)                                                      \
  if (G <= GM && D <= DM) {                                                    \
    launch<GM, DM>(a, n_waves, s);                                             \
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
  LPLB_REQUIRE(group_size * dup_per_rank <= kWave, LPLB_EUNSUPPORTED,
               "solve: group_size*dup_per_rank=%d exceeds the 64 edges one wave holds",
               group_size * dup_per_rank);
  const int64_t L = (int64_t)dup_per_rank * n_experts_per_var + n_experts_fixed;
  const int64_t n_experts = (int64_t)n_group * group_size * L;
  LPLB_REQUIRE(n_experts > 0 && n_experts <= (1 << 24) && (int64_t)n_instances * n_group <= INT32_MAX,
               LPLB_EINVAL, "solve: %lld experts x %d instances out of range",
               (long long)n_experts, n_instances);
  SolveArgs a;
  a.workload = workloads; a.gw_out = global_workloads; a.r2o = r2o; a.phy2log = phy2log;
  a.avail = avail_num; a.result = results; a.n_group = n_group; a.G = group_size;
  a.D = dup_per_rank; a.C = n_experts_per_var; a.n_fixed = n_experts_fixed;
  a.n_experts = (int)n_experts; a.step_rule = step_rule; a.n_steps = n_steps;
  int rc = dispatch(a, n_instances * n_group, static_cast<hipStream_t>(stream));
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
