"""HIP path vs the CPU oracle on the same seeded inputs (needs an MI355X).

Bars: histogram, prefix and redirect are bit-exact; the LP result must give an
objective (max rank load) within 1e-3 relative and edge flows within 1e-4 of the
total token count of the oracle's, which follows the reference's fp32 arithmetic.
"""
import numpy as np
import pytest
import torch

from lplb_amd import Planner, synth, topology
from lplb_amd._native import CompiledSolver
from oracle import oracle
from tests.helpers import CASE_SEED, REFERENCE_SOLVE_CASES, Shape, reference_style_case

pytestmark = pytest.mark.gpu

OBJ_RTOL = 1e-3      # objective, relative
FLOW_TOL = 1e-4      # edge flows, relative to the total token count


def dev(a, cuda, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(cuda)


def solver_for(s: Shape) -> CompiledSolver:
    return CompiledSolver(s.n_group, s.G, s.D, s.P, s.C)


# ----------------------------------------------------------------- histogram
@pytest.mark.parametrize("n,n_experts,n_sms", [
    (4096 * 8, 256, 256), (65536, 256, 100), (0, 256, 8), (1, 32, 4), (255, 32, 3), (257, 32, 3),
    (1000003, 256, 256), (70001, 1000, 37), (65536, 256, 1), (8192 * 8, 256, 304),
    # the LDS histogram is kept in eight copies up to 2016 experts and in one beyond
    (300007, 2016, 64), (300007, 2017, 64), (100003, 5000, 19), (40000, 16384, 5), (99991, 33, 7), (99991, 1000, 256),
])
def test_count_idx_matches_oracle(cuda, n, n_experts, n_sms):
    rng = np.random.default_rng(n + n_experts + n_sms)
    idx = rng.integers(-1, n_experts, size=n, dtype=np.int64)
    if n > 1000:
        idx[n // 5:n // 2] = n_experts // 3          # a hot expert: whole waves on one counter
    solver = CompiledSolver(1, 1, 1, n_experts + 1, 1)   # n_experts logical experts
    assert solver.n_experts == n_experts
    total, by_sm = solver.count_idx(dev(idx, cuda), n_sms)
    torch.cuda.synchronize()
    want = oracle.count_idx(idx, n_experts, n_sms)
    assert by_sm.shape == (n_sms, n_experts) and by_sm.dtype == torch.int32
    np.testing.assert_array_equal(by_sm.cpu().numpy(), want)
    # properties the reference's own test checks (tests/test_idx_processing.py:36-48)
    assert total.shape == (n_experts,)
    assert int(total.min()) >= 0
    assert int(total.sum()) == int((idx != -1).sum())
    np.testing.assert_array_equal(total.cpu().numpy(), np.bincount(idx[idx >= 0], minlength=n_experts))


# ------------------------------------------------------------------ redirect
def _random_weights(shape: Shape, rng):
    w = rng.standard_normal((shape.n_group, shape.G, shape.D)) / 3 + 0.5
    return np.clip(w, 0, 1).astype(np.float32)


@pytest.mark.parametrize("n,n_experts,offset", [(65536, 256, 0), (65537, 256, 1), (4099, 30, 0), (1, 7, 0), (0, 64, 0),
                                                (131072, 256, 1), (100000, 2017, 0), (70000, 16384, 2), (8193, 5, 0)])
def test_count_totals_add_swaps_two_vectors(cuda, n, n_experts, offset):
    """lplb_count_totals_add: the batch's counts are added to a zeroed vector and the other vector comes back
    zeroed, call after call with the two swapped; a second call into the same vector adds to what is there.
    Masked and out-of-range values, odd lengths, views at an odd multiple of 8 bytes, one and eight LDS copies."""
    rng = np.random.default_rng(n + n_experts)
    solver = CompiledSolver(1, 1, 1, n_experts + 1, 1)
    assert solver.n_experts == n_experts
    pair = [torch.zeros(n_experts, dtype=torch.int32, device=cuda),
            torch.full((n_experts,), 77, dtype=torch.int32, device=cuda)]       # (the other one starts dirty)
    turn = 0
    for call in range(3):
        host = rng.integers(-1, n_experts, size=n + offset).astype(np.int64)
        if n > 10:
            host[offset + 3] = n_experts          # out of range: not counted
            host[offset + 7] = -5
            host[offset + 5:offset + 5 + n // 3] = (call * 7) % n_experts      # a hot expert
        want = np.bincount(host[offset:][(host[offset:] >= 0) & (host[offset:] < n_experts)], minlength=n_experts)
        got = solver.count_totals_add(dev(host, cuda)[offset:], pair[turn], clear=pair[1 - turn])
        torch.cuda.synchronize()
        assert got is pair[turn]
        np.testing.assert_array_equal(got.cpu().numpy(), want)
        assert int(pair[1 - turn].abs().max()) == 0
        if call == 2:                             # once more into the same vector: the counts double
            solver.count_totals_add(dev(host, cuda)[offset:], pair[turn])
            np.testing.assert_array_equal(pair[turn].cpu().numpy(), 2 * want)
        turn = 1 - turn


@pytest.mark.parametrize("n,n_experts,offset", [(65536, 256, 0), (65537, 256, 1), (4099, 30, 0), (1, 7, 0), (0, 64, 0),
                                                (131072, 1024, 3), (2, 3, 1), (50000, 257, 0)])
def test_count_totals_matches_oracle(cuda, n, n_experts, offset):
    """The one-launch totals (what Planner.run feeds the all-reduce with) equal the last row of the table, for
    masked and out-of-range values, odd lengths, and views that start at an odd multiple of 8 bytes."""
    rng = np.random.default_rng(n + n_experts)
    host = rng.integers(-1, n_experts, size=n + offset).astype(np.int64)
    if n > 10:
        host[offset + 3] = n_experts          # out of range: not counted
        host[offset + 7] = -5
        host[offset + 5:offset + 5 + n // 3] = n_experts - 1      # a hot expert, the last one
    from lplb_amd._native import CompiledSolver, load
    lib = load()
    d_idx = dev(host, cuda)[offset:]
    totals = torch.full((n_experts,), -9, dtype=torch.int32, device=cuda)
    rc = lib.lplb_count_totals(d_idx.data_ptr(), n, n_experts, totals.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.lplb_last_error()
    want = oracle.count_idx(host[offset:], n_experts, 4)[-1]
    np.testing.assert_array_equal(totals.cpu().numpy(), want)
    # beyond what it serves it refuses (the caller then runs histogram and scan)
    some = torch.zeros(2, dtype=torch.int64, device=cuda)
    assert lib.lplb_count_totals(some.data_ptr(), (1 << 17) + 2, n_experts, totals.data_ptr(), None) == 2
    assert lib.lplb_count_totals(some.data_ptr(), 2, 1025, totals.data_ptr(), None) == 2


@pytest.mark.parametrize("case", ["cube8_ep32", "cube8_ep32_c2", "ring8_ep32", "hypercube16", "torus8x4"])
@pytest.mark.parametrize("n,n_sms", [(65536, 256), (4099, 7), (300, 256), (1 << 20, 256)])
def test_map_idx_matches_oracle(cuda, case, n, n_sms):
    name, r2o, nl, ep, red, reorder, _ = next(c for c in REFERENCE_SOLVE_CASES if c[0] == case)
    shape, _, phy2log, log2phy, _ = reference_style_case(r2o, nl, ep, red, True, seed=7)
    rng = np.random.default_rng(n * 31 + n_sms)
    idx = rng.integers(-1, nl, size=n, dtype=np.int64)
    o_weight = _random_weights(shape, rng)
    solver = solver_for(shape)
    d_idx = dev(idx, cuda)
    _, by_sm = solver.count_idx(d_idx, n_sms)
    phys = torch.full((shape.n_physical,), -7, dtype=torch.int32, device=cuda)
    out = solver.map_idx(d_idx, dev(o_weight, cuda), by_sm, dev(shape.o2r, cuda), dev(phy2log, cuda), n_sms,
                         physical_counts=phys)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = oracle.map_idx(idx, o_weight, by_sm.cpu().numpy(), shape.o2r, phy2log, shape.n_group, shape.C, shape.P)
    np.testing.assert_array_equal(got, want)
    # tokens per physical expert, as the reference's test counts them (tests/test_idx_processing.py:100-101)
    np.testing.assert_array_equal(phys.cpu().numpy(), np.bincount(want[want >= 0], minlength=shape.n_physical))
    # the same through a table prepared once for the mapping
    table = solver.prepare_mapping(dev(shape.o2r, cuda), dev(phy2log, cuda))
    phys2 = torch.full((shape.n_physical,), -7, dtype=torch.int32, device=cuda)
    out2 = solver.map_idx(d_idx, dev(o_weight, cuda), by_sm, dev(shape.o2r, cuda), dev(phy2log, cuda), n_sms,
                          physical_counts=phys2, prepared=table)
    np.testing.assert_array_equal(out2.cpu().numpy(), want)
    np.testing.assert_array_equal(phys2.cpu().numpy(), phys.cpu().numpy())
    # reference test's properties (tests/test_idx_processing.py:88-98)
    assert got.min() >= -1 and got.max() < shape.n_physical
    assert np.array_equal(got == -1, idx == -1)
    padded = np.concatenate([np.full((1, 2), -1, np.int32), log2phy])
    assert np.all((got == padded[idx + 1, 0]) | (got == padded[idx + 1, 1]))
    # conservation
    assert np.bincount(got[got >= 0], minlength=shape.n_physical).sum() == (idx != -1).sum()


def test_map_idx_is_independent_of_slicing(cuda):
    shape, _, phy2log, _, _ = reference_style_case(*REFERENCE_SOLVE_CASES[0][1:6], seed=3)
    rng = np.random.default_rng(5)
    idx = rng.integers(-1, shape.n_logical, size=50000, dtype=np.int64)
    o_weight = _random_weights(shape, rng)
    solver = solver_for(shape)
    outs = []
    for n_sms in (1, 13, 256):
        d_idx = dev(idx, cuda)
        _, by_sm = solver.count_idx(d_idx, n_sms)
        outs.append(solver.map_idx(d_idx, dev(o_weight, cuda), by_sm, dev(shape.o2r, cuda), dev(phy2log, cuda),
                                   n_sms).cpu().numpy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_map_idx_extreme_weights(cuda):
    """o_weight outside [0, 1] and NaN: everything to the replica / original, nothing lost."""
    shape, _, phy2log, _, _ = reference_style_case(*REFERENCE_SOLVE_CASES[0][1:6], seed=3)
    rng = np.random.default_rng(11)
    idx = rng.integers(-1, shape.n_logical, size=20000, dtype=np.int64)
    o_weight = rng.choice(np.array([-1.5, 0.0, 0.3, 1.0, 2.5, np.nan, 1e30, -1e30], np.float32),
                          size=(shape.n_group, shape.G, shape.D))
    solver = solver_for(shape)
    d_idx = dev(idx, cuda)
    _, by_sm = solver.count_idx(d_idx, 64)
    phys = torch.empty(shape.n_physical, dtype=torch.int32, device=cuda)
    got = solver.map_idx(d_idx, dev(o_weight, cuda), by_sm, dev(shape.o2r, cuda), dev(phy2log, cuda), 64,
                         physical_counts=phys).cpu().numpy()
    want = oracle.map_idx(idx, o_weight, by_sm.cpu().numpy(), shape.o2r, phy2log, shape.n_group, shape.C, shape.P)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(phys.cpu().numpy(), np.bincount(want[want >= 0], minlength=shape.n_physical))
    table = solver.prepare_mapping(dev(shape.o2r, cuda), dev(phy2log, cuda))
    got = solver.map_idx(d_idx, dev(o_weight, cuda), by_sm, dev(shape.o2r, cuda), dev(phy2log, cuda), 64,
                         prepared=table).cpu().numpy()
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("multiple", [1, 2, 7])
def test_physical_counts_when_499_divides_a_total(cuda, multiple):
    """The per-expert hash (499 k + 41) mod total is a bijection unless 499 divides total; then it takes
    total / 499 values 499 times each and the closed form of the counts changes."""
    name, r2o, nl, ep, red, reorder, _ = REFERENCE_SOLVE_CASES[0]
    shape, _, phy2log, _, _ = reference_style_case(r2o, nl, ep, red, True, seed=7)
    rng = np.random.default_rng(multiple)
    replicated = [int(phy2log[r * shape.P + s]) for r in range(ep) for s in range(shape.C * shape.D)]
    counts = rng.integers(1, 300, size=nl)
    counts[replicated[:6]] = 499 * multiple            # replicated experts with degenerate totals
    counts[replicated[6]] = 499 * multiple + 1
    idx = rng.permutation(np.repeat(np.arange(nl, dtype=np.int64), counts))
    solver = solver_for(shape)
    d_idx = dev(idx, cuda)
    _, by_sm = solver.count_idx(d_idx, 32)
    for trial in range(4):
        o_weight = rng.uniform(0, 1, size=(shape.n_group, shape.G, shape.D)).astype(np.float32)
        if trial == 0:
            o_weight[:] = 41.0 / (499 * multiple)      # expected = 41 (or 40): the first hash value is 41
        phys = torch.empty(shape.n_physical, dtype=torch.int32, device=cuda)
        table = solver.prepare_mapping(dev(shape.o2r, cuda), dev(phy2log, cuda)) if trial % 2 else None
        got = solver.map_idx(d_idx, dev(o_weight, cuda), by_sm, dev(shape.o2r, cuda), dev(phy2log, cuda), 32,
                             physical_counts=phys, prepared=table).cpu().numpy()
        want = oracle.map_idx(idx, o_weight, by_sm.cpu().numpy(), shape.o2r, phy2log, shape.n_group, shape.C, shape.P)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(phys.cpu().numpy(), np.bincount(want[want >= 0], minlength=shape.n_physical))


def test_count_and_redirect_random_shapes(cuda):
    """Forty seeded draws of batch length, slice count, topology and weights: histogram table and
    redirected indices bit-exact against the oracle, counts per physical expert against its bincount."""
    from lplb_amd import topology
    from lplb_amd.mapping import build_redundancy_mapping
    rng = np.random.default_rng(2024)
    topologies = [(topology.CUBE_8P2E, 1), (topology.RING_8P, 1), (topology.HYPERCUBE_16P2E, 1),
                  (topology.torus_2d(8, 4), 1), (topology.CUBE_8P2E, 4), (_shifted_ring(6, [1, 2]), 2),
                  (_shifted_ring(4, [1, 2, 3]), 3)]
    for trial in range(40):
        r2o, n_group = topologies[int(rng.integers(len(topologies)))]
        r2o = np.asarray(r2o, np.int32)
        g, d = r2o.shape
        ep = g * n_group
        combined = int(rng.integers(1, 3))
        per_rank = d * combined + int(rng.integers(d * combined, 12))       # at least as many as replicas
        n_logical = ep * per_rank
        shape = Shape(r2o, ep, n_logical, n_logical + d * combined * ep)
        hist = rng.integers(1, 1 << 20, size=n_logical).astype(np.int64)
        phy2log, _, _ = build_redundancy_mapping(r2o, ep, n_logical, shape.n_physical, hist, n_nodes=1)
        n = int(rng.choice([0, 1, 63, 64, 65, 255, 256, 257, 1000, 4097, 70000, 300001]))
        n_sms = int(rng.choice([1, 2, 3, 17, 64, 255, 256, 304, 700]))
        idx = rng.integers(-1, n_logical, size=n, dtype=np.int64)
        if n and trial % 5 == 0:
            idx[rng.integers(0, n, size=max(1, n // 50))] = n_logical + int(rng.integers(0, 5))   # out of range
        o_weight = _random_weights(shape, rng)
        solver = solver_for(shape)
        d_idx = dev(idx, cuda)
        total, by_sm = solver.count_idx(d_idx, n_sms)
        want_by = oracle.count_idx(idx, n_logical, n_sms)
        np.testing.assert_array_equal(by_sm.cpu().numpy(), want_by, err_msg=f"trial {trial}")
        phys = torch.full((shape.n_physical,), -3, dtype=torch.int32, device=cuda)
        table = solver.prepare_mapping(dev(shape.o2r, cuda), dev(phy2log, cuda)) if trial % 2 else None
        got = solver.map_idx(d_idx, dev(o_weight, cuda), by_sm, dev(shape.o2r, cuda), dev(phy2log, cuda), n_sms,
                             physical_counts=phys, prepared=table).cpu().numpy()
        want = oracle.map_idx(idx, o_weight, want_by, shape.o2r, phy2log, shape.n_group, shape.C, shape.P)
        np.testing.assert_array_equal(got, want, err_msg=f"trial {trial}")
        np.testing.assert_array_equal(phys.cpu().numpy(), np.bincount(want[want >= 0], minlength=shape.n_physical),
                                      err_msg=f"trial {trial}")


# -------------------------------------------------------------------- solver

def _why_flags_may_differ(wl, r2o, phy2log, n_group, C, n_fixed, step_rule=0):
    """The feasibility test compares three quantities with fixed thresholds (minilp.cu:381-382):
    the last step's d_max < 0.1, 0 <= x_M < 1e-4 and the residual < 0.05.  Two correct evaluations
    of the same algorithm can only disagree on the flag of a group when one of them is within
    rounding reach of its threshold.  Returns, per group, the quantities that lie within 10 % of
    a threshold in the fp64 evaluation (for the lower bound 0 of x_M: |x_M| below 1e-5, the
    absolute counterpart), or 'not finite'; an empty list means the flag is not in doubt."""
    _, _, _, x, trace, resid = oracle.solve(wl, r2o, phy2log, n_group, C, n_fixed, precision=64, details=True,
                                            step_rule=step_rule)
    out = []
    for g in range(n_group):
        d_max, x_m, res = float(trace[g, -1, 0]), float(x[g, -1]), float(resid[g])
        near = []
        if not np.isfinite([d_max, x_m, res]).all():
            near.append("not finite")
        if abs(d_max - 0.1) <= 0.01:
            near.append(f"d_max={d_max:.4g}")
        if abs(x_m - 1e-4) <= 1e-5 or abs(x_m) <= 1e-5:
            near.append(f"x_M={x_m:.3g}")
        if abs(res - 0.05) <= 0.005:
            near.append(f"residual={res:.4g}")
        out.append(near)
    return out

def _compare_solve(shape, phy2log, workload, res, gw, avail, step_rule=0, n_steps=5):
    o_res, o_gw, o_avail = oracle.solve(workload, shape.r2o, phy2log, shape.n_group, shape.C, shape.n_fixed,
                                        step_rule=step_rule, n_steps=n_steps)
    o64, _, _ = oracle.solve(workload, shape.r2o, phy2log, shape.n_group, shape.C, shape.n_fixed,
                             step_rule=step_rule, n_steps=n_steps, precision=64)
    np.testing.assert_array_equal(gw.reshape(-1), o_gw)          # fp32 divide, bit-exact
    assert avail == o_avail
    total = float(np.sum(workload, dtype=np.float64))
    args = (shape.r2o, phy2log, shape.n_group, shape.C)
    out = {}
    for tag, ref in (("f32", o_res), ("f64", o64)):
        flow = np.abs(oracle.edge_flows(workload, res, *args) - oracle.edge_flows(workload, ref, *args)).max() / total
        obj_ref = oracle.rank_loads(workload, ref, *args).max(axis=1)
        obj = oracle.rank_loads(workload, res, *args).max(axis=1)
        out[tag] = (flow, (np.abs(obj - obj_ref) / obj_ref).max(), np.abs(res - ref).max())
    print(f"  flow/obj/p diff vs oracle f32 {out['f32']}, vs f64 {out['f64']}")
    assert out["f32"][0] <= FLOW_TOL and out["f32"][1] <= OBJ_RTOL
    return out


@pytest.mark.parametrize("case", REFERENCE_SOLVE_CASES, ids=[c[0] for c in REFERENCE_SOLVE_CASES])
def test_solve_reference_cases(cuda, case):
    """The reference's solver test (tests/test_solve.py:13-89) plus parity with the oracle."""
    name, r2o, nl, ep, red, reorder, tol = case
    shape, hist, phy2log, _, workload = reference_style_case(r2o, nl, ep, red, reorder, seed=CASE_SEED[name])
    planner = Planner(torch.from_numpy(shape.r2o), shape.n_physical, nl, ep, gpus_per_node=8)
    got_p2l, _, _ = planner.update_redundancy_mapping(None if hist is None else torch.from_numpy(hist))
    np.testing.assert_array_equal(got_p2l.cpu().numpy(), phy2log)
    avail = torch.zeros((), dtype=torch.int32, device=cuda)
    probs, gw = planner.solve_probs(dev(workload, cuda), avail)
    torch.cuda.synchronize()
    assert probs.shape == (shape.n_group, shape.G, shape.D) and probs.dtype == torch.float32
    assert int(avail) == planner.n_group
    res = probs.cpu().numpy()
    loads = oracle.rank_loads(workload, res, shape.r2o, phy2log, shape.n_group, shape.C)
    balance = loads.max() / loads.mean()
    print(f"{name}: balance {balance:.4f} (tolerance {tol})")
    assert balance < tol
    _compare_solve(shape, phy2log, workload, res, gw.cpu().numpy(), int(avail))


@pytest.mark.parametrize("cfg", ["cpu_ref_ep8", "v3_ep8_cube", "ep16_hypercube", "ep32_torus"])
@pytest.mark.parametrize("step_rule", [0, 1])
def test_solve_benchmark_configs(cuda, cfg, step_rule):
    inp = synth.make_inputs(cfg, tokens=64)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    solver = solver_for(shape)
    solver.step_rule = step_rule
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    wl = dev(inp.global_counts.reshape(shape.n_group, shape.G, shape.L), cuda)
    res, gw = solver.solve(wl, dev(shape.r2o, cuda), dev(inp.phy2log, cuda), avail)
    torch.cuda.synchronize()
    _compare_solve(shape, inp.phy2log, inp.global_counts, res.cpu().numpy(), gw.cpu().numpy(), int(avail[0]),
                   step_rule=step_rule)


@pytest.mark.parametrize("topo", ["cube8", "ring8", "hyper16", "torus32"])
def test_solve_adversarial_distributions(cuda, topo):
    """Skewed, sparse, one-hot and nearly uniform count vectors, small and large totals.  On such inputs the
    dense fp32 evaluation of the reference algorithm is itself up to 2e-4 (flows) / 1.3e-3 (objective) away
    from its fp64 evaluation, so the yardstick here is the fp64 oracle: the GPU result (fp32 with an fp64
    normal-equation solve) must be within the stated tolerances of it, and agree on feasibility."""
    from lplb_amd import topology
    from lplb_amd.mapping import build_redundancy_mapping
    r2o, ep = {"cube8": (topology.CUBE_8P2E, 8), "ring8": (topology.RING_8P, 8),
               "hyper16": (topology.HYPERCUBE_16P2E, 16), "torus32": (topology.torus_2d(8, 4), 32)}[topo]
    r2o = np.asarray(r2o, np.int32)
    nl = 256
    shape = Shape(r2o, ep, nl, nl + r2o.shape[1] * ep)
    solver = solver_for(shape)
    rng = np.random.default_rng(99)

    def draw(kind):
        ranks = np.arange(1, nl + 1)
        p = {"zipf1": 1.0 / ranks, "zipf2": 1.0 / ranks ** 2.0, "lognorm": rng.lognormal(0, 1.0, nl),
             "near_uniform": 1 + rng.normal(0, 0.01, nl), "sparse": rng.random(nl) * (rng.random(nl) < 0.2) + 1e-6,
             "one_hot": np.where(np.arange(nl) == rng.integers(nl), 1.0, 1e-3)}[kind]
        p = rng.permutation(np.abs(p))
        return rng.multinomial(int(rng.choice([1000, 65536, 1 << 22])), p / p.sum()).astype(np.int32)

    flags_differ = checked = 0
    skipped = []
    worst = [0.0, 0.0]
    for kind in ("zipf1", "zipf2", "lognorm", "near_uniform", "sparse", "one_hot"):
        for _ in range(8):
            hist = rng.integers(1, 1 << 20, size=nl)
            phy2log, _, _ = build_redundancy_mapping(r2o, ep, nl, shape.n_physical, hist, n_nodes=1)
            wl = draw(kind)
            avail = torch.zeros(1, dtype=torch.int32, device=cuda)
            res, gw = solver.solve(dev(wl.reshape(shape.n_group, shape.G, shape.L), cuda), dev(r2o, cuda),
                                   dev(phy2log, cuda), avail)
            res = res.cpu().numpy()
            o64, o_gw, o_avail = oracle.solve(wl, r2o, phy2log, shape.n_group, shape.C, shape.n_fixed, precision=64)
            np.testing.assert_array_equal(gw.cpu().numpy().reshape(-1), o_gw)
            if int(avail[0]) != o_avail:
                # allowed only where the fp64 evaluation itself sits on a threshold
                why = _why_flags_may_differ(wl, r2o, phy2log, shape.n_group, shape.C, shape.n_fixed)
                assert any(why), f"{topo}/{kind}: feasible on GPU {int(avail[0])}, fp64 oracle {o_avail}, no quantity near a threshold"
                skipped.append(f"{kind}: flags differ ({int(avail[0])} vs {o_avail}), {why}")
                flags_differ += 1
                continue
            if o_avail != shape.n_group:
                assert np.all(res == 0.5)
                skipped.append(f"{kind}: infeasible in both evaluations, neutral split returned")
                continue
            args = (r2o, phy2log, shape.n_group, shape.C)
            flow = np.abs(oracle.edge_flows(wl, res, *args) - oracle.edge_flows(wl, o64, *args)).max() / float(wl.sum())
            obj, obj64 = (oracle.rank_loads(wl, x, *args).max(axis=1) for x in (res, o64))
            worst = [max(worst[0], flow), max(worst[1], float((np.abs(obj - obj64) / obj64).max()))]
            checked += 1
    print(f"{topo}: {checked} compared, worst flow {worst[0]:.1e} objective {worst[1]:.1e}, feasibility differs in {flags_differ}")
    for line in skipped:
        print("  not compared:", line)
    assert worst[0] <= FLOW_TOL and worst[1] <= OBJ_RTOL
    # of 48 inputs per topology: at most 2 threshold cases, at most 8 without flows to compare
    assert flags_differ <= 2 and len(skipped) <= 8 and checked >= 40


@pytest.mark.gpu
@pytest.mark.parametrize("G,D,C,n_group", [(3, 1, 1, 1), (5, 2, 1, 3), (6, 3, 2, 1), (7, 4, 1, 2), (8, 8, 1, 1),
                                           (10, 6, 1, 1), (12, 2, 3, 2), (12, 5, 1, 1), (16, 4, 1, 1), (21, 3, 1, 1),
                                           (24, 2, 1, 2), (32, 2, 2, 1), (40, 1, 1, 1), (64, 1, 1, 1),
                                           # 65..128 replica edges or more than 8 slots per rank: two edges per lane
                                           (16, 5, 1, 1), (12, 6, 1, 2), (8, 9, 1, 1), (8, 12, 1, 1), (10, 8, 2, 1),
                                           (4, 12, 1, 1), (16, 8, 1, 1), (11, 9, 1, 1), (32, 3, 1, 1), (32, 4, 1, 1),
                                           (24, 4, 1, 1), (64, 2, 1, 1), (48, 2, 1, 1), (8, 16, 1, 1), (20, 6, 1, 1), (17, 7, 1, 1),
                                           (33, 3, 1, 1), (42, 3, 1, 1)])
def test_solve_random_topologies(cuda, G, D, C, n_group):
    """Replica topologies that are no named graph: every column of r2o is a random permutation
    (self-loops included), group sizes that do not fill the kernels' register arrays (padded
    instantiations), several replicated experts per slot.  Yardstick: the fp64 oracle."""
    rng = np.random.default_rng(1000 * G + 10 * D + C)
    r2o = np.stack([rng.permutation(G) for _ in range(D)], axis=1).astype(np.int32)
    ep = G * n_group
    per_rank = D * C + int(rng.integers(0, 5))
    nl = ep * per_rank
    shape = Shape(r2o, ep, nl, nl + D * C * ep)
    assert (shape.C, shape.n_fixed) == (C, per_rank - D * C)
    solver = solver_for(shape)
    compared = 0
    skipped = []
    for trial in range(6):
        # any assignment of logical experts to slots is a legal phy2log layout: originals are a
        # permutation, replica slot (rank, c*D+d) copies slot c*D+d of rank r2o[rank][d]
        originals = rng.permutation(nl).reshape(ep, per_rank)
        phy2log = np.empty((ep, shape.P), np.int32)
        phy2log[:, :per_rank] = originals
        for rank in range(ep):
            g0 = rank // G * G
            for c in range(C):
                for d in range(D):
                    phy2log[rank, per_rank + c * D + d] = originals[g0 + r2o[rank % G, d], c * D + d]
        phy2log = phy2log.reshape(-1)
        p = rng.dirichlet(np.full(nl, [0.3, 1.0, 5.0][trial % 3]))
        wl = rng.multinomial(int(rng.choice([2000, 1 << 17, 1 << 22])), p).astype(np.int32)
        wl[rng.integers(nl)] += 1          # never all zero
        avail = torch.zeros(1, dtype=torch.int32, device=cuda)
        res, gw = solver.solve(dev(wl.reshape(n_group, G, per_rank), cuda), dev(r2o, cuda), dev(phy2log, cuda), avail)
        res = res.cpu().numpy()
        o64, o_gw, o_avail = oracle.solve(wl, r2o, phy2log, n_group, C, shape.n_fixed, precision=64)
        np.testing.assert_array_equal(gw.cpu().numpy().reshape(-1), o_gw)
        if int(avail[0]) != o_avail:
            # allowed only where the fp64 evaluation itself sits on a threshold
            why = _why_flags_may_differ(wl, r2o, phy2log, n_group, C, shape.n_fixed)
            assert any(why), f"trial {trial}: feasible on GPU {int(avail[0])}, fp64 oracle {o_avail}, no quantity near a threshold"
            skipped.append(f"trial {trial}: flags differ ({int(avail[0])} vs {o_avail}), {why}")
            continue
        if o_avail != n_group:
            # some group infeasible in both: it must carry the neutral split, the others are compared below
            failed = [g for g in range(n_group) if np.all(o64[g] == 0.5)]
            assert len(failed) == n_group - o_avail and all(np.all(res[g] == 0.5) for g in failed), trial
            skipped.append(f"trial {trial}: {len(failed)} of {n_group} groups infeasible in both evaluations")
        args = (r2o, phy2log, n_group, C)
        flow = np.abs(oracle.edge_flows(wl, res, *args) - oracle.edge_flows(wl, o64, *args)).max() / float(wl.sum())
        obj, obj64 = (oracle.rank_loads(wl, x, *args).max(axis=1) for x in (res, o64))
        assert flow <= FLOW_TOL and np.all(np.abs(obj - obj64) <= OBJ_RTOL * obj64), (trial, flow)   # a group may be empty
        compared += 1
    for line in skipped:
        print("  note:", line)
    # six draws per topology: at most one may end on a threshold
    assert compared >= 5 and sum("flags differ" in line for line in skipped) <= 1


@pytest.mark.gpu
def test_solve_every_shape_inside_the_limits(cuda):
    """Every (G, D) with G <= 64, D <= 16 and G * D <= 128 finds a kernel (one edge per lane up to 64 edges and
    8 slots per rank, two beyond) and, on one moderately skewed draw each, lands on the fp64 oracle's flows.
    Shapes outside are refused before anything is launched."""
    rng = np.random.default_rng(2024)
    shapes = [(g, d) for g in range(1, 65) for d in range(1, 17) if g * d <= 128]
    compared = 0
    for g, d in shapes:
        r2o = np.stack([rng.permutation(g) for _ in range(d)], axis=1).astype(np.int32)
        per_rank = d + 2
        nl = g * per_rank
        shape = Shape(r2o, g, nl, nl + d * g)
        originals = rng.permutation(nl).reshape(g, per_rank)
        phy2log = np.empty((g, shape.P), np.int32)
        phy2log[:, :per_rank] = originals
        for rank in range(g):
            for k in range(d):
                phy2log[rank, per_rank + k] = originals[r2o[rank, k], k]
        phy2log = phy2log.reshape(-1)
        wl = rng.multinomial(1 << 17, rng.dirichlet(np.full(nl, 1.0))).astype(np.int32)
        wl[rng.integers(nl)] += 1
        avail = torch.zeros(1, dtype=torch.int32, device=cuda)
        res, gw = solver_for(shape).solve(dev(wl.reshape(1, g, per_rank), cuda), dev(r2o, cuda), dev(phy2log, cuda), avail)
        res = res.cpu().numpy()
        o64, o_gw, o_avail = oracle.solve(wl, r2o, phy2log, 1, 1, shape.n_fixed, precision=64)
        np.testing.assert_array_equal(gw.cpu().numpy().reshape(-1), o_gw, err_msg=f"{g} x {d}")
        if int(avail[0]) != o_avail or o_avail != 1:
            continue      # on a threshold, or infeasible in both: the seeded tests above look at those closely
        args = (r2o, phy2log, 1, 1)
        flow = np.abs(oracle.edge_flows(wl, res, *args) - oracle.edge_flows(wl, o64, *args)).max() / float(wl.sum())
        assert flow <= FLOW_TOL, (g, d, flow)
        compared += 1
    assert compared >= 0.9 * len(shapes), (compared, len(shapes))
    for g, d in [(65, 1), (8, 17), (43, 3), (16, 9)]:
        r2o = np.zeros((g, d), np.int32)
        with pytest.raises(RuntimeError):
            solver_for(Shape(r2o, g, g * (d + 1), g * (2 * d + 1))).solve(
                torch.zeros((1, g, d + 1), dtype=torch.int32, device=cuda), dev(r2o, cuda),
                torch.zeros(g * (2 * d + 1), dtype=torch.int32, device=cuda),
                torch.zeros(1, dtype=torch.int32, device=cuda))


def test_solve_window_rule_chaos_regression(cuda):
    """A legal input on which the reference's step rule (d_max over the last 32 columns only,
    minilp.cu:355-359) lets the iterates leave [0, 1] by far: 64 ranks on one random replica
    permutation, 4 194 305 tokens (tests/golden/window_chaos_ring64.json, written by
    make_window_chaos_case.py).  The exact-arithmetic iteration returns shares between -84 and
    +49 and still reports feasible.  In that regime rounding is amplified: the dense fp32
    evaluation ends 2.4e-3 of the tokens away from the fp64 one, beyond the 1e-4 parity
    tolerance, so the tolerance cannot hold against the fp32 oracle here.  Expected
    classification: window-rule chaos; the GPU result (fp64 normal-equation core) is feasible
    like both oracles and lies closer to the fp64 evaluation than the fp32 evaluation does."""
    import json
    from pathlib import Path
    case = json.loads((Path(__file__).parent / "golden" / "window_chaos_ring64.json").read_text())
    r2o = np.asarray(case["r2o"], np.int32).reshape(64, 1)
    phy2log, wl = np.asarray(case["phy2log"], np.int32), np.asarray(case["workload"], np.int32)
    shape = Shape(r2o, 64, 64, 128)
    solver = solver_for(shape)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    res, gw = solver.solve(dev(wl.reshape(1, 64, 1), cuda), dev(r2o, cuda), dev(phy2log, cuda), avail)
    res = res.cpu().numpy()
    o64, o_gw, ok64 = oracle.solve(wl, r2o, phy2log, 1, 1, 0, precision=64)
    o32, _, ok32 = oracle.solve(wl, r2o, phy2log, 1, 1, 0, precision=32)
    np.testing.assert_array_equal(gw.cpu().numpy().reshape(-1), o_gw)
    assert int(avail[0]) == ok64 == ok32 == 1
    assert o64.min() < -50 and o64.max() > 40          # the classification: shares far outside [0, 1]
    args = (r2o, phy2log, 1, 1)
    total = float(wl.sum())
    flows = {k: oracle.edge_flows(wl, v, *args) for k, v in (("gpu", res), ("f64", o64), ("f32", o32))}
    gpu_vs_64 = np.abs(flows["gpu"] - flows["f64"]).max() / total
    f32_vs_64 = np.abs(flows["f32"] - flows["f64"]).max() / total
    print(f"window chaos: GPU {gpu_vs_64:.2e} of the tokens from fp64, fp32 oracle {f32_vs_64:.2e}")
    assert f32_vs_64 > FLOW_TOL              # the fp32 evaluation itself is outside the tolerance
    assert gpu_vs_64 < f32_vs_64 and gpu_vs_64 <= 1e-3
    # with the step taken over all columns the same input is tame and the usual bar holds
    solver.step_rule = 1
    avail.zero_()
    res1, gw1 = solver.solve(dev(wl.reshape(1, 64, 1), cuda), dev(r2o, cuda), dev(phy2log, cuda), avail)
    _compare_solve(shape, phy2log, wl, res1.cpu().numpy(), gw1.cpu().numpy(), int(avail[0]), step_rule=1)
    assert 0 <= res1.min() and res1.max() <= 1


def test_solve_fallback_and_counter(cuda):
    """Infeasible / degenerate LPs give 0.5 everywhere and leave the counter alone;
    the counter accumulates across calls (minilp.cu:379-400)."""
    shape, _, phy2log, _, workload = reference_style_case(*REFERENCE_SOLVE_CASES[0][1:6])
    solver = solver_for(shape)
    args = (dev(shape.r2o, cuda), dev(phy2log, cuda))
    avail = torch.full((1,), 7, dtype=torch.int32, device=cuda)
    zero = torch.zeros((shape.n_group, shape.G, shape.L), dtype=torch.int32, device=cuda)
    res, gw = solver.solve(zero, *args, avail)
    assert torch.all(res == 0.5) and int(avail[0]) == 7
    assert torch.isnan(gw).all()
    solver.n_steps = 1          # one step cannot pass the feasibility test
    res, _ = solver.solve(dev(workload.reshape(zero.shape), cuda), *args, avail)
    assert torch.all(res == 0.5) and int(avail[0]) == 7
    solver.n_steps = 5
    for k in (1, 2):
        res, _ = solver.solve(dev(workload.reshape(zero.shape), cuda), *args, avail)
        assert int(avail[0]) == 7 + k * shape.n_group
    o_res, _, _ = oracle.solve(workload, shape.r2o, phy2log, shape.n_group, shape.C, shape.n_fixed, n_steps=1)
    assert np.all(o_res == 0.5)


def test_solve_batched_matches_single(cuda):
    inp = synth.make_inputs("v3_ep8_cube", tokens=8)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    counts = synth.sweep_counts(64)
    solver = solver_for(shape)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    r2o, p2l = dev(shape.r2o, cuda), dev(inp.phy2log, cuda)
    batched, gws = solver.solve_batched(dev(counts.reshape(64, 1, shape.G, shape.L), cuda), r2o, p2l, avail,
                                        want_global=True)
    assert int(avail[0]) == 64
    for i in (0, 17, 63):
        single, gw = solver.solve(dev(counts[i].reshape(1, shape.G, shape.L), cuda), r2o, p2l, avail)
        assert torch.equal(single[0], batched[i, 0]) and torch.equal(gw, gws[i])
        _compare_solve(shape, inp.phy2log, counts[i], batched[i].cpu().numpy(), gws[i].cpu().numpy(), 1)


def test_solve_batched_throughput_sweep_all_2048_against_oracle(cuda):
    """The solver half of the throughput sweep: 2048 independent V3 / EP8-cube count vectors in one
    launch (one block per LP in the reference, csrc/plugin.cpp:559-565; here four LPs per wave from
    1536 LPs on).  Every one of the 2048 results is held against the fp32 oracle."""
    inp = synth.make_inputs("v3_ep8_cube", tokens=8)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    counts = synth.sweep_counts(2048)
    solver = solver_for(shape)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    res, gws = solver.solve_batched(dev(counts.reshape(2048, 1, shape.G, shape.L), cuda), dev(shape.r2o, cuda),
                                    dev(inp.phy2log, cuda), avail, want_global=True)
    torch.cuda.synchronize()
    flow, obj, n_ok = oracle.compare_batch(counts, res.cpu().numpy(), shape.r2o, inp.phy2log, 1, shape.C, shape.n_fixed)
    print(f"2048 LPs: worst flow diff {flow:.2e} of the tokens, worst objective diff {obj:.2e}, feasible {n_ok}")
    assert flow <= FLOW_TOL and obj <= OBJ_RTOL
    assert int(avail[0]) == n_ok == 2048
    for i in (0, 1000, 2047):
        np.testing.assert_array_equal(gws[i].cpu().numpy().reshape(-1), oracle.normalise(counts[i]))


def _shifted_ring(g, shifts):
    return np.array([[(i + s) % g for s in shifts] for i in range(g)], np.int32)


@pytest.mark.parametrize("name,r2o,ep,n_logical,n_inst", [
    ("cube8x2", None, 8, 256, 1541),                         # exact instantiation, last wave part full
    ("ring8x1", _shifted_ring(8, [1]), 8, 128, 1538),
    ("ring6x2_padded", _shifted_ring(6, [1, 2]), 6, 60, 1537),  # rounded up to the 8 x 2 instantiation
    ("ring16x1", _shifted_ring(16, [1]), 32, 256, 771),      # two groups per instance
])
def test_solve_batched_four_per_wave(cuda, name, r2o, ep, n_logical, n_inst):
    """From 1536 LPs on, small shapes are solved four to a wave (one per 16-lane row).  That kernel
    must agree with the one-LP-per-wave kernel (smaller batches) and with the oracle, also in a
    wave that is only partly filled, and the feasibility counter must add up either way."""
    from lplb_amd import topology
    from lplb_amd.mapping import build_redundancy_mapping
    r2o = topology.CUBE_8P2E if r2o is None else r2o
    shape = Shape(np.asarray(r2o, np.int32), ep, n_logical, n_logical + np.asarray(r2o).shape[1] * ep)
    phy2log, _, _ = build_redundancy_mapping(shape.r2o, ep, n_logical, shape.n_physical, None, n_nodes=1)
    rng = np.random.default_rng(7)
    skew = rng.uniform(0.05, 0.6, size=(n_inst, 1))
    counts = (np.clip(rng.standard_normal((n_inst, n_logical)) * skew + 1, 0, None) * 2 ** 12).astype(np.int32)
    solver = solver_for(shape)
    d_r2o, d_p2l = dev(shape.r2o, cuda), dev(phy2log, cuda)
    wl = dev(counts.reshape(n_inst, shape.n_group, shape.G, shape.L), cuda)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    packed, gws = solver.solve_batched(wl, d_r2o, d_p2l, avail, want_global=True)
    n_ok = int(avail[0])
    avail.zero_()
    chunk = 500 // shape.n_group
    by_wave = torch.cat([solver.solve_batched(wl[i:i + chunk], d_r2o, d_p2l, avail) for i in range(0, n_inst, chunk)])
    assert int(avail[0]) == n_ok
    assert packed.shape == by_wave.shape == (n_inst, shape.n_group, shape.G, shape.D)
    # b_i is summed by a different number of lanes in the two kernels, so the shares differ by
    # rounding, amplified where the LP is ill-conditioned (a long ring): compare the flows.
    a, b = packed.cpu().numpy(), by_wave.cpu().numpy()
    args = (shape.r2o, phy2log, shape.n_group, shape.C)
    for i in range(n_inst):
        flow = np.abs(oracle.edge_flows(counts[i], a[i], *args) - oracle.edge_flows(counts[i], b[i], *args)).max()
        assert flow <= FLOW_TOL * counts[i].sum(), (i, flow)
    total_ok = 0
    for i in (0, n_inst // 2, n_inst - 1):
        o_avail = oracle.solve(counts[i], shape.r2o, phy2log, shape.n_group, shape.C, shape.n_fixed)[2]
        _compare_solve(shape, phy2log, counts[i], packed[i].cpu().numpy(), gws[i].cpu().numpy(), o_avail)
        total_ok += o_avail
    assert n_ok >= total_ok


# ------------------------------------------------------------------ whole plan
@pytest.mark.parametrize("cfg,mask", [("cpu_ref_ep8", 0.0), ("v3_ep8_cube", 0.05), ("ep16_hypercube", 0.05),
                                      ("ep32_torus", 0.0)])
def test_run_matches_oracle_chain(cuda, cfg, mask):
    inp = synth.make_inputs(cfg, mask_fraction=mask)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    planner = Planner(torch.from_numpy(c.r2o), c.n_physical, c.n_logical, c.ep_size)
    planner.phy2log = dev(inp.phy2log, cuda)
    n_sms = 256
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    d_idx = dev(inp.indices, cuda)
    out = planner.run(d_idx, avail, n_sms)
    torch.cuda.synchronize()
    assert out.shape == d_idx.shape and out.dtype == torch.int64
    # the same chain on the CPU, fed with the GPU's own flow vector for the redirect
    by_sm = oracle.count_idx(inp.indices, c.n_logical, n_sms)
    local, by_sm_gpu = planner.count_workload(d_idx, n_sms)
    np.testing.assert_array_equal(by_sm_gpu.cpu().numpy(), by_sm)
    o_weight, gw = planner.solve_probs(local, torch.zeros(1, dtype=torch.int32, device=cuda))
    _compare_solve(shape, inp.phy2log, by_sm[-1], o_weight.cpu().numpy(), gw.cpu().numpy(), int(avail[0]))
    want = oracle.map_idx(inp.indices, o_weight.cpu().numpy(), by_sm, shape.o2r, inp.phy2log, shape.n_group,
                          shape.C, shape.P)
    np.testing.assert_array_equal(out.cpu().numpy(), want)


@pytest.mark.gpu
@pytest.mark.parametrize("g,shifts,n_group", [(16, [1, 2, 3, 4, 5], 1), (12, [1, 2, 3, 5, 7, 11], 2),
                                             (8, [1, 2, 3, 4, 5, 6, 7, 1, 2], 1), (32, [1, 2, 16], 1)])
def test_run_with_more_than_64_replica_edges(cuda, g, shifts, n_group):
    """Groups with 65 to 128 replica edges (two edges per lane in the LP): Planner.run against the chain on
    the CPU, as for the benchmark configurations."""
    from lplb_amd.mapping import build_redundancy_mapping
    rng = np.random.default_rng(g * 100 + len(shifts))
    r2o = _shifted_ring(g, shifts)
    d = len(shifts)
    assert g * d > 64
    ep = g * n_group
    per_rank = d + 3
    n_logical = ep * per_rank
    shape = Shape(r2o, ep, n_logical, n_logical + d * ep)
    hist = rng.integers(1, 1 << 20, size=n_logical).astype(np.int64)
    phy2log, _, _ = build_redundancy_mapping(r2o, ep, n_logical, shape.n_physical, hist, n_nodes=1)
    idx = rng.choice(n_logical, size=(6000, 4), p=rng.dirichlet(np.full(n_logical, 0.7))).astype(np.int64)
    idx[rng.random(idx.shape) < 0.03] = -1
    planner = Planner(torch.from_numpy(r2o), shape.n_physical, n_logical, ep)
    planner.phy2log = dev(phy2log, cuda)
    n_sms = 64
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    d_idx = dev(idx, cuda)
    out = planner.run(d_idx, avail, n_sms)
    torch.cuda.synchronize()
    by_sm = oracle.count_idx(idx, n_logical, n_sms)
    local, by_sm_gpu = planner.count_workload(d_idx, n_sms)
    np.testing.assert_array_equal(by_sm_gpu.cpu().numpy(), by_sm)
    o_weight, gw = planner.solve_probs(local, torch.zeros(1, dtype=torch.int32, device=cuda))
    _compare_solve(shape, phy2log, by_sm[-1], o_weight.cpu().numpy(), gw.cpu().numpy(), int(avail[0]))
    want = oracle.map_idx(idx, o_weight.cpu().numpy(), by_sm, shape.o2r, phy2log, shape.n_group, shape.C, shape.P)
    np.testing.assert_array_equal(out.cpu().numpy(), want)


@pytest.mark.gpu
@pytest.mark.parametrize("offset", [1, 3, 256, 257])
def test_run_on_a_view_that_starts_inside_a_tensor(cuda, offset):
    """A contiguous view whose first element sits at an odd multiple of 8 bytes is a legal
    input of the reference (csrc/plugin.cpp:582-584 asks for int64 and contiguity only)."""
    c = synth.CONFIGS["cpu_ref_ep8"]
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    rng = np.random.default_rng(900 + offset)
    whole = rng.integers(-1, c.n_logical, size=offset + 5001, dtype=np.int64)
    d_whole = dev(whole, cuda)
    d_idx = d_whole[offset:]
    assert d_idx.is_contiguous() and d_idx.data_ptr() == d_whole.data_ptr() + 8 * offset
    idx = whole[offset:]
    planner = Planner(torch.from_numpy(c.r2o), c.n_physical, c.n_logical, c.ep_size)
    phy2log = planner.phy2log.cpu().numpy()
    for n_sms in (2, 16, 64):
        by_sm = oracle.count_idx(idx, c.n_logical, n_sms)
        local, by_sm_gpu = planner.count_workload(d_idx, n_sms)
        np.testing.assert_array_equal(by_sm_gpu.cpu().numpy(), by_sm)
        np.testing.assert_array_equal(local.cpu().numpy().ravel(), by_sm[-1])
        avail = torch.zeros(1, dtype=torch.int32, device=cuda)
        out = planner.run(d_idx, avail, n_sms)
        o_weight, _ = planner.solve_probs(local, torch.zeros(1, dtype=torch.int32, device=cuda))
        want = oracle.map_idx(idx, o_weight.cpu().numpy(), by_sm, shape.o2r, phy2log, shape.n_group, shape.C, shape.P)
        np.testing.assert_array_equal(out.cpu().numpy(), want)
    np.testing.assert_array_equal(d_whole.cpu().numpy(), whole)   # nothing outside the view was touched


@pytest.mark.parametrize("kind", ["empty", "all_masked", "one_token", "odd_length", "one_expert_only"])
def test_run_edge_inputs(cuda, kind):
    """Degenerate batches go through the same three kernels (tests/test_idx_processing.py of the
    reference only draws full random batches; these are the corners it leaves out)."""
    c = synth.CONFIGS["cpu_ref_ep8"]
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    rng = np.random.default_rng(11)
    idx = {"empty": np.zeros((0, c.topk), np.int64),
           "all_masked": np.full((77, c.topk), -1, np.int64),
           "one_token": rng.integers(0, c.n_logical, size=(1, c.topk), dtype=np.int64),
           "odd_length": rng.integers(-1, c.n_logical, size=(1237, 1), dtype=np.int64),
           "one_expert_only": np.full((4096, 1), 5, np.int64)}[kind]
    planner = Planner(torch.from_numpy(c.r2o), c.n_physical, c.n_logical, c.ep_size)
    phy2log = planner.phy2log.cpu().numpy()
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    n_sms = 16
    d_idx = dev(idx, cuda)
    out = planner.run(d_idx, avail, n_sms)
    torch.cuda.synchronize()
    assert out.shape == d_idx.shape and out.dtype == torch.int64
    phys = torch.full((c.n_physical,), -7, dtype=torch.int32, device=cuda)
    out2, _, _ = planner.solver.plan(d_idx, planner.r2o, planner.o2r, planner.phy2log,
                                     torch.zeros(1, dtype=torch.int32, device=cuda), n_sms, physical_counts=phys)
    assert torch.equal(out, out2)
    np.testing.assert_array_equal(phys.cpu().numpy(), np.bincount(out.cpu().numpy()[out.cpu().numpy() >= 0].ravel(),
                                                                  minlength=c.n_physical))
    by_sm = oracle.count_idx(idx.reshape(-1), c.n_logical, n_sms)
    o_res, _, o_avail = oracle.solve(by_sm[-1], shape.r2o, phy2log, shape.n_group, shape.C, shape.n_fixed)
    assert int(avail[0]) == o_avail
    if kind in ("empty", "all_masked"):
        assert o_avail == 0 and np.all(o_res == 0.5)      # no tokens: the LP has no scale, fallback shares
    local, by_sm_gpu = planner.count_workload(d_idx, n_sms)
    np.testing.assert_array_equal(by_sm_gpu.cpu().numpy(), by_sm)
    o_weight, _ = planner.solve_probs(local, torch.zeros(1, dtype=torch.int32, device=cuda))
    want = oracle.map_idx(idx.reshape(-1), o_weight.cpu().numpy(), by_sm, shape.o2r, phy2log, shape.n_group,
                          shape.C, shape.P).reshape(idx.shape)
    got = out.cpu().numpy()
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got == -1, idx == -1)
    valid = got >= 0
    np.testing.assert_array_equal(phy2log[got[valid]], idx[valid])   # every token still reaches its expert


def test_redirect_full_size_sweep(cuda):
    """[262144 x 8] indices: bit-exact against the oracle, exact split counts, conservation."""
    inp = synth.make_inputs("sweep_redirect")
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    solver = solver_for(shape)
    d_idx = dev(inp.indices, cuda)
    total, by_sm = solver.count_idx(d_idx, 256)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    o_weight, _ = solver.solve(total.view(1, shape.G, shape.L), dev(shape.r2o, cuda), dev(inp.phy2log, cuda), avail)
    out = solver.map_idx(d_idx, o_weight, by_sm, dev(shape.o2r, cuda), dev(inp.phy2log, cuda), 256)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = oracle.map_idx(inp.indices, o_weight.cpu().numpy(), by_sm.cpu().numpy(), shape.o2r, inp.phy2log, 1,
                          shape.C, shape.P)
    np.testing.assert_array_equal(got, want)
    # exact number of tokens kept on the original: clamp(trunc(w * total), 0, total) when 499 does not divide total
    tot = total.cpu().numpy().astype(np.int64)
    phys = np.bincount(got.reshape(-1), minlength=c.n_physical)
    assert phys.sum() == inp.indices.size
    w = o_weight.cpu().numpy().reshape(shape.G, shape.D)
    p2l = inp.phy2log.reshape(c.ep_size, shape.P)
    for rank in range(c.ep_size):
        for slot in range(shape.C * shape.D):
            e = p2l[rank, slot]
            if tot[e] % 499 == 0:
                continue
            keep = int(np.clip(np.trunc(np.float32(w[rank, slot % shape.D]) * np.float32(tot[e])), 0, tot[e]))
            assert phys[rank * shape.P + slot] == keep, (rank, slot)


@pytest.mark.gpu
def test_redirect_when_the_hash_wraps(cuda):
    """An expert with more than (2^31 - 42) / 499 = 4 303 556 tokens makes 499 k + 41 wrap to negative
    int32 values, whose remainder is negative too (minilp.cu:505 computes in int).  Bit-exact against
    the oracle, through both the three entry points and the single call."""
    c = synth.CONFIGS["cpu_ref_ep8"]
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    planner = Planner(torch.from_numpy(c.r2o), c.n_physical, c.n_logical, c.ep_size)
    phy2log = planner.phy2log.cpu().numpy()
    rng = np.random.default_rng(4303557)
    n = 12_000_000
    heavy = int(phy2log.reshape(c.ep_size, shape.P)[3, 0])      # an expert that has a replica
    p = np.full(c.n_logical, 0.45 / (c.n_logical - 1))
    p[heavy] = 0.55
    idx = rng.choice(c.n_logical, size=n, p=p).astype(np.int64)
    idx[rng.random(n) < 0.01] = -1
    assert np.count_nonzero(idx == heavy) > 6_000_000
    d_idx = dev(idx, cuda)
    n_sms = 256
    local, by_sm = planner.count_workload(d_idx, n_sms)
    want_by_sm = oracle.count_idx(idx, c.n_logical, n_sms)
    np.testing.assert_array_equal(by_sm.cpu().numpy(), want_by_sm)
    o_weight, _ = planner.solve_probs(local, torch.zeros(1, dtype=torch.int32, device=cuda))
    got = planner.weighted_select_target(d_idx, o_weight, by_sm, n_sms).cpu().numpy()
    want = oracle.map_idx(idx, o_weight.cpu().numpy(), want_by_sm, shape.o2r, phy2log, shape.n_group, shape.C, shape.P)
    np.testing.assert_array_equal(got, want)
    both = np.unique(got[idx == heavy])
    assert len(both) == 2                                        # the heavy expert really is split
    out = planner.run(d_idx, torch.zeros(1, dtype=torch.int32, device=cuda), n_sms)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    # the closed form behind physical_counts assumes no wrap: asked for here, it is refused
    with pytest.raises(RuntimeError, match="physical_counts"):
        planner.run(d_idx, torch.zeros(1, dtype=torch.int32, device=cuda), n_sms,
                    physical_counts=torch.empty(c.n_physical, dtype=torch.int32, device=cuda))


# ------------------------------------------------------- single-call plan, graphs
def _plan_setup(cuda, cfg_name, mask=0.05):
    inp = synth.make_inputs(cfg_name, mask_fraction=mask)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    solver = solver_for(shape)
    t = dict(idx=dev(inp.indices, cuda), r2o=dev(shape.r2o, cuda), o2r=dev(shape.o2r, cuda),
             phy2log=dev(inp.phy2log, cuda), counts=dev(inp.global_counts, cuda))
    return inp, shape, solver, t


@pytest.mark.parametrize("cfg", ["cpu_ref_ep8", "v3_ep8_cube", "ep32_torus"])
@pytest.mark.parametrize("use_global", [True, False])
def test_plan_entry_point_matches_three_calls(cuda, cfg, use_global):
    """lplb_plan == count_idx + solve + map_idx, with the LP fed by the supplied global counts or by
    this GPU's own histogram (lplb/planner.py:264-266)."""
    inp, shape, solver, t = _plan_setup(cuda, cfg)
    n_sms = 200
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    out, o_weight, by_sm = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, n_sms,
                                       global_counts=t["counts"] if use_global else None)
    torch.cuda.synchronize()
    want_by_sm = oracle.count_idx(inp.indices, shape.n_logical, n_sms)
    # the last row always holds this GPU's totals; the rows above it are the library's workspace
    np.testing.assert_array_equal(by_sm[-1].cpu().numpy(), want_by_sm[-1])
    workload = inp.global_counts if use_global else want_by_sm[-1]
    avail2 = torch.zeros(1, dtype=torch.int32, device=cuda)
    ref_w, _ = solver.solve(dev(workload.reshape(shape.n_group, shape.G, shape.L), cuda), t["r2o"], t["phy2log"], avail2)
    assert torch.equal(o_weight, ref_w) and int(avail[0]) == int(avail2[0]) == shape.n_group
    want = oracle.map_idx(inp.indices, o_weight.cpu().numpy(), want_by_sm, shape.o2r, inp.phy2log, shape.n_group,
                          shape.C, shape.P)
    np.testing.assert_array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("cfg", ["cpu_ref_ep8", "v3_ep8_cube", "ep16_hypercube", "ep32_torus"])
@pytest.mark.parametrize("use_global", [True, False])
@pytest.mark.parametrize("tokens,n_sms", [(None, 256), (37, 256), (4100, 9), (16384, 40), (20000, 256), (32768, 65), (40000, 256)])
def test_plan_one_launch_equals_chain(cuda, cfg, use_global, tokens, n_sms):
    """Short batches run as one kernel launch whose workgroups exchange histogram rows and the
    LP's shares through memory; the result must be the chain's, bit for bit, call after call."""
    inp = synth.make_inputs(cfg, tokens=tokens, mask_fraction=0.05) if tokens else synth.make_inputs(cfg, mask_fraction=0.05)
    _one_launch_equals_chain(cuda, inp, use_global, n_sms, expect_one_launch=True)


MANY_GROUPS = {
    # the LPs of a batch are spread over workgroups of four: 5 groups leave the second one partly empty
    "ep40_5_cubes": synth.PlanConfig("ep40", topology.CUBE_8P2E, 40, 240, 2, 4096, 8, 1.0, jitter_sigma=0.3, seed=40),
    "v3_ep64_8_cubes": synth.PlanConfig("ep64", topology.CUBE_8P2E, 64, 256, 2, 4096, 8, 1.0, jitter_sigma=0.3, seed=64),
    "v3_ep128_16_cubes": synth.PlanConfig("ep128", topology.CUBE_8P2E, 128, 256, 2, 512, 8, 1.0, jitter_sigma=0.3, seed=128),
    "v3_ep256_32_rings": synth.PlanConfig("ep256", topology.RING_8P, 256, 256, 1, 128, 8, 1.0, jitter_sigma=0.3, seed=256),
    "v3_ep64_4_hypercubes": synth.PlanConfig("ep64h", topology.HYPERCUBE_16P2E, 64, 256, 2, 4096, 8, 1.0, seed=65),
    "v3_ep192_6_tori": synth.PlanConfig("ep192", topology.torus_2d(8, 4), 192, 384, 2, 2048, 8, 1.0, seed=192),
    # more logical experts: the slice workgroups' LDS tables then leave room for 8 waves only
    "ep8_512_experts": synth.PlanConfig("e512", topology.CUBE_8P2E, 8, 512, 2, 4096, 10, 1.0, jitter_sigma=0.3, seed=512),
    "ep32_384_experts": synth.PlanConfig("e384", topology.CUBE_8P2E, 32, 384, 2, 4096, 8, 1.0, jitter_sigma=0.3, seed=384),
    "ep16_1024_experts": synth.PlanConfig("e1024", topology.HYPERCUBE_16P2E, 16, 1024, 2, 2048, 8, 1.0, seed=1024),
}


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(MANY_GROUPS))
@pytest.mark.parametrize("use_global", [True, False])
def test_plan_one_launch_with_many_groups(cuda, name, use_global):
    """Large EP sizes: several LPs per batch, up to four per LP workgroup."""
    inp = synth.make_inputs(MANY_GROUPS[name], mask_fraction=0.02)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    got = _one_launch_equals_chain(cuda, inp, use_global, 256, expect_one_launch=True)
    # and the chain's result is the oracle's
    counts = inp.global_counts if use_global else np.bincount(inp.indices[inp.indices >= 0].ravel(),
                                                              minlength=c.n_logical).astype(np.int32)
    _, _, o_avail = oracle.solve(counts, shape.r2o, inp.phy2log, shape.n_group, shape.C, shape.n_fixed)
    assert got[3] == o_avail
    by_sm = oracle.count_idx(inp.indices.reshape(-1), c.n_logical, 256)
    want = oracle.map_idx(inp.indices.reshape(-1), got[1], by_sm, shape.o2r, inp.phy2log, shape.n_group, shape.C,
                          shape.P).reshape(inp.indices.shape)
    np.testing.assert_array_equal(got[0], want)


def _one_launch_equals_chain(cuda, inp, use_global, n_sms, expect_one_launch=None):
    """Runs the plan as the chain, then twice in the default mode; everything must agree bit for bit.
    expect_one_launch=True additionally requires that the default mode really ran as one kernel launch
    (the library counts those), so that the comparison is not the chain against itself."""
    from lplb_amd import _native
    timeouts_before = _native.plan_sync_timeouts()
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    solver = solver_for(shape)
    t = dict(idx=dev(inp.indices, cuda), r2o=dev(shape.r2o, cuda), o2r=dev(shape.o2r, cuda),
             phy2log=dev(inp.phy2log, cuda), counts=dev(inp.global_counts, cuda))
    counts = t["counts"] if use_global else None
    runs = {}
    try:
        for mode in (False, True, True):
            _native.set_plan_cooperative(mode)
            avail = torch.zeros(1, dtype=torch.int32, device=cuda)
            phys = torch.full((shape.n_physical,), -7, dtype=torch.int32, device=cuda)
            launches_before = _native.plan_one_launch_count()
            out, o_weight, by_sm = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, n_sms,
                                               global_counts=counts, physical_counts=phys)
            torch.cuda.synchronize()
            as_one_launch = _native.plan_one_launch_count() - launches_before
            assert as_one_launch == 0 if not mode else as_one_launch in (0, 1)
            if mode and expect_one_launch is not None:
                assert as_one_launch == int(expect_one_launch), "the plan did not take the expected form"
            got = (out.cpu().numpy(), o_weight.cpu().numpy(), by_sm[-1].cpu().numpy(), int(avail[0]),
                   phys.cpu().numpy())
            if mode not in runs:
                runs[mode] = got
            for a, b in zip(got, runs[False]):
                np.testing.assert_array_equal(a, b)
    finally:
        _native.set_plan_cooperative(True)
    assert _native.plan_sync_timeouts() == timeouts_before
    np.testing.assert_array_equal(runs[True][2], np.bincount(inp.indices[inp.indices >= 0].ravel(),
                                                             minlength=c.n_logical))
    out = runs[True][0]
    np.testing.assert_array_equal(runs[True][4], np.bincount(out[out >= 0].ravel(), minlength=c.n_physical))
    return runs[True]


def test_plan_random_shapes_one_launch_equals_chain(cuda):
    """Thirty seeded draws of topology, experts per rank, batch length and slice bound, in both LP
    feeding modes: the one-launch plan (where it applies) and the chain agree bit for bit."""
    from lplb_amd import _native, topology
    from lplb_amd.mapping import build_redundancy_mapping
    rng = np.random.default_rng(77)
    timeouts_before = _native.plan_sync_timeouts()
    topologies = [(topology.CUBE_8P2E, 1), (topology.RING_8P, 1), (topology.HYPERCUBE_16P2E, 1),
                  (topology.torus_2d(8, 4), 1), (topology.CUBE_8P2E, 4), (_shifted_ring(6, [1, 2]), 2),
                  (_shifted_ring(4, [1, 2, 3]), 3), (_shifted_ring(16, [1]), 2), (topology.CUBE_8P2E, 9),
                  (topology.RING_8P, 16)]
    try:
        for trial in range(30):
            r2o, n_group = topologies[int(rng.integers(len(topologies)))]
            r2o = np.asarray(r2o, np.int32)
            g, d = r2o.shape
            ep = g * n_group
            per_rank = d + int(rng.integers(d, 10))
            n_logical = ep * per_rank
            shape = Shape(r2o, ep, n_logical, n_logical + d * ep)
            hist = rng.integers(1, 1 << 20, size=n_logical).astype(np.int64)
            phy2log, _, _ = build_redundancy_mapping(r2o, ep, n_logical, shape.n_physical, hist, n_nodes=1)
            n = int(rng.choice([1, 300, 1024, 5000, 65536, 100000, 262144, 270000]))
            n_sms = int(rng.choice([2, 9, 64, 65, 256]))
            popularity = rng.dirichlet(np.full(n_logical, 0.7))
            idx = rng.choice(n_logical, size=n, p=popularity).astype(np.int64)
            idx[rng.random(n) < 0.03] = -1
            counts = (np.bincount(idx[idx >= 0], minlength=n_logical) * ep +
                      rng.integers(0, 50, size=n_logical)).astype(np.int32)
            solver = solver_for(shape)
            t = dict(idx=dev(idx, cuda), r2o=dev(r2o, cuda), o2r=dev(shape.o2r, cuda), phy2log=dev(phy2log, cuda))
            for global_counts in (dev(counts, cuda), None):
                got = {}
                for mode in (False, True):
                    _native.set_plan_cooperative(mode)
                    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
                    phys = torch.empty(shape.n_physical, dtype=torch.int32, device=cuda)
                    out, w, by = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, n_sms,
                                             global_counts=global_counts, physical_counts=phys)
                    torch.cuda.synchronize()
                    got[mode] = (out.cpu().numpy(), w.cpu().numpy(), by[-1].cpu().numpy(), int(avail[0]),
                                 phys.cpu().numpy())
                for a, b in zip(got[True], got[False]):
                    np.testing.assert_array_equal(a, b, err_msg=f"trial {trial} {r2o.shape} n={n} n_sms={n_sms}")
    finally:
        _native.set_plan_cooperative(True)
    assert _native.plan_sync_timeouts() == timeouts_before


def test_planner_run_equals_plan_with_local_counts(cuda):
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    c = inp.cfg
    planner = Planner(torch.from_numpy(c.r2o), c.n_physical, c.n_logical, c.ep_size)
    planner.phy2log = t["phy2log"]
    a1 = torch.zeros(1, dtype=torch.int32, device=cuda)
    a2 = torch.zeros(1, dtype=torch.int32, device=cuda)
    got = planner.run(t["idx"], a1, 128)
    want, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], a2, 128)
    assert torch.equal(got, want) and int(a1[0]) == int(a2[0]) == 1


def test_planner_run_with_a_process_group(cuda, monkeypatch):
    """With a group, run() sums the local histogram over the ranks before the LP (lplb/planner.py:214-216).
    The collective is stubbed here (one GPU): it adds what the other ranks would contribute."""
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    c = inp.cfg
    local = np.bincount(inp.indices[inp.indices >= 0].ravel(), minlength=c.n_logical).astype(np.int32)
    others = dev(inp.global_counts - np.minimum(local, inp.global_counts), cuda)
    calls = []

    def fake_all_reduce(tensor, group=None):
        calls.append(group)
        tensor += others.view_as(tensor)

    monkeypatch.setattr(torch.distributed, "all_reduce", fake_all_reduce)
    took = []          # which of the three ways to this GPU's counts a call took
    for way in ("count_totals_add", "count_totals", "count_idx"):
        def spy(self, *a, _way=way, _real=getattr(CompiledSolver, way), **kw):
            took.append(_way)
            return _real(self, *a, **kw)
        monkeypatch.setattr(CompiledSolver, way, spy)
    group = object()
    planner = Planner(torch.from_numpy(c.r2o), c.n_physical, c.n_logical, c.ep_size, group)
    planner.phy2log = t["phy2log"]
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    out = planner.run(t["idx"], avail, 256)
    assert calls == [group] and int(avail[0]) == shape.n_group and took == ["count_totals_add"]
    summed = dev(local, cuda) + others
    avail2 = torch.zeros(1, dtype=torch.int32, device=cuda)
    want, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail2, 256, global_counts=summed)
    assert torch.equal(out, want)
    # the three public steps give the same (lplb/planner.py:264-266)
    lw, by_sm = planner.count_workload(t["idx"], 256)
    o_weight, _ = planner.solve_probs(lw, avail2)
    assert torch.equal(planner.weighted_select_target(t["idx"], o_weight, by_sm, 256), out)
    # a batch too long for the one-launch totals takes histogram + scan, then a short one again
    from lplb_amd import _native
    long_idx = t["idx"].repeat(3, 1)
    assert t["idx"].numel() <= _native.COUNT_TOTALS_MAX_INDICES < long_idx.numel()
    for batch, times in ((long_idx, 3), (t["idx"], 1)):
        avail.zero_(), avail2.zero_()
        got = planner.run(batch, avail, 256)
        want, _, _ = solver.plan(batch, t["r2o"], t["o2r"], t["phy2log"], avail2, 256,
                                 global_counts=times * dev(local, cuda) + others)
        assert int(avail[0]) == int(avail2[0]) == shape.n_group, (times, int(avail[0]), int(avail2[0]))
        assert torch.equal(got, want), (times, int((got != want).sum()))
    assert len(calls) == 4   # run, solve_probs, and the two runs above
    assert took == ["count_totals_add", "count_idx", "count_idx", "count_totals_add"]   # (count_workload is the third)
    took.clear()
    # captured into a graph, the call must not rely on what an earlier call left in its vectors
    # (LP and redirect as the chain of kernels here: a captured one-launch plan keeps its share of the GPU
    # reserved for as long as the process lives, and this test is about the counts)
    _native.set_plan_cooperative(False)
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            planner.run(t["idx"], avail, 256)                       # (buffers of this stream, outside the capture)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = planner.run(t["idx"], avail, 256)
        for replay in range(3):
            avail.zero_()
            captured.fill_(-7)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(captured, out) and int(avail[0]) == shape.n_group, replay
            planner.run(t["idx"], torch.zeros_like(avail), 256)     # eager work between the replays
            torch.cuda.synchronize()
        assert took == ["count_totals_add", "count_totals"] + 3 * ["count_totals_add"]
    finally:
        _native.set_plan_cooperative(True)


@pytest.mark.parametrize("use_global", [True, False])
def test_plan_at_the_sweep_shape_is_one_launch_and_equals_the_chain(cuda, use_global):
    """[262144 x 8] indices: 256 slices of 8192 indices (16 chunks per wave) and the LP in one grid.
    (Ahead of the tests that capture plans into graphs: a captured one-launch plan keeps its share of the GPU
    reserved for as long as the process lives, and this plan needs a third of the GPU.)"""
    inp = synth.make_inputs("sweep_redirect", mask_fraction=0.01)
    got = _one_launch_equals_chain(cuda, inp, use_global, 512, expect_one_launch=True)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    by_sm = oracle.count_idx(inp.indices.reshape(-1), c.n_logical, 512)
    want = oracle.map_idx(inp.indices.reshape(-1), got[1], by_sm, shape.o2r, inp.phy2log, shape.n_group, shape.C,
                          shape.P).reshape(inp.indices.shape)
    np.testing.assert_array_equal(got[0], want)


@pytest.mark.parametrize("use_global", [True, False])
@pytest.mark.parametrize("one_launch", [True, False])
def test_plan_replays_from_a_hip_graph(cuda, use_global, one_launch):
    """Capture two plans into a graph; every replay, with eager work and synchronisation between
    replays, must reproduce the eager result and advance the counter.  (The one-launch plan keeps
    counters in device memory that its last workgroup clears: a replay has the same arguments.
    The chain of kernels is captured too: its histogram launch is marked as free to overtake
    the LP before it.)"""
    from lplb_amd import _native
    _native.set_plan_cooperative(one_launch)
    try:
        _replay_plans_from_a_graph(cuda, use_global)
    finally:
        _native.set_plan_cooperative(True)


def _replay_plans_from_a_graph(cuda, use_global):
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    counts = t["counts"] if use_global else None
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    eager, eager_w, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=counts)
    torch.cuda.synchronize()
    ws = {"out": torch.empty_like(eager), "o_weight": torch.empty_like(eager_w),
          "by_sm": torch.empty(256, shape.n_logical, dtype=torch.int32, device=cuda),
          "global_workload": torch.empty(shape.n_logical, dtype=torch.float32, device=cuda)}
    phys = torch.empty(shape.n_physical, dtype=torch.int32, device=cuda)

    def plan():
        solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=counts, workspace=ws,
                    physical_counts=phys)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        plan()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    before = int(avail[0])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan()
        plan()
    for rep in range(4):
        ws["out"].fill_(-5)
        ws["o_weight"].zero_()
        phys.fill_(-5)
        scratch = torch.randn(1 << 16, device=cuda).sum()      # unrelated eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(ws["out"], eager) and torch.equal(ws["o_weight"], eager_w), rep
        assert int(avail[0]) == before + 2 * (rep + 1)
        assert torch.equal(phys.long(), torch.bincount(eager[eager >= 0].flatten(), minlength=shape.n_physical))
        del scratch


def test_planner_run_replays_from_a_hip_graph(cuda):
    """Planner.run keeps its scratch buffers per stream; captured on torch's capture stream and
    replayed, it still gives the eager result."""
    inp = synth.make_inputs("v3_ep8_cube", mask_fraction=0.05)
    c = inp.cfg
    planner = Planner(torch.from_numpy(c.r2o), c.n_physical, c.n_logical, c.ep_size)
    planner.phy2log = dev(inp.phy2log, cuda)
    idx = dev(inp.indices, cuda)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    eager = planner.run(idx, avail, 128).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        planner.run(idx, avail, 128)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    before = int(avail[0])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = planner.run(idx, avail, 128)
    for rep in range(3):
        out.fill_(-9)
        assert torch.equal(planner.run(idx, avail, 128), eager)     # eager calls between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        assert int(avail[0]) == before + 2 * (rep + 1)


def test_forgetting_captured_plans_gives_their_share_back(cuda):
    """Plans captured on stream after stream fill the library's eight blocks of counters, and later plans on a new
    stream run as the chain; once the graphs are gone and the caller has said so, they run as one launch again."""
    from lplb_amd import _native
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)

    def plan_on(stream):
        before = _native.plan_one_launch_count()
        with torch.cuda.stream(stream):
            out, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=t["counts"])
        stream.synchronize()
        return out, _native.plan_one_launch_count() - before

    torch.cuda.synchronize()
    want, one = plan_on(torch.cuda.Stream())
    assert one == 1
    streams, graphs = [], []
    for _ in range(10):                          # more than there are blocks
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        plan_on(s)                               # (buffers and first-call work outside the capture)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=t["counts"])
        streams.append(s), graphs.append(g)
    out, one = plan_on(torch.cuda.Stream())
    assert one == 0 and torch.equal(out, want)   # no block left, or no room beside the reserved shares: the chain
    del graphs
    for s in streams:
        _native.plan_forget_captured(s)
    out, one = plan_on(torch.cuda.Stream())
    assert one == 1 and torch.equal(out, want)


@pytest.mark.parametrize("cooperative", [False, True])
def test_plans_on_two_streams(cuda, cooperative):
    """Plans on different streams may overlap on the device.  The one-launch form keeps its
    counters per stream, and the chain of kernels has no shared state at all."""
    from lplb_amd import _native
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    other = synth.make_inputs("v3_ep8_cube", tokens=5000, mask_fraction=0.1)
    idx_b = dev(other.indices, cuda)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    want_a, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256)
    want_b, _, _ = solver.plan(idx_b, t["r2o"], t["o2r"], t["phy2log"], avail, 256)
    torch.cuda.synchronize()
    streams = [torch.cuda.current_stream(), torch.cuda.Stream(), torch.cuda.Stream()]
    timeouts_before, launches_before = _native.plan_sync_timeouts(), _native.plan_one_launch_count()
    _native.set_plan_cooperative(cooperative)
    try:
        for rep in range(30):
            outs = []
            for s_, idx in zip(streams, (t["idx"], idx_b, t["idx"])):
                with torch.cuda.stream(s_):
                    outs.append(solver.plan(idx, t["r2o"], t["o2r"], t["phy2log"], avail, 256)[0])
            torch.cuda.synchronize()
            assert torch.equal(outs[0], want_a) and torch.equal(outs[1], want_b) and torch.equal(outs[2], want_a), rep
        assert _native.plan_sync_timeouts() == timeouts_before
        # three plans of 65 workgroups fit the GPU side by side: all 90 ran as one launch each (or none)
        assert _native.plan_one_launch_count() - launches_before == (90 if cooperative else 0)
    finally:
        _native.set_plan_cooperative(True)


def test_one_launch_plan_while_another_stream_fills_the_gpu(cuda):
    """The workgroups of the one-launch plan wait for each other; they must still all get their turn when
    another stream keeps every CU busy (here with matrix products), and no wait may run out."""
    from lplb_amd import _native
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    want, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=t["counts"])
    want = want.clone()
    torch.cuda.synchronize()
    a = torch.randn(4096, 4096, device=cuda, dtype=torch.bfloat16)
    b = torch.randn(4096, 4096, device=cuda, dtype=torch.bfloat16)
    busy, planning = torch.cuda.Stream(), torch.cuda.Stream()
    timeouts_before, launches_before = _native.plan_sync_timeouts(), _native.plan_one_launch_count()
    for rep in range(10):
        with torch.cuda.stream(busy):
            for _ in range(4):
                c = a @ b
        with torch.cuda.stream(planning):
            outs = [solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=t["counts"])[0]
                    for _ in range(4)]
        torch.cuda.synchronize()
        assert all(torch.equal(o, want) for o in outs), rep
        del c
    assert _native.plan_sync_timeouts() == timeouts_before
    assert _native.plan_one_launch_count() - launches_before == 40     # not the chain by accident


@pytest.mark.parametrize("use_global", [True, False])
def test_one_launch_plan_gives_up_in_a_defined_way(cuda, use_global):
    """A wait between workgroups that cannot be met (forced from the host: the kernel is told to expect
    one slice more than its grid has, and to poll 2000 times instead of millions) must end in the
    documented fallback -- every token on its expert's original slot, physical_counts filled with -1,
    the give-ups counted -- with every kernel ending normally.  The block of counters the launch used
    is switched off after that: the next plan on the stream falls back in the same way and counts one
    more failure, until lplb_plan_sync_timeouts has been called; then plans are right again
    (minilp.cu:395-397 is the reference's own neutral fallback for an LP that fails)."""
    from lplb_amd import _native
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    lib = _native.load()
    counts = t["counts"] if use_global else None
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    phys = torch.full((shape.n_physical,), -7, dtype=torch.int32, device=cuda)
    want, want_w, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=counts,
                                  physical_counts=phys)
    want, want_w, want_phys = want.clone(), want_w.clone(), phys.clone()
    torch.cuda.synchronize()
    assert int(avail[0]) == 1
    timeouts_before, launches_before = _native.plan_sync_timeouts(), _native.plan_one_launch_count()
    print("injecting a wait that cannot be met", flush=True)
    assert lib.lplb_plan_inject_fault(1, 2000) == 0
    # the fallback: the redirect with every share = 1 keeps every token on the original
    by_sm = oracle.count_idx(inp.indices, shape.n_logical, 256)
    stay = oracle.map_idx(inp.indices, np.ones((1, shape.G, shape.D), np.float32), by_sm, shape.o2r, inp.phy2log, 1,
                          shape.C, shape.P)
    for later in range(2):   # the launch in which the wait runs out, then one that finds the block switched off
        phys.fill_(-7)
        out, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=counts,
                                physical_counts=phys)
        torch.cuda.synchronize()
        assert _native.plan_one_launch_count() == launches_before + 1 + later
        np.testing.assert_array_equal(out.cpu().numpy(), stay)
        assert torch.all(phys == -1)
    # The counter of feasible LPs must not vouch for a batch that was not balanced (the reference's callers
    # assert on it, tests/test_solve.py:58): with the counts supplied the LP is solved all the same in the first
    # of the two launches, and whichever comes first, its add or the first give-up, the add does not stay; a
    # launch that finds the block switched off adds nothing.
    assert int(avail[0]) == 1
    # the report that does not wait says the same as the synchronous one is about to
    report = torch.full((2,), -1, dtype=torch.int32, device=cuda)
    _native.plan_poll_timeouts(report)
    torch.cuda.synchronize()
    assert int(report[1]) == 1 and int(report[0]) - timeouts_before >= 64 + 1
    gave_up = _native.plan_sync_timeouts() - timeouts_before      # ... which also switches the block on again
    pinned = torch.full((2,), -1, dtype=torch.int32).pin_memory()
    _native.plan_poll_timeouts(pinned)
    torch.cuda.synchronize()
    assert int(pinned[1]) == 0 and int(pinned[0]) - timeouts_before == gave_up
    assert gave_up >= 64 + 1, gave_up           # every slice workgroup's wait (and the LP's, if it waited too), and the second plan
    # the next plans on the same stream are healthy
    avail.zero_()
    for _ in range(3):
        out, o_w, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256, global_counts=counts,
                                  physical_counts=phys)
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(o_w, want_w) and torch.equal(phys, want_phys)
    assert int(avail[0]) == 3
    assert _native.plan_sync_timeouts() - timeouts_before == gave_up
    assert _native.plan_one_launch_count() == launches_before + 5


def test_planner_run_notices_a_wait_that_ran_out(cuda):
    """Planner.run looks at the health report every few calls without waiting for the GPU; after a forced
    give-up it warns, switches the one-launch form on again and plans correctly from then on."""
    from lplb_amd import _native
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    planner = Planner(torch.from_numpy(inp.cfg.r2o), inp.cfg.n_physical, inp.cfg.n_logical, inp.cfg.ep_size, device=cuda)
    planner.phy2log = t["phy2log"]
    planner.health_check_every = 2
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    want = planner.run(t["idx"], avail, 256).clone()
    torch.cuda.synchronize()
    before = _native.plan_sync_timeouts()
    planner.plan_timeouts = before
    print("injecting a wait that cannot be met", flush=True)
    assert _native.load().lplb_plan_inject_fault(1, 2000) == 0
    avail.zero_()
    with pytest.warns(RuntimeWarning, match="not balanced"):
        for _ in range(8):
            out = planner.run(t["idx"], avail, 256)
            torch.cuda.synchronize()
    assert planner.plan_timeouts > before
    unbalanced = 8 - int(avail[0])
    assert 1 <= unbalanced <= 5, unbalanced      # from the give-up to the look that re-armed: two looks at most, two calls apart
    assert torch.equal(out, want)
    assert _native.plan_sync_timeouts() == planner.plan_timeouts


def test_one_launch_slots_pass_from_stream_to_stream(cuda):
    """More streams than the library has counter blocks: a block whose last launch has completed
    passes to the next stream, so a long-running process keeps the one-launch form."""
    from lplb_amd import _native
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    want, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256)
    want = want.clone()
    torch.cuda.synchronize()
    launches_before = _native.plan_one_launch_count()
    streams = [torch.cuda.Stream() for _ in range(20)]
    for s_ in streams:
        s_.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s_):
            out, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256)
        s_.synchronize()
        assert torch.equal(out, want)
    assert _native.plan_one_launch_count() - launches_before == 20


def test_one_launch_plans_beyond_what_fits_the_gpu_run_as_the_chain(cuda):
    """Twelve streams plan at the same time without waiting for each other.  Only as many one-launch
    plans as fit the GPU side by side are admitted (their workgroups wait for each other); the rest
    run as the chain.  Every result is right and no wait runs out."""
    from lplb_amd import _native
    inp, shape, solver, t = _plan_setup(cuda, "v3_ep8_cube")
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    want, _, _ = solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256)
    want = want.clone()
    torch.cuda.synchronize()
    timeouts_before, launches_before = _native.plan_sync_timeouts(), _native.plan_one_launch_count()
    streams = [torch.cuda.Stream() for _ in range(12)]
    for rep in range(5):
        outs = []
        for s_ in streams:
            with torch.cuda.stream(s_):
                outs.append(solver.plan(t["idx"], t["r2o"], t["o2r"], t["phy2log"], avail, 256)[0])
        torch.cuda.synchronize()
        assert all(torch.equal(o, want) for o in outs), rep
    as_one_launch = _native.plan_one_launch_count() - launches_before
    print(f"{as_one_launch} of 60 concurrent plans ran as one launch")
    assert 5 <= as_one_launch <= 60
    assert _native.plan_sync_timeouts() == timeouts_before


@pytest.mark.parametrize("n", [2, 4096, 2048 * 2 * 512, 2048 * 2 * 512 + 6, 5_000_002])
def test_copy_calibration_copies(cuda, n):
    """The yardstick kernel really moves the bytes it is credited with (whole tiles, ragged ends, more tiles
    than resident workgroups)."""
    from lplb_amd import _native
    lib = _native.load()
    src = torch.arange(n, dtype=torch.int64, device=cuda) * 7 - 3
    dst = torch.zeros(n + 2, dtype=torch.int64, device=cuda)
    assert lib.lplb_copy_calibration(src.data_ptr(), dst.data_ptr(), n, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst[:n], src) and int(dst[n]) == 0 and int(dst[n + 1]) == 0


def test_series_aids_equal_single_calls(cuda):
    """lplb_map_idx_prepared_series / lplb_copy_calibration_series are the single calls in a loop."""
    import ctypes
    from lplb_amd import _native
    lib = _native.load()
    shape, _, phy2log, _, _ = reference_style_case(*REFERENCE_SOLVE_CASES[0][1:6], seed=3)
    rng = np.random.default_rng(17)
    solver = solver_for(shape)
    o_weight = dev(_random_weights(shape, rng), cuda)
    d_o2r, d_p2l = dev(shape.o2r, cuda), dev(phy2log, cuda)
    table = solver.prepare_mapping(d_o2r, d_p2l)
    n, n_sms = 40960, 20
    idx = [dev(rng.integers(-1, shape.n_logical, size=n, dtype=np.int64), cuda) for _ in range(3)]
    by = [solver.count_idx(t, n_sms)[1] for t in idx]
    want = [solver.map_idx(t, o_weight, b, d_o2r, d_p2l, n_sms) for t, b in zip(idx, by)]
    out = [torch.full_like(t, -9) for t in idx]
    ptrs = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    rc = lib.lplb_map_idx_prepared_series(ptrs(idx), o_weight.data_ptr(), ptrs(by), table.data_ptr(), n, shape.n_group,
                                          shape.G, shape.D, shape.C, shape.P, n_sms, ptrs(out), 3, None, None, None)
    assert rc == 0, lib.lplb_last_error()
    torch.cuda.synchronize()
    for o, w in zip(out, want):
        assert torch.equal(o, w)
    back = [torch.zeros_like(t) for t in idx]
    assert lib.lplb_copy_calibration_series(ptrs(idx), ptrs(back), n, 3, None, None, None) == 0
    torch.cuda.synchronize()
    for o, w in zip(back, idx):
        assert torch.equal(o, w)
    # the copy in another launch shape, and the histogram kernel without the scan behind it
    back = [torch.zeros_like(t) for t in idx]
    assert lib.lplb_copy_shape_series(ptrs(idx), ptrs(back), n, 3, 4, 256, 1, 0, None, None, None) == 0
    rows = [torch.full_like(b, -3) for b in by]
    assert lib.lplb_slice_histogram_series(ptrs(idx), n, shape.n_logical, n_sms, ptrs(rows), 3, None, None, None) == 0
    torch.cuda.synchronize()
    for o, w in zip(back, idx):
        assert torch.equal(o, w)
    for r, b in zip(rows, by):
        assert torch.equal(torch.cumsum(r, dim=0, dtype=torch.int32), b)
    assert lib.lplb_copy_shape_series(ptrs(idx), ptrs(back), n, 3, 3, 256, 1, 0, None, None, None) == 1   # loads: 1, 2, 4 or 8
    assert lib.lplb_copy_shape_series(ptrs(idx), ptrs(back), n + 2, 3, 4, 256, 1, 0, None, None, None) == 1   # whole tiles only


def test_kernel_timestamp_hook(cuda):
    import ctypes
    inp, shape, solver, t = _plan_setup(cuda, "cpu_ref_ep8")
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipEventCreate(ctypes.byref(a)) == 0 and hip.hipEventCreate(ctypes.byref(b)) == 0
    total, by_sm = solver.count_idx(t["idx"], 16)
    avail = torch.zeros(1, dtype=torch.int32, device=cuda)
    solver.lib.lplb_time_next_launch(a, b)
    res, _ = solver.solve(total.view(1, shape.G, shape.L), t["r2o"], t["phy2log"], avail)
    torch.cuda.synchronize()
    ms = ctypes.c_float()
    assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
    assert 0.0 < ms.value < 5.0 and int(avail[0]) == 1
    # the pair is consumed by one launch: the next call runs untimed and still works
    res2, _ = solver.solve(total.view(1, shape.G, shape.L), t["r2o"], t["phy2log"], avail)
    assert torch.equal(res, res2)


@pytest.mark.parametrize("n,n_experts,n_sms", [(100000, 64, 700), (300000, 20, 1000), (5000, 7, 300)])
def test_count_idx_many_slices(cuda, n, n_experts, n_sms):
    """More than 256 slices: the prefix kernel takes several sweeps with a running carry."""
    rng = np.random.default_rng(n)
    idx = rng.integers(-1, n_experts, size=n, dtype=np.int64)
    solver = CompiledSolver(1, 1, 1, n_experts + 1, 1)
    _, by_sm = solver.count_idx(dev(idx, cuda), n_sms)
    np.testing.assert_array_equal(by_sm.cpu().numpy(), oracle.count_idx(idx, n_experts, n_sms))
