"""Pins the CPU oracle (oracle/lplb_oracle.c) without running the reference:
closed forms, brute force on tiny inputs, invariants the mathematics fixes, an
independent LP optimum from HiGHS, and the properties the reference's own tests
assert (tests/test_idx_processing.py, tests/test_solve.py of the reference)."""
import json
from pathlib import Path

import numpy as np
import pytest
from scipy.optimize import linprog

from lplb_amd import synth, topology
from lplb_amd.mapping import build_redundancy_mapping
from oracle import oracle
from tests.helpers import CASE_SEED, REFERENCE_SOLVE_CASES, Shape, reference_style_case

GOLDEN = Path(__file__).parent / "golden"


# ------------------------------------------------------------------ slicing
@pytest.mark.parametrize("n,size,align", [(0, 4, 256), (1, 4, 256), (1000, 7, 256), (65536, 256, 256),
                                          (65537, 100, 256), (10, 3, 2), (2 ** 31 - 1, 256, 256)])
def test_split_and_align_closed_form(n, size, align):
    per = -(-(-(-n // size)) // align) * align
    bounds = [oracle.split_and_align(n, p, size, align) for p in range(size + 1)]
    assert bounds == [min(n, per * p) for p in range(size + 1)]
    assert bounds[0] == 0 and bounds[-1] == n and all(a <= b for a, b in zip(bounds, bounds[1:]))
    assert all(b % align == 0 or b == n for b in bounds)


# ---------------------------------------------------------------- histogram
@pytest.mark.parametrize("n,n_experts,n_prog", [(4096 * 8, 256, 132), (0, 16, 4), (1, 16, 4), (777, 5, 3),
                                                (100000, 256, 256), (513, 64, 2)])
def test_count_idx_is_bincount_then_cumsum(n, n_experts, n_prog):
    rng = np.random.default_rng(n + n_prog)
    idx = rng.integers(-1, n_experts, size=n, dtype=np.int64)
    got = oracle.count_idx(idx, n_experts, n_prog)
    rows = []
    for p in range(n_prog):
        lo, hi = oracle.split_and_align(n, p, n_prog), oracle.split_and_align(n, p + 1, n_prog)
        part = idx[lo:hi]
        rows.append(np.bincount(part[part >= 0], minlength=n_experts))
    want = np.cumsum(np.array(rows).reshape(n_prog, n_experts), axis=0)
    np.testing.assert_array_equal(got, want)
    # what the reference's test asserts (tests/test_idx_processing.py:37-48)
    assert got[-1].sum() == (idx != -1).sum() and got.min() >= 0
    hist = np.zeros(n_experts + 1, dtype=np.int64)
    np.add.at(hist, idx + 1, 1)
    np.testing.assert_array_equal(got[-1], hist[1:])


# ----------------------------------------------------------------- redirect
def _redirect_by_definition(idx, o_weight, phy2log, r2o, ep_size, n_logical, n_physical):
    """Per-token rule written out in plain Python from the kernel's definition
    (minilp.cu:466-513), with ordinals in index order.  Small inputs only."""
    r2o = np.asarray(r2o)
    G, D = r2o.shape
    L, P = n_logical // ep_size, n_physical // ep_size
    C = (P - L) // D
    o2r = np.argsort(r2o, axis=0, kind="stable")
    total = np.bincount(idx[idx >= 0], minlength=n_logical)
    orig, rep, expected = {}, {}, {e: int(total[e]) for e in range(n_logical)}
    for rank in range(ep_size):
        for s in range(L):
            orig[int(phy2log[rank * P + s])] = rank * P + s
        for s in range(C * D):
            e = int(phy2log[rank * P + s])
            d = s % D
            group, gr = divmod(rank, G)
            w = np.float32(np.asarray(o_weight, np.float32).reshape(-1)[rank * D + d])
            prod = np.float32(w * np.float32(total[e]))
            expected[e] = 0 if np.isnan(prod) else int(np.clip(np.trunc(np.float64(prod)), -2 ** 31, 2 ** 31 - 1))
            rep[e] = (group * G + int(o2r[gr, d]) + 1) * P - C * D + s
    seen = [0] * n_logical
    out = []
    for e in idx:
        if e < 0:
            out.append(-1)
            continue
        k = seen[e]
        seen[e] += 1
        h = (k * 499 + 41) % int(total[e])
        out.append(orig[e] if h < expected[e] else rep.get(e, -1))
    return np.array(out, dtype=np.int64)


def test_redirect_hand_enumerated_case():
    g = json.loads((GOLDEN / "redirect_tiny.json").read_text())
    idx = np.array(g["idx"], dtype=np.int64)
    for n_prog, block in [(1, 256), (3, 2), (5, 2), (2, 4)]:
        by_sm = oracle.count_idx(idx, g["n_logical"], n_prog, block)
        np.testing.assert_array_equal(by_sm[-1], g["totals"])
        out = oracle.map_idx(idx, np.array(g["o_weight"], np.float32), by_sm, np.array(g["o2r"]), g["phy2log"],
                             1, 1, 3, block)
        np.testing.assert_array_equal(out, g["out"])


@pytest.mark.parametrize("seed", range(6))
def test_redirect_matches_definition_on_small_inputs(seed):
    rng = np.random.default_rng(seed)
    r2o, ep, nl, red = [(topology.CUBE_8P2E, 8, 32, 2), (topology.RING_8P, 8, 16, 1),
                        (topology.CUBE_8P2E, 16, 64, 4)][seed % 3]
    hist = rng.integers(1, 1000, size=nl)
    phy2log, _, _ = build_redundancy_mapping(r2o, ep, nl, nl + red * ep, hist)
    s = Shape(np.asarray(r2o), ep, nl, nl + red * ep)
    idx = rng.integers(-1, nl, size=400, dtype=np.int64)
    w = np.clip(rng.standard_normal((s.n_group, s.G, s.D)) / 3 + 0.5, 0, 1).astype(np.float32)
    want = _redirect_by_definition(idx, w, phy2log, r2o, ep, nl, s.n_physical)
    for n_prog in (1, 2, 7):
        by_sm = oracle.count_idx(idx, nl, n_prog)
        got = oracle.map_idx(idx, w, by_sm, s.o2r, phy2log, s.n_group, s.C, s.P)
        np.testing.assert_array_equal(got, want)


def test_redirect_hash_wraps_like_32_bit_int_arithmetic():
    """minilp.cu:505 computes (k * 499 + 41) % total in int: beyond k = 4 303 556 the product wraps to
    negative values and the remainder takes the sign of the dividend.  Restated here in 64-bit
    arithmetic with the wrap and the truncating remainder written out."""
    r2o, ep, nl = np.asarray(topology.RING_8P), 8, 16
    phy2log, _, _ = build_redundancy_mapping(r2o, ep, nl, nl + ep, None)
    s = Shape(r2o, ep, nl, nl + ep)
    heavy = int(np.asarray(phy2log).reshape(ep, s.P)[2, 0])        # has a replica
    n = 5_000_000
    idx = np.full(n, heavy, np.int64)
    idx[::1000] = (heavy + 1) % nl
    w = np.full((1, s.G, s.D), 0.4, np.float32)
    by_sm = oracle.count_idx(idx, nl, 64)
    got = oracle.map_idx(idx, w, by_sm, s.o2r, phy2log, 1, s.C, s.P)
    mine = idx == heavy
    total = int(mine.sum())
    assert total > 4_303_557
    k = np.arange(total, dtype=np.int64)
    h = (k * 499 + 41 + 2 ** 31) % 2 ** 32 - 2 ** 31             # what a 32-bit int holds
    assert h.min() < 0
    rem = np.fmod(h, total)                                       # truncating, sign of the dividend
    expected = int(np.trunc(np.float32(0.4) * np.float32(total)))
    slots = np.unique(got[mine])
    assert len(slots) == 2
    original = 2 * s.P
    replica = int(slots[slots != original][0])
    np.testing.assert_array_equal(got[mine], np.where(rem < expected, original, replica))


def test_redirect_reference_test_properties():
    """tests/test_idx_processing.py:51-138 of the reference, on a numpy draw."""
    name, r2o, nl, ep, red, _, _ = REFERENCE_SOLVE_CASES[0]
    s, _, phy2log, log2phy, _ = reference_style_case(r2o, nl, ep, red, True, seed=42)
    rng = np.random.default_rng(42)
    idx = rng.integers(-1, nl, size=65536, dtype=np.int64)
    w = np.clip(rng.standard_normal((s.n_group, s.G, s.D)) / 3 + 0.5, 0, 1).astype(np.float32)
    by_sm = oracle.count_idx(idx, nl, 132)
    out = oracle.map_idx(idx, w, by_sm, s.o2r, phy2log, s.n_group, s.C, s.P)
    assert out.shape == idx.shape and out.min() >= -1 and out.max() < s.n_physical
    assert np.array_equal(out == -1, idx == -1)
    padded = np.concatenate([np.full((1, 2), -1), log2phy])
    assert np.all((out == padded[idx + 1, 0]) | (out == padded[idx + 1, 1]))
    freq = np.bincount(out[out >= 0], minlength=s.n_physical).reshape(s.n_group, s.G, s.P)
    cd = s.C * s.D
    originals = freq[:, :, :cd].reshape(s.n_group, s.G, s.C, s.D)
    replicas = freq[:, :, s.P - cd:].reshape(s.n_group, s.G, s.C, s.D)
    replicas = np.take_along_axis(replicas, np.broadcast_to(s.o2r[None, :, None, :], replicas.shape), axis=1)
    originals, replicas = originals.sum(2), replicas.sum(2)
    err = np.abs(w * (originals + replicas) - originals) / (originals + replicas)
    assert err.max() < 5e-2
    # exact closed form: clamp(trunc(w * total), 0, total) stay, when 499 does not divide total
    tot = by_sm[-1].astype(np.int64)
    p2l = phy2log.reshape(ep, s.P)
    phys = np.bincount(out[out >= 0], minlength=s.n_physical)
    for rank in range(ep):
        for slot in range(cd):
            e = p2l[rank, slot]
            if tot[e] % 499:
                keep = int(np.clip(np.trunc(np.float32(w.reshape(-1)[rank * s.D + slot % s.D]) * np.float32(tot[e])),
                                   0, tot[e]))
                assert phys[rank * s.P + slot] == keep


# ------------------------------------------------------------------ LP build
@pytest.mark.parametrize("case", REFERENCE_SOLVE_CASES, ids=[c[0] for c in REFERENCE_SOLVE_CASES])
def test_lp_structure(case):
    name, r2o, nl, ep, red, reorder, _ = case
    s, _, phy2log, _, workload = reference_style_case(r2o, nl, ep, red, reorder, seed=CASE_SEED[name])
    G, D = s.G, s.D
    for g in range(s.n_group):
        dupw, b, a, c = oracle.build_lp(workload, s.r2o, phy2log, s.n_group, g, s.C, s.n_fixed)
        NC, NV = a.shape
        assert (NC, NV) == (G + G * D, 2 * G * D + G + 2)
        # Big-M column makes x = 1 feasible (minilp.cu:275-281)
        np.testing.assert_allclose(a.astype(np.float64) @ np.ones(NV), b, atol=2e-6)
        nnz = (a != 0).sum(0)
        assert np.all(nnz[:2 * G * D] == 2) and np.all(nnz[2 * G * D:2 * G * D + G] == 1)
        assert nnz[2 * G * D + G] == G and np.all(a[:G, 2 * G * D + G] == -1)
        # edge rows: x_orig + x_rep - x_M = 1
        for j in range(G * D):
            row = a[G + j]
            assert row[j] == 1 and row[G * D + j] == 1 and row[-1] == -1 and np.count_nonzero(row) == 3
        # rank rows carry the pooled replica-set loads and the fixed load
        gw = oracle.normalise(workload)
        pw = gw[phy2log].reshape(s.n_group, G, s.P)[g]
        np.testing.assert_allclose(dupw, pw[:, :s.C * D].reshape(G, s.C, D).sum(1), rtol=1e-6)
        np.testing.assert_allclose(b[:G], -pw[:, s.C * D:s.L].sum(1), rtol=1e-5)
        for i in range(G):
            for d in range(D):
                assert a[i, i * D + d] == dupw[i, d]
                k = s.r2o[i, d]
                assert a[i, G * D + k * D + d] == dupw[k, d]
        assert np.array_equal(c, np.r_[np.zeros(NV - 2), 1, 1000])


def test_lp_two_rank_case_by_hand():
    # 2 ranks, 1 slot, L = 2: rank 0 = experts {0 (replicated on rank 1), 1}, rank 1 = {2 (on rank 0), 3}
    r2o = np.array([[1], [0]], np.int32)
    phy2log = np.array([0, 1, 2, 2, 3, 0], np.int32)
    workload = np.array([40, 10, 20, 30], np.int32)          # max 40 -> gw = 1, .25, .5, .75
    dupw, b, a, c = oracle.build_lp(workload, r2o, phy2log, 1, 0, 1, 1)
    np.testing.assert_array_equal(dupw.reshape(-1), [1.0, 0.5])
    np.testing.assert_array_equal(b, [-0.25, -0.75, 1, 1])
    want = np.array([
        # xo0  xo1  xr0  xr1  s0  s1   t    M
        [1.0, 0.0, 0.0, 0.5, 1, 0, -1, -0.25 - 1.5],
        [0.0, 0.5, 1.0, 0.0, 0, 1, -1, -0.75 - 1.5],
        [1.0, 0.0, 1.0, 0.0, 0, 0, 0, -1],
        [0.0, 1.0, 0.0, 1.0, 0, 0, 0, -1]], np.float32)
    np.testing.assert_array_equal(a, want)


# -------------------------------------------------------------------- solver
def _highs_optimum(workload, s, phy2log, g):
    _, b, a, c = oracle.build_lp(workload, s.r2o, phy2log, s.n_group, g, s.C, s.n_fixed)
    NV = a.shape[1]
    r = linprog(c[:NV - 1].astype(float), A_eq=a[:, :NV - 1].astype(float), b_eq=b.astype(float),
                bounds=[(0, None)] * (NV - 1), method="highs")
    assert r.status == 0
    return r.fun


@pytest.mark.parametrize("case", REFERENCE_SOLVE_CASES, ids=[c[0] for c in REFERENCE_SOLVE_CASES])
@pytest.mark.parametrize("precision", [32, 64])
def test_solver_invariants_and_optimum(case, precision):
    name, r2o, nl, ep, red, reorder, tol = case
    s, _, phy2log, _, workload = reference_style_case(r2o, nl, ep, red, reorder, seed=CASE_SEED[name])
    G, D, n = s.G, s.D, s.G * s.D
    # rounding lets the fp32 iterate drift off A x = b (its own feasibility test allows 0.05)
    drift = 2e-3 if precision == 32 else 2e-6   # (A, b below are the fp32 build)
    for n_steps in (1, 3, 5):
        res, gw, avail, x, trace, resid = oracle.solve(workload, s.r2o, phy2log, s.n_group, s.C, s.n_fixed,
                                                       step_rule=1, n_steps=n_steps, precision=precision, details=True)
        for g in range(s.n_group):
            _, b, a, _ = oracle.build_lp(workload, s.r2o, phy2log, s.n_group, g, s.C, s.n_fixed)
            # affine scaling never leaves the affine set A x = b
            np.testing.assert_allclose(a.astype(np.float64) @ x[g].astype(np.float64), b, atol=drift)
            np.testing.assert_allclose(x[g, :n] + x[g, n:2 * n] - x[g, -1], 1, atol=drift)
            assert np.all(x[g] > 0)                       # full-max rule keeps x interior
        # the objective t + 1000 x_M never increases
        obj = trace[:, :, 2] + 1000 * trace[:, :, 3]
        assert np.all(np.diff(np.concatenate([np.full((s.n_group, 1), 1001.0), obj], axis=1), axis=1) <= 1e-3)
    assert avail == s.n_group
    # after 5 steps t is within 1.5 % of the true optimum and never below it
    for g in range(s.n_group):
        opt = _highs_optimum(workload, s, phy2log, g)
        assert opt - 1e-5 <= x[g, -2] <= opt * 1.015, (g, opt, x[g, -2])
    # the reference's acceptance test: balance after redirecting (tests/test_solve.py:58-89)
    res, _, avail = oracle.solve(workload, s.r2o, phy2log, s.n_group, s.C, s.n_fixed, precision=precision)
    loads = oracle.rank_loads(workload, res, s.r2o, phy2log, s.n_group, s.C)
    assert avail == s.n_group and loads.max() / loads.mean() < tol


def test_solver_t_equals_realised_max_load():
    """x_t (never returned by the reference) is the max rank load the returned shares realise."""
    name, r2o, nl, ep, red, reorder, _ = REFERENCE_SOLVE_CASES[0]
    s, _, phy2log, _, workload = reference_style_case(r2o, nl, ep, red, reorder)
    res, _, _, x, _, _ = oracle.solve(workload, s.r2o, phy2log, s.n_group, s.C, s.n_fixed, details=True, precision=64)
    loads = oracle.rank_loads(workload, res, s.r2o, phy2log, s.n_group, s.C)
    np.testing.assert_allclose(loads.max(1), x[:, -2] * workload.max(), rtol=2e-3)


def test_solver_symmetric_workload_gives_symmetric_answer():
    r2o = topology.CUBE_8P2E
    phy2log, _, _ = build_redundancy_mapping(r2o, 8, 64, 80)
    workload = np.full(64, 1000, np.int32)
    res, _, avail = oracle.solve(workload, r2o, phy2log, 1, 1, 6, precision=64)
    assert avail == 1 and np.ptp(res) < 1e-6
    loads = oracle.rank_loads(workload, res, r2o, phy2log, 1, 1)
    np.testing.assert_allclose(loads, 8000, rtol=1e-6)
    # In fp32 this already-balanced input converges by step 4; d_max falls to 1e-5, alpha = 0.999 / d_max
    # reaches 7e4 and amplifies rounding noise until the feasibility test rejects the iterate.  Whether
    # it does depends on the arithmetic order, so only the returned shares are bounded here.
    res32, _, avail32 = oracle.solve(workload, r2o, phy2log, 1, 1, 6, precision=32)
    assert avail32 in (0, 1) and np.abs(res32 - 0.5).max() < 2e-2


def test_solver_two_rank_closed_form():
    # rank 0: movable 60 + fixed 30, rank 1: movable 10 + fixed 20 -> optimum equalises at 60 each
    r2o = np.array([[1], [0]], np.int32)
    phy2log = np.array([0, 1, 2, 2, 3, 0], np.int32)
    workload = np.array([60, 30, 10, 20], np.int32)
    res, _, avail = oracle.solve(workload, r2o, phy2log, 1, 1, 1, precision=64)
    loads = oracle.rank_loads(workload, res, r2o, phy2log, 1, 1)
    assert avail == 1
    assert loads.max() <= 60 * 1.01 and abs(loads.sum() - 120) < 1e-6


def test_solver_fallback_and_nan():
    name, r2o, nl, ep, red, reorder, _ = REFERENCE_SOLVE_CASES[0]
    s, _, phy2log, _, workload = reference_style_case(r2o, nl, ep, red, reorder)
    res, _, avail = oracle.solve(workload, s.r2o, phy2log, s.n_group, s.C, s.n_fixed, n_steps=1, avail=5)
    assert np.all(res == 0.5) and avail == 5
    res, gw, avail = oracle.solve(np.zeros(nl, np.int32), s.r2o, phy2log, s.n_group, s.C, s.n_fixed, avail=5)
    assert np.all(res == 0.5) and avail == 5 and np.isnan(gw).all()
    res, _, avail = oracle.solve(workload, s.r2o, phy2log, s.n_group, s.C, s.n_fixed, avail=5)
    assert avail == 5 + s.n_group


def test_solver_window_rule_matches_full_rule_when_window_holds_the_maximum():
    # NV = 42 for the EP8 cube: the last 32 columns hold every slack, t, the Big-M column and most flows
    inp = synth.make_inputs("v3_ep8_cube", tokens=8)
    c = inp.cfg
    s = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    a = oracle.solve(inp.global_counts, c.r2o, inp.phy2log, 1, s.C, s.n_fixed, step_rule=0)[0]
    b = oracle.solve(inp.global_counts, c.r2o, inp.phy2log, 1, s.C, s.n_fixed, step_rule=1)[0]
    np.testing.assert_array_equal(a, b)


def test_solver_fp32_tracks_fp64():
    for name in ("cpu_ref_ep8", "v3_ep8_cube"):
        inp = synth.make_inputs(name, tokens=8)
        c = inp.cfg
        s = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
        r32 = oracle.solve(inp.global_counts, c.r2o, inp.phy2log, 1, s.C, s.n_fixed)[0]
        r64 = oracle.solve(inp.global_counts, c.r2o, inp.phy2log, 1, s.C, s.n_fixed, precision=64)[0]
        assert np.abs(r32 - r64).max() < 1e-3


def test_window_rule_chaos_fixture_is_what_it_says():
    """tests/golden/window_chaos_ring64.json: under the reference's step rule (d_max over the last 32
    columns, minilp.cu:355-359) the exact iteration leaves [0, 1] by far, stays 'feasible', keeps
    A x = b (x_o + x_r - x_M = 1 on every edge) -- and its fp32 evaluation drifts beyond the parity
    tolerance; with the maximum over all columns the same input is tame."""
    case = json.loads((Path(__file__).parent / "golden" / "window_chaos_ring64.json").read_text())
    r2o = np.asarray(case["r2o"], np.int32).reshape(64, 1)
    phy2log, wl = np.asarray(case["phy2log"], np.int32), np.asarray(case["workload"], np.int32)
    r64, _, ok64, x, _, _ = oracle.solve(wl, r2o, phy2log, 1, 1, 0, precision=64, details=True)
    r32, _, ok32 = oracle.solve(wl, r2o, phy2log, 1, 1, 0)
    assert ok64 == ok32 == 1 and r64.min() < -50 and r64.max() > 40
    x = x[0]
    np.testing.assert_allclose(x[:64] + x[64:128] - x[-1], 1.0, atol=1e-9)
    args = (r2o, phy2log, 1, 1)
    drift = np.abs(oracle.edge_flows(wl, r32, *args) - oracle.edge_flows(wl, r64, *args)).max() / wl.sum()
    assert 1e-4 < drift < 1e-2
    tame = oracle.solve(wl, r2o, phy2log, 1, 1, 0, precision=64, step_rule=1)[0]
    assert 0 <= tame.min() and tame.max() <= 1


@pytest.mark.parametrize("name", ["cpu_ref_ep8", "v3_ep8_cube", "ep16_hypercube"])
def test_torch_restatement_agrees_with_the_c_restatement(name):
    """oracle/torch_plan.py (the multi-threaded CPU baseline that bench.py times) against
    lplb_oracle.c: histogram and redirect bit for bit, LP shares to fp32 rounding."""
    import torch
    from oracle import torch_plan
    inp = synth.make_inputs(name, mask_fraction=0.05, tokens=600)
    c = inp.cfg
    s = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    idx = torch.from_numpy(inp.indices)
    by = torch_plan.count_idx(idx, c.n_logical, 7)
    want_by = oracle.count_idx(inp.indices, c.n_logical, 7)
    np.testing.assert_array_equal(by.numpy(), want_by)
    lp = torch_plan.DenseLp(c.r2o, s.C, s.n_fixed)
    dupw, b, a, cost = oracle.build_lp(inp.global_counts, c.r2o, inp.phy2log, s.n_group, 0, s.C, s.n_fixed)
    gw = torch.from_numpy(oracle.normalise(inp.global_counts))
    A, bb = lp.build(gw, torch.from_numpy(inp.phy2log.reshape(s.n_group, s.G, s.P)[0].astype(np.int64)))
    np.testing.assert_allclose(A.numpy(), a, atol=2e-6)
    np.testing.assert_allclose(bb.numpy(), b, atol=1e-6)
    np.testing.assert_array_equal(lp.c.numpy(), cost)
    res, gw2, n_ok = torch_plan.solve(torch.from_numpy(inp.global_counts), lp, torch.from_numpy(inp.phy2log), s.n_group)
    want, want_gw, want_ok = oracle.solve(inp.global_counts, c.r2o, inp.phy2log, s.n_group, s.C, s.n_fixed)
    np.testing.assert_array_equal(gw2.numpy(), want_gw)
    assert n_ok == want_ok == s.n_group
    args = (c.r2o, inp.phy2log, s.n_group, s.C)
    flow = np.abs(oracle.edge_flows(inp.global_counts, res.numpy(), *args) - oracle.edge_flows(inp.global_counts, want, *args))
    assert flow.max() <= 1e-3 * inp.global_counts.sum()     # two fp32 evaluations of an ill-conditioned iteration
    out = torch_plan.map_idx(idx, torch.from_numpy(want), by, torch.from_numpy(s.o2r), torch.from_numpy(inp.phy2log),
                             s.n_group, s.C, s.P)
    want_out = oracle.map_idx(inp.indices, want, want_by, s.o2r, inp.phy2log, s.n_group, s.C, s.P)
    np.testing.assert_array_equal(out.numpy(), want_out)
