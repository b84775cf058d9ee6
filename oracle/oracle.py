"""TEST INFRASTRUCTURE ONLY: numpy front-end to the C restatement in
``lplb_oracle.c`` (see that file's header for what each function follows in the
reference and how it is pinned).  Importable from ``tests/``, the smoke check and
the benchmark's cpu_baseline leg; the product package never imports it.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "liblplb_oracle.so"
_lib = None

_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(ctypes.c_float)


def build() -> Path:
    """Compile the C oracle with the Makefile beside it."""
    subprocess.run(["make", "-C", str(_HERE), "-B", "liblplb_oracle.so"], check=True,
                   capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        _lib = ctypes.CDLL(str(_LIB_PATH))
        _lib.lplb_oracle_split_and_align.restype = ctypes.c_int
        _lib.lplb_oracle_split_and_align.argtypes = [ctypes.c_int] * 4
    return _lib


def _p(a: np.ndarray, typ):
    return a.ctypes.data_as(typ)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a), dtype=np.int32)


def split_and_align(n: int, rank: int, size: int, align: int = 256) -> int:
    return lib().lplb_oracle_split_and_align(n, rank, size, align)


def count_idx(idx: np.ndarray, n_experts: int, n_prog: int, block: int = 256) -> np.ndarray:
    """Inclusive per-slice prefix of the expert histogram, int32 [n_prog, n_experts]."""
    idx = np.ascontiguousarray(idx, dtype=np.int64).reshape(-1)
    out = np.zeros((n_prog, n_experts), dtype=np.int32)
    lib().lplb_oracle_count_idx(_p(idx, _i64p), ctypes.c_int(idx.size), ctypes.c_int(n_experts),
                                ctypes.c_int(n_prog), ctypes.c_int(block), _p(out, _i32p))
    return out


def normalise(workload: np.ndarray) -> np.ndarray:
    w = _i32(workload).reshape(-1)
    gw = np.zeros(w.size, dtype=np.float32)
    lib().lplb_oracle_normalise(_p(w, _i32p), ctypes.c_int(w.size), _p(gw, _f32p))
    return gw


def lp_dims(G: int, D: int) -> tuple[int, int]:
    return G + G * D, 2 * G * D + G + 2


def build_lp(workload, r2o, phy2log, n_group: int, group: int, n_per_var: int, n_fixed: int):
    """Dense (dupw, b, A, c) of one group's LP in fp32."""
    r2o = _i32(r2o)
    G, D = r2o.shape
    NC, NV = lp_dims(G, D)
    w = _i32(workload).reshape(-1)
    p2l = _i32(phy2log).reshape(-1)
    dupw = np.zeros(G * D, np.float32)
    b = np.zeros(NC, np.float32)
    a = np.zeros((NC, NV), np.float32)
    c = np.zeros(NV, np.float32)
    lib().lplb_oracle_build_lp(_p(w, _i32p), _p(r2o, _i32p), _p(p2l, _i32p), ctypes.c_int(n_group),
                               ctypes.c_int(group), ctypes.c_int(G), ctypes.c_int(D),
                               ctypes.c_int(n_per_var), ctypes.c_int(n_fixed), _p(dupw, _f32p),
                               _p(b, _f32p), _p(a, _f32p), _p(c, _f32p))
    return dupw.reshape(G, D), b, a, c


def solve(workload, r2o, phy2log, n_group: int, n_per_var: int, n_fixed: int, *,
          avail: int = 0, step_rule: int = 0, n_steps: int = 5, precision: int = 32,
          details: bool = False):
    """Returns (result [n_group,G,D] f32, global_workload f32, avail) and, with
    details=True, additionally x [n_group,NV], trace [n_group,n_steps,4] and
    residual [n_group] in the working precision."""
    r2o = _i32(r2o)
    G, D = r2o.shape
    _, NV = lp_dims(G, D)
    w = _i32(workload).reshape(-1)
    p2l = _i32(phy2log).reshape(-1)
    L = D * n_per_var + n_fixed
    assert w.size == n_group * G * L, (w.size, n_group, G, L)
    assert p2l.size == n_group * G * (L + D * n_per_var)
    gw = np.zeros(w.size, np.float32)
    res = np.zeros((n_group, G, D), np.float32)
    av = np.array([avail], np.int32)
    ft = np.float64 if precision == 64 else np.float32
    x = np.zeros((n_group, NV), ft)
    tr = np.zeros((n_group, max(n_steps, 1), 4), ft)
    rs = np.zeros(n_group, ft)
    lib().lplb_oracle_solve(_p(w, _i32p), _p(gw, _f32p), _p(r2o, _i32p), _p(p2l, _i32p),
                            ctypes.c_int(n_group), ctypes.c_int(G), ctypes.c_int(D),
                            ctypes.c_int(n_per_var), ctypes.c_int(n_fixed), _p(av, _i32p),
                            _p(res, _f32p), ctypes.c_int(step_rule), ctypes.c_int(n_steps),
                            ctypes.c_int(precision), x.ctypes.data_as(ctypes.c_void_p),
                            tr.ctypes.data_as(ctypes.c_void_p), rs.ctypes.data_as(ctypes.c_void_p))
    if details:
        return res, gw, int(av[0]), x, tr, rs
    return res, gw, int(av[0])


def map_idx(idx, o_weight, by_sm, o2r, phy2log, n_group: int, n_combined: int, n_local: int,
            block: int = 256) -> np.ndarray:
    idx = np.ascontiguousarray(idx, dtype=np.int64)
    flat = idx.reshape(-1)
    o2r = _i32(o2r)
    G, D = o2r.shape
    ow = np.ascontiguousarray(o_weight, dtype=np.float32).reshape(-1)
    assert ow.size == n_group * G * D
    by_sm = _i32(by_sm)
    n_prog = by_sm.shape[0]
    assert by_sm.shape[1] == n_group * G * (n_local - D * n_combined)
    p2l = _i32(phy2log).reshape(-1)
    assert p2l.size == n_group * G * n_local
    out = np.empty_like(flat)
    lib().lplb_oracle_map_idx(_p(flat, _i64p), _p(ow, _f32p), _p(by_sm, _i32p), _p(o2r, _i32p),
                              _p(p2l, _i32p), ctypes.c_int(flat.size), ctypes.c_int(n_group),
                              ctypes.c_int(G), ctypes.c_int(D), ctypes.c_int(n_combined),
                              ctypes.c_int(n_local), ctypes.c_int(n_prog), ctypes.c_int(block),
                              _p(out, _i64p))
    return out.reshape(idx.shape)


def rank_loads(workload, probs, r2o, phy2log, n_group: int, n_per_var: int) -> np.ndarray:
    """Per-rank load after balancing, in tokens, float64 [n_group, G] -- the closed
    form the reference's solver test evaluates (tests/test_solve.py:60-84)."""
    r2o = np.asarray(r2o, dtype=np.int64)
    G, D = r2o.shape
    w = np.asarray(workload, dtype=np.float64).reshape(-1)
    pw = w[np.asarray(phy2log).reshape(-1)].reshape(n_group, G, -1)
    cd = n_per_var * D
    dup = pw[:, :, :cd].reshape(n_group, G, n_per_var, D).sum(2)
    p = np.asarray(probs, dtype=np.float64).reshape(n_group, G, D)
    moved = dup * (1 - p)
    recv = np.take_along_axis(moved, np.broadcast_to(r2o, p.shape), axis=1)
    fixed = pw[:, :, cd:pw.shape[2] - cd].sum(2)
    return (dup * p + recv).sum(2) + fixed


def edge_flows(workload, probs, r2o, phy2log, n_group: int, n_per_var: int) -> np.ndarray:
    """Tokens sent along each replica edge (k, d): (1 - p[k,d]) * w[k,d]."""
    r2o = np.asarray(r2o)
    G, D = r2o.shape
    w = np.asarray(workload, dtype=np.float64).reshape(-1)
    pw = w[np.asarray(phy2log).reshape(-1)].reshape(n_group, G, -1)
    dup = pw[:, :, :n_per_var * D].reshape(n_group, G, n_per_var, D).sum(2)
    return (1 - np.asarray(probs, dtype=np.float64).reshape(n_group, G, D)) * dup


def compare_batch(workloads, got, r2o, phy2log, n_group: int, n_per_var: int, n_fixed: int, *,
                  step_rule: int = 0, n_steps: int = 5):
    """Checks a batch of independent solves against this oracle (fp32).  workloads int32
    [N, n_logical], got fp32 [N, n_group, G, D].  Returns (largest edge-flow difference as a
    fraction of the instance's token count, largest relative objective difference, number of
    feasible (instance, group) pairs according to the oracle)."""
    workloads = np.asarray(workloads)
    got = np.asarray(got)
    worst_flow = worst_obj = 0.0
    n_ok = 0
    for w, res in zip(workloads, got):
        ref, _, ok = solve(w, r2o, phy2log, n_group, n_per_var, n_fixed, step_rule=step_rule, n_steps=n_steps)
        n_ok += ok
        args = (r2o, phy2log, n_group, n_per_var)
        flow = np.abs(edge_flows(w, res, *args) - edge_flows(w, ref, *args)).max() / float(w.sum(dtype=np.float64))
        obj_ref = rank_loads(w, ref, *args).max(axis=1)
        obj = rank_loads(w, res, *args).max(axis=1)
        worst_flow = max(worst_flow, float(flow))
        worst_obj = max(worst_obj, float((np.abs(obj - obj_ref) / obj_ref).max()))
    return worst_flow, worst_obj, n_ok
