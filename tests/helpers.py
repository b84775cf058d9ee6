"""Shared builders for the parity tests: reference-test-style workloads
(tests/test_solve.py:40-49 of the reference draws them from the CUDA generator,
which cannot be reproduced, so the same distributions are drawn from numpy)."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from lplb_amd import topology
from lplb_amd.mapping import build_redundancy_mapping

# (name, r2o, n_logical, ep_size, redundants per rank, reorder, balance tolerance):
# the reference's solver test matrix, tests/test_solve.py:16-21.
REFERENCE_SOLVE_CASES = [
    ("cube8_ep32", topology.CUBE_8P2E, 256, 32, 2, True, 1.07),
    ("cube8_ep32_c2", topology.CUBE_8P2E, 256, 32, 4, False, 1.07),
    ("cube8_ep64", topology.CUBE_8P2E, 256, 64, 2, True, 1.1),
    ("ring8_ep32", topology.RING_8P, 256, 32, 1, True, 1.07),
    ("hypercube16", topology.HYPERCUBE_16P2E, 256, 16, 2, True, 1.03),
    ("torus8x4", topology.torus_2d(8, 4), 256, 32, 2, False, 1.01),
]
# The balance tolerances above hold for the reference's CUDA-generator draw.  For a
# numpy draw they hold only when the LP optimum itself admits them (a ring with one
# replica cannot flatten every draw), so each case uses a seed whose HiGHS optimum
# is inside the tolerance.
CASE_SEED = {"cube8_ep32": 42, "cube8_ep32_c2": 42, "cube8_ep64": 42, "ring8_ep32": 3,
             "hypercube16": 42, "torus8x4": 42}


@dataclass
class Shape:
    r2o: np.ndarray
    ep_size: int
    n_logical: int
    n_physical: int

    @property
    def G(self): return self.r2o.shape[0]
    @property
    def D(self): return self.r2o.shape[1]
    @property
    def n_group(self): return self.ep_size // self.G
    @property
    def L(self): return self.n_logical // self.ep_size
    @property
    def P(self): return self.n_physical // self.ep_size
    @property
    def C(self): return (self.P - self.L) // self.D
    @property
    def n_fixed(self): return self.L - self.C * self.D
    @property
    def o2r(self): return np.argsort(self.r2o, axis=0, kind="stable").astype(np.int32)


def reference_style_case(r2o, n_logical, ep_size, red, reorder, seed=42, gpus_per_node=8):
    """History ~ N(1, 0.15) * 2^20 and batch workload ~ N(1, 0.3) * 2^12, clamped at 0."""
    rng = np.random.default_rng(seed)
    shape = Shape(np.asarray(r2o, np.int32), ep_size, n_logical, n_logical + red * ep_size)
    hist = None
    if reorder:
        hist = (np.clip(rng.standard_normal(n_logical) * 0.15 + 1, 0, None) * 2 ** 20).astype(np.int64)
    phy2log, log2phy, logcnt = build_redundancy_mapping(shape.r2o, ep_size, n_logical, shape.n_physical, hist,
                                                        n_nodes=max(1, ep_size // gpus_per_node))
    workload = (np.clip(rng.standard_normal(n_logical) * 0.3 + 1, 0, None) * 2 ** 12).astype(np.int32)
    return shape, hist, phy2log, log2phy, workload
