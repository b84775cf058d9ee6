"""Replica topologies (``r2o`` matrices).

``r2o[i, d] = k`` means: the d-th replica slot of group-rank ``i`` holds a copy of
the d-th to-be-replicated expert set of group-rank ``k``.  Every column must be a
permutation of ``0..G-1`` so that each replica edge joins exactly two ranks.

The constants are the reference's published topologies (data, tests/utils.py:97-119
of the reference).
"""
from __future__ import annotations

import numpy as np

# Cube with diagonals on 8 ranks, 2 replicas per rank (tests/utils.py:97-102).
CUBE_8P2E = np.array(
    [[3, 0, 1, 2, 7, 4, 5, 6],
     [6, 7, 4, 5, 0, 1, 2, 3]], dtype=np.int32).T.copy()

# Ring on 8 ranks, 1 replica per rank (tests/utils.py:103-107).
RING_8P = np.array([[1, 2, 3, 4, 5, 6, 7, 0]], dtype=np.int32).T.copy()

# Hypercube on 16 ranks without diagonals, 2 replicas per rank (tests/utils.py:108-113).
HYPERCUBE_16P2E = np.array(
    [[3, 0, 1, 2, 7, 4, 5, 6, 11, 8, 9, 10, 15, 12, 13, 14],
     [12, 13, 14, 15, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11]], dtype=np.int32).T.copy()


def torus_2d(m: int, n: int) -> np.ndarray:
    """m x n torus: slot 0 copies from the next row, slot 1 from the next column
    (tests/utils.py:116-119)."""
    i, j = np.divmod(np.arange(m * n), n)
    return np.stack([((i + 1) % m) * n + j, i * n + (j + 1) % n], axis=1).astype(np.int32)


def is_valid_r2o(r2o: np.ndarray) -> bool:
    """True when every column is a permutation of 0..G-1."""
    r2o = np.asarray(r2o)
    if r2o.ndim != 2:
        return False
    G = r2o.shape[0]
    return all(np.array_equal(np.sort(r2o[:, d]), np.arange(G)) for d in range(r2o.shape[1]))
