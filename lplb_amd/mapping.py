"""Physical <-> logical expert layout of the planner (host side, numpy).

Per EP rank the physical slots are laid out as

    [ C*D originals that have a replica (slot = c*D + d) | n_fixed other originals | C*D replicas ]

where replica slot ``(c, d)`` of group-rank ``i`` copies original slot ``(c, d)`` of
group-rank ``r2o[i, d]``.  This is the layout the solver and redirect kernels index
(reference: lplb/planner.py:115-182).
"""
from __future__ import annotations

import numpy as np

from .eplb import rebalance_experts


def build_redundancy_mapping(r2o: np.ndarray, ep_size: int, n_logical: int, n_physical: int,
                             workload: np.ndarray | None = None, n_nodes: int = 1):
    """Returns (phy2log int32 [n_physical], log2phy int32 [n_logical, 2], logcnt int32 [n_logical]).

    workload: optional per-logical-expert history.  When given, experts are first
    spread over ranks with EPLB (reorder only, no replication) and each rank's
    experts are sorted heaviest first, so the heaviest C*D of every rank get the
    replicas (lplb/planner.py:127-147).  Equal histories keep index order.
    Raises AssertionError unless every logical expert ends up with at most one
    replica and at least one expert has one (lplb/planner.py:173).
    """
    r2o = np.asarray(r2o, dtype=np.int64)
    G, D = r2o.shape
    n_group = ep_size // G
    L = n_logical // ep_size
    P = n_physical // ep_size
    C = (P - L) // D

    if workload is None:
        nored = np.arange(n_logical, dtype=np.int64)
    else:
        workload = np.asarray(workload).reshape(-1)
        assert workload.size == n_logical
        nored = rebalance_experts(workload[None].astype(np.float32), n_logical, n_group,
                                  n_nodes, ep_size)[0][0]
    nored = nored.reshape(n_group, G, L)
    if workload is not None:
        order = np.argsort(-workload[nored].astype(np.float64), axis=-1, kind="stable")
        nored = np.take_along_axis(nored, order, axis=-1)

    tored = nored[:, :, :C * D].reshape(n_group, G, C, D)
    # replica (c, d) on rank i <- original (c, d) of rank r2o[i, d]
    dup = tored[:, r2o, :, np.arange(D)[None, :]]          # [G, D, n_group, C]
    dup = dup.transpose(2, 0, 3, 1)                        # [n_group, G, C, D]
    phy2log = np.concatenate([nored, dup.reshape(n_group, G, C * D)], axis=-1).reshape(-1)
    assert phy2log.shape[0] == n_physical, (phy2log.shape, n_physical)

    # log2phy lists originals before replicas: walk physical ids by (local slot, rank).
    by_slot = np.arange(n_physical).reshape(ep_size, P).T.reshape(-1)
    logs = phy2log[by_slot]
    order = np.argsort(logs, kind="stable")
    logcnt = np.bincount(logs, minlength=n_logical)
    max_cnt = int(logcnt.max())
    assert max_cnt == 2, f"every logical expert may have at most one replica (got {max_cnt} copies)"
    starts = np.cumsum(logcnt) - logcnt
    sorted_logs = logs[order]
    pos = np.arange(order.size) - starts[sorted_logs]
    log2phy = np.full((n_logical, max_cnt), -1, dtype=np.int32)
    log2phy[sorted_logs, pos] = by_slot[order]
    return phy2log.astype(np.int32), log2phy, logcnt.astype(np.int32)
