"""Static expert placement (EPLB) used by ``Planner.update_redundancy_mapping``.

Host-side numpy code; it runs once per re-shuffle, never per batch.  Behaviour
follows the reference's embedded EPLB (lplb/eplb.py:6-190): greedy
longest-processing-time packing into equally sized packs, optional replication of
the currently heaviest expert, and the hierarchical groups -> nodes -> GPUs
policy.  All weights are handled in float32 like there.

Tie-breaking: items of equal weight are taken in index order (stable sort) and
a tie between packs goes to the lowest pack index.  The reference leaves the
first to an unstable sort, so results can differ from it only when weights tie.
"""
from __future__ import annotations

import numpy as np


def balanced_packing(weight: np.ndarray, num_packs: int) -> tuple[np.ndarray, np.ndarray]:
    """Pack n weighted items into ``num_packs`` packs of exactly n/num_packs items,
    heaviest first, each into the lightest pack that still has room
    (lplb/eplb.py:6-46).

    weight: [X, n].  Returns (pack_index [X, n], rank_in_pack [X, n]), int64.
    """
    weight = np.asarray(weight, dtype=np.float32)
    n_layers, n_items = weight.shape
    assert n_items % num_packs == 0
    cap = n_items // num_packs
    if cap == 1:
        pack_index = np.broadcast_to(np.arange(n_items, dtype=np.int64), weight.shape).copy()
        return pack_index, np.zeros_like(pack_index)

    order = np.argsort(-weight, axis=-1, kind="stable")
    pack_index = np.full(weight.shape, -1, dtype=np.int64)
    rank_in_pack = np.full(weight.shape, -1, dtype=np.int64)
    for layer in range(n_layers):
        load = np.zeros(num_packs, dtype=np.float32)
        fill = np.zeros(num_packs, dtype=np.int64)
        for item in order[layer]:
            masked = np.where(fill < cap, load, np.float32(np.inf))
            pack = int(np.argmin(masked))
            pack_index[layer, item] = pack
            rank_in_pack[layer, item] = fill[pack]
            load[pack] += weight[layer, item]
            fill[pack] += 1
    return pack_index, rank_in_pack


def replicate_experts(weight: np.ndarray, num_phy: int) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Add ``num_phy - num_log`` replicas, each time to the expert whose
    per-replica load is currently largest (lplb/eplb.py:49-77).

    Returns (phy2log [X, num_phy], replica rank [X, num_phy], logcnt [X, num_log]).
    """
    weight = np.asarray(weight, dtype=np.float32)
    n, num_log = weight.shape
    assert num_phy >= num_log
    phy2log = np.tile(np.arange(num_phy, dtype=np.int64), (n, 1))
    rank = np.zeros((n, num_phy), dtype=np.int64)
    logcnt = np.ones((n, num_log), dtype=np.int64)
    rows = np.arange(n)
    for slot in range(num_log, num_phy):
        pick = np.argmax(weight / logcnt.astype(np.float32), axis=-1)
        phy2log[:, slot] = pick
        rank[:, slot] = logcnt[rows, pick]
        logcnt[rows, pick] += 1
    return phy2log, rank, logcnt


def _inverse_perm(perm: np.ndarray) -> np.ndarray:
    inv = np.empty_like(perm)
    np.put_along_axis(inv, perm, np.broadcast_to(np.arange(perm.shape[1]), perm.shape), axis=1)
    return inv


def rebalance_experts_hierarchical(weight: np.ndarray, num_physical_experts: int, num_groups: int,
                                   num_nodes: int, num_gpus: int):
    """Groups -> nodes, replicate inside nodes, physical experts -> GPUs
    (lplb/eplb.py:80-148).  Returns (phy2log, phyrank, logcnt), each [layers, ...]."""
    weight = np.asarray(weight, dtype=np.float32)
    n_layers, n_log = weight.shape
    assert n_log % num_groups == 0
    group_size = n_log // num_groups
    assert num_groups % num_nodes == 0
    groups_per_node = num_groups // num_nodes
    assert num_gpus % num_nodes == 0
    assert num_physical_experts % num_gpus == 0
    phy_per_gpu = num_physical_experts // num_gpus

    # 1. whole expert groups onto nodes
    tokens_per_group = weight.reshape(n_layers, num_groups, group_size).sum(-1, dtype=np.float32)
    g_pack, g_rank = balanced_packing(tokens_per_group, num_nodes)
    log2mlog = (((g_pack * groups_per_node + g_rank) * group_size)[..., None]
                + np.arange(group_size, dtype=np.int64)).reshape(n_layers, -1)
    mlog2log = _inverse_perm(log2mlog)

    # 2. replicas inside each node
    log_per_node = n_log // num_nodes
    tokens_per_mlog = np.take_along_axis(weight, mlog2log, axis=-1).reshape(-1, log_per_node)
    phy2mlog, phyrank, mlogcnt = replicate_experts(tokens_per_mlog, num_physical_experts // num_nodes)

    # 3. physical experts onto the node's GPUs
    tokens_per_phy = np.take_along_axis(tokens_per_mlog / mlogcnt.astype(np.float32), phy2mlog, axis=-1)
    p_pack, p_rank = balanced_packing(tokens_per_phy, num_gpus // num_nodes)
    phy2pphy = p_pack * phy_per_gpu + p_rank
    pphy2phy = _inverse_perm(phy2pphy)

    pphy2mlog = np.take_along_axis(phy2mlog, pphy2phy, axis=-1)
    pphy2mlog = (pphy2mlog.reshape(n_layers, num_nodes, -1)
                 + (np.arange(num_nodes, dtype=np.int64) * log_per_node)[None, :, None]
                 ).reshape(n_layers, -1)
    pphy2log = np.take_along_axis(mlog2log, pphy2mlog, axis=-1)
    pphyrank = np.take_along_axis(phyrank, pphy2phy, axis=-1).reshape(n_layers, -1)
    logcnt = np.take_along_axis(mlogcnt.reshape(n_layers, -1), log2mlog, axis=-1)
    return pphy2log, pphyrank, logcnt


def rebalance_experts(weight: np.ndarray, num_replicas: int, num_groups: int, num_nodes: int,
                      num_gpus: int):
    """Entry point (lplb/eplb.py:151-190).  weight: [layers, num_logical].
    Returns (phy2log [layers, num_replicas], log2phy [layers, num_logical, X],
    logcnt [layers, num_logical]), int64."""
    weight = np.asarray(weight, dtype=np.float32)
    n_layers, n_log = weight.shape
    if num_groups % num_nodes == 0:
        phy2log, phyrank, logcnt = rebalance_experts_hierarchical(
            weight, num_replicas, num_groups, num_nodes, num_gpus)
    else:
        phy2log, phyrank, logcnt = rebalance_experts_hierarchical(
            weight, num_replicas, 1, 1, num_gpus)
    max_cnt = int(logcnt.max())
    log2phy = np.full((n_layers, n_log * max_cnt), -1, dtype=np.int64)
    np.put_along_axis(log2phy, phy2log * max_cnt + phyrank,
                      np.broadcast_to(np.arange(num_replicas, dtype=np.int64), phy2log.shape), axis=-1)
    return phy2log, log2phy.reshape(n_layers, n_log, max_cnt), logcnt
