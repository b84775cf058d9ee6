"""Seeded synthetic planning workloads (numpy, host side) shared by the benchmark
and the parity tests, so that the HIP path and its CPU checker see identical bytes.

Every configuration is an EP deployment described by a replica topology plus a
token-routing distribution:

* expert popularity ``p_e ~ rank_e^-s`` (Zipf) with ranks assigned by a seeded
  permutation, optionally with a few hot experts raised to 10x the mean;
* a per-batch multiplicative lognormal jitter;
* global per-expert counts (the solver's input) drawn multinomially for the
  whole EP group, ``ep_size * tokens * topk`` tokens;
* this GPU's share of the routing decisions, int64 ``[tokens, topk]`` with
  ``topk`` distinct experts per row (Gumbel top-k), optionally with masked (-1)
  entries.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from . import topology
from .mapping import build_redundancy_mapping


@dataclass
class PlanConfig:
    name: str
    r2o: np.ndarray
    ep_size: int
    n_logical: int
    redundants_per_rank: int
    tokens: int
    topk: int
    zipf_s: float
    jitter_sigma: float = 0.0
    hot_experts: int = 0
    seed: int = 0

    @property
    def n_physical(self) -> int:
        return self.n_logical + self.redundants_per_rank * self.ep_size


CONFIGS: dict[str, PlanConfig] = {
    # 8 simulated ranks, 32 logical experts, top-2 of 1024 tokens
    "cpu_ref_ep8": PlanConfig("cpu_ref_ep8", topology.CUBE_8P2E, 8, 32, 2, 1024, 2, 1.2, seed=1001),
    # DeepSeek-V3 MoE shape on an EP8 cube
    "v3_ep8_cube": PlanConfig("v3_ep8_cube", topology.CUBE_8P2E, 8, 256, 2, 8192, 8, 1.0,
                              jitter_sigma=0.3, seed=1002),
    "ep16_hypercube": PlanConfig("ep16_hypercube", topology.HYPERCUBE_16P2E, 16, 256, 2, 4096, 8, 1.1,
                                 seed=1003),
    "ep32_torus": PlanConfig("ep32_torus", topology.torus_2d(8, 4), 32, 256, 2, 16384, 8, 1.5,
                             hot_experts=3, seed=1004),
    # redirect half of the throughput sweep (its 2048 LP instances come from sweep_counts)
    "sweep_redirect": PlanConfig("sweep_redirect", topology.CUBE_8P2E, 8, 256, 2, 262144, 8, 1.0,
                                 jitter_sigma=0.3, seed=1005),
}


@dataclass
class PlanInputs:
    cfg: PlanConfig
    popularity: np.ndarray          # float64 [n_logical], sums to 1
    batch_p: np.ndarray             # float64 [n_logical], sums to 1
    global_counts: np.ndarray       # int32 [n_logical]
    indices: np.ndarray             # int64 [tokens, topk]
    phy2log: np.ndarray             # int32 [n_physical]
    log2phy: np.ndarray             # int32 [n_logical, 2]
    extras: dict = field(default_factory=dict)


def popularity(cfg: PlanConfig, rng: np.random.Generator) -> np.ndarray:
    ranks = rng.permutation(cfg.n_logical) + 1
    p = ranks.astype(np.float64) ** (-cfg.zipf_s)
    p /= p.sum()
    if cfg.hot_experts:
        hot = rng.choice(cfg.n_logical, size=cfg.hot_experts, replace=False)
        p[hot] = 10.0 / cfg.n_logical
        p /= p.sum()
    return p


def batch_distribution(cfg: PlanConfig, p: np.ndarray, rng: np.random.Generator) -> np.ndarray:
    if cfg.jitter_sigma > 0:
        q = p * rng.lognormal(0.0, cfg.jitter_sigma, size=p.shape)
        return q / q.sum()
    return p.copy()


def draw_indices(q: np.ndarray, tokens: int, topk: int, rng: np.random.Generator,
                 mask_fraction: float = 0.0, chunk: int = 32768) -> np.ndarray:
    """Rows of ``topk`` distinct experts drawn without replacement ~ q (Gumbel top-k)."""
    out = np.empty((tokens, topk), dtype=np.int64)
    logq = np.log(q)
    for lo in range(0, tokens, chunk):
        hi = min(tokens, lo + chunk)
        keys = logq[None, :] + rng.gumbel(size=(hi - lo, q.size))
        part = np.argpartition(-keys, topk - 1, axis=1)[:, :topk]
        order = np.argsort(-np.take_along_axis(keys, part, axis=1), axis=1)
        out[lo:hi] = np.take_along_axis(part, order, axis=1)
    if mask_fraction > 0:
        out[rng.random(out.shape) < mask_fraction] = -1
    return out


def make_inputs(cfg: PlanConfig | str, *, mask_fraction: float = 0.0, reorder: bool = True,
                tokens: int | None = None) -> PlanInputs:
    if isinstance(cfg, str):
        cfg = CONFIGS[cfg]
    rng = np.random.default_rng(cfg.seed)
    p = popularity(cfg, rng)
    q = batch_distribution(cfg, p, rng)
    n_tok = cfg.tokens if tokens is None else tokens
    counts = rng.multinomial(cfg.ep_size * cfg.tokens * cfg.topk, q).astype(np.int32)
    idx = draw_indices(q, n_tok, cfg.topk, rng, mask_fraction)
    history = np.round(p * 2 ** 24).astype(np.int64) if reorder else None
    phy2log, log2phy, _ = build_redundancy_mapping(cfg.r2o, cfg.ep_size, cfg.n_logical,
                                                   cfg.n_physical, history, n_nodes=1)
    return PlanInputs(cfg, p, q, counts, idx, phy2log, log2phy)


def sweep_counts(n_instances: int = 2048, base: PlanConfig | str = "v3_ep8_cube") -> np.ndarray:
    """Independent per-batch global count vectors, int32 [n_instances, n_logical]:
    instance i redraws the jitter and the multinomial with seed 2000 + i around the
    base configuration's popularity."""
    if isinstance(base, str):
        base = CONFIGS[base]
    p = popularity(base, np.random.default_rng(base.seed))
    out = np.empty((n_instances, base.n_logical), dtype=np.int32)
    for i in range(n_instances):
        rng = np.random.default_rng(2000 + i)
        q = batch_distribution(base, p, rng)
        out[i] = rng.multinomial(base.ep_size * base.tokens * base.topk, q)
    return out
