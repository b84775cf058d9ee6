"""Writes tests/golden/eplb_vectors.json: inputs and outputs of the reference's EPLB
entry point for a handful of small seeded cases.

Run in the build container only (it needs the reference checkout):

    python tests/golden/make_eplb_vectors.py /root/reference

The reference module is pure PyTorch on CPU; it is loaded by file path because the
package's __init__ pulls in its CUDA extension.  Only data (weights in, index maps
out) is written to the fixture.
"""
import importlib.util
import json
import sys
from pathlib import Path

import numpy as np
import torch

# (n_logical, num_replicas, num_groups, num_nodes, num_gpus)
CASES = [
    (32, 32, 1, 1, 8),      # reorder only, global policy
    (256, 256, 4, 4, 32),   # reorder only, hierarchical (the planner's EP32 call)
    (256, 256, 1, 8, 8),    # groups not divisible by nodes -> global policy
    (64, 64, 8, 2, 16),     # hierarchical, several groups per node
    (32, 40, 4, 2, 8),      # with replication
    (64, 80, 1, 1, 16),     # replication, global policy
]


def _primes(lo: int, count: int) -> np.ndarray:
    out, k = [], lo
    while len(out) < count:
        if all(k % d for d in range(2, int(k ** 0.5) + 1)):
            out.append(k)
        k += 1
    return np.array(out, dtype=np.int64)


PRIMES = _primes(101, 1024)


def main(ref_root: str) -> None:
    spec = importlib.util.spec_from_file_location("ref_eplb", Path(ref_root) / "lplb" / "eplb.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = []
    for case_id, (n_log, n_rep, n_groups, n_nodes, n_gpus) in enumerate(CASES):
        rng = np.random.default_rng(100 + case_id)
        layers = 2
        # distinct primes: exactly representable in float32, and no two experts can tie
        # even after their loads are divided by their replica counts
        weight = np.stack([rng.permutation(PRIMES)[:n_log] for _ in range(layers)])
        phy2log, log2phy, logcnt = mod.rebalance_experts(torch.from_numpy(weight), n_rep, n_groups, n_nodes, n_gpus)
        out.append({
            "n_logical": n_log, "num_replicas": n_rep, "num_groups": n_groups, "num_nodes": n_nodes,
            "num_gpus": n_gpus, "weight": weight.tolist(), "phy2log": phy2log.tolist(),
            "log2phy": log2phy.tolist(), "logcnt": logcnt.tolist(),
        })
    path = Path(__file__).with_name("eplb_vectors.json")
    path.write_text(json.dumps(out))
    print(f"wrote {path} ({path.stat().st_size} bytes, {len(out)} cases)")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
