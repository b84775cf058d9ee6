"""Writes tests/golden/window_chaos_ring64.json: the one input of a 228 000-LP differential run
(random replica permutations, Dirichlet workloads) on which the GPU solver ended further than
1e-4 of the tokens from the fp64 oracle.  It is the first draw of the random-topology generator
of tests/test_gpu_parity.py::test_solve_random_topologies for (G, D, C, n_group) = (64, 1, 1, 1)
with its seed advanced by 7919 * 371.  Nothing of the reference is involved; the file is data
from numpy's generator."""
import json
from pathlib import Path

import numpy as np

G, D, C = 64, 1, 1
rng = np.random.default_rng(1000 * G + 10 * D + C + 7919 * 371)
r2o = np.stack([rng.permutation(G) for _ in range(D)], axis=1).astype(np.int32)
per_rank = D * C + int(rng.integers(0, 5))
assert per_rank == 1
nl = G * per_rank
originals = rng.permutation(nl).reshape(G, per_rank)
phy2log = np.empty((G, per_rank + C * D), np.int32)
phy2log[:, :per_rank] = originals
for rank in range(G):
    phy2log[rank, per_rank] = originals[r2o[rank, 0], 0]
p = rng.dirichlet(np.full(nl, 0.3))
wl = rng.multinomial(int(rng.choice([2000, 1 << 17, 1 << 22])), p).astype(np.int32)
wl[rng.integers(nl)] += 1
out = {"r2o": r2o.reshape(-1).tolist(), "phy2log": phy2log.reshape(-1).tolist(), "workload": wl.tolist()}
Path(__file__).with_name("window_chaos_ring64.json").write_text(json.dumps(out) + "\n")
print("tokens", int(wl.sum()))
