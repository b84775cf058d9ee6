"""TEST INFRASTRUCTURE ONLY: the reference's per-batch plan restated with PyTorch CPU
tensor operations (bincount / cumsum, a dense fp32 constraint matrix, torch.linalg.cholesky
and cholesky_solve, a vectorised redirect).  It exists to be TIMED beside the GPU path as the
multi-threaded CPU baseline of bench.py (the scalar C restatement in lplb_oracle.c is the
single-threaded one and the parity checker); tests/test_oracle.py holds it against that C
restatement.  The product package never imports it.

Follows lplb/resources/csrc-tmpl/minilp.cu of the reference: count :410-443, LP build
:203-293, five affine-scaling steps :331-367, feasibility :369-400, redirect :445-515.
"""
from __future__ import annotations

import numpy as np
import torch


def count_idx(idx: torch.Tensor, n_experts: int, n_prog: int, block: int = 256) -> torch.Tensor:
    """int32 [n_prog, n_experts]: occurrences of each expert in slices 0..p (minilp.cu:404-443)."""
    flat = idx.reshape(-1)
    n = flat.numel()
    per = -(-n // n_prog)
    per = -(-per // block) * block
    valid = (flat >= 0) & (flat < n_experts)
    pos = torch.arange(n, dtype=torch.int64)
    key = (pos // max(per, 1)) * n_experts + flat
    rows = torch.bincount(key[valid], minlength=n_prog * n_experts).reshape(n_prog, n_experts)
    return rows.cumsum(0).to(torch.int32)


class DenseLp:
    """Index pattern of the dense constraint matrix of one group (minilp.cu:236-293), built once."""

    def __init__(self, r2o: np.ndarray, n_per_var: int, n_fixed: int):
        r2o = np.asarray(r2o, np.int64)
        self.G, self.D = G, D = r2o.shape
        self.C, self.n_fixed = n_per_var, n_fixed
        self.L = D * n_per_var + n_fixed
        self.P = self.L + D * n_per_var
        self.NC, self.NV = G + G * D, 2 * G * D + G + 2
        n = G * D
        i = np.repeat(np.arange(G), D)
        d = np.tile(np.arange(D), G)
        self.own = (torch.from_numpy(i), torch.from_numpy(i * D + d))                    # row i, column x_orig(i, d)
        src = r2o[i, d]
        self.copy = (torch.from_numpy(i), torch.from_numpy(n + src * D + d))             # row i, column x_rep(src, d)
        self.copy_src = torch.from_numpy(src * D + d)
        self.r2o = torch.from_numpy(r2o)
        c = torch.zeros(self.NV, dtype=torch.float32)
        c[self.NV - 2], c[self.NV - 1] = 1.0, 1000.0
        self.c = c

    def build(self, gw: torch.Tensor, p2l: torch.Tensor):
        """gw fp32 [n_experts] normalised counts, p2l int64 [G, P] of this group -> (A, b)."""
        G, D, C, n = self.G, self.D, self.C, self.G * self.D
        pw = gw[p2l]                                                    # [G, P]
        dupw = pw[:, :C * D].reshape(G, C, D).sum(1).reshape(-1)        # [G * D], index i * D + d
        fixed = pw[:, C * D:C * D + self.n_fixed]
        b = torch.ones(self.NC, dtype=torch.float32)
        acc = torch.zeros(G, dtype=torch.float32)
        for j in range(self.n_fixed):                                   # sequential fp32 subtraction, :225-229
            acc = acc - fixed[:, j]
        b[:G] = acc
        A = torch.zeros(self.NC, self.NV, dtype=torch.float32)
        A[self.own] = dupw
        A.index_put_(self.copy, dupw[self.copy_src], accumulate=True)   # a self-loop adds to the same row
        r = torch.arange(G)
        A[r, 2 * n + r] = 1.0
        A[:G, 2 * n + G] = -1.0
        e = torch.arange(n)
        A[G + e, e] = 1.0
        A[G + e, n + e] = 1.0
        A[:, self.NV - 1] = b - A[:, :self.NV - 1].sum(1)
        return A, b


def solve(counts: torch.Tensor, lp: DenseLp, phy2log: torch.Tensor, n_group: int, n_steps: int = 5,
          step_rule: int = 0):
    """counts int32 [n_logical] -> (shares fp32 [n_group, G, D], normalised counts, feasible groups)."""
    gw = counts.to(torch.float32) / counts.max().to(torch.float32)
    G, D, NV = lp.G, lp.D, lp.NV
    out = torch.empty(n_group, G, D, dtype=torch.float32)
    n_ok = 0
    p2l = phy2log.reshape(n_group, G, lp.P).to(torch.int64)
    lo = max(0, NV - 32) if step_rule == 0 else 0
    for g in range(n_group):
        A, b = lp.build(gw, p2l[g])
        x = torch.ones(NV, dtype=torch.float32)
        d_max = torch.zeros((), dtype=torch.float32)
        for _ in range(n_steps):
            ax2 = A * (x * x)
            m = ax2 @ A.T
            rhs = ax2 @ lp.c
            chol, info = torch.linalg.cholesky_ex(m)
            w = torch.cholesky_solve(rhs[:, None], chol)[:, 0]
            d = x * (lp.c - A.T @ w)
            d_max = d[lo:].max()
            if step_rule != 0 or NV < 32:
                d_max = torch.clamp_min(d_max, 0.0)
            alpha = (0.999 / d_max.double()).float()
            x = x * (1 - alpha * d)
        res = (A @ x - b).abs().max()
        ok = bool(d_max.double() < 0.1) and bool(0 <= x[-1].double() < 1e-4) and bool(res.double() < 0.05)
        n_ok += ok
        out[g] = x[:G * D].reshape(G, D) if ok else 0.5
    return out, gw, n_ok


def map_idx(idx: torch.Tensor, o_weight: torch.Tensor, by_sm: torch.Tensor, o2r: torch.Tensor,
            phy2log: torch.Tensor, n_group: int, n_combined: int, n_local: int) -> torch.Tensor:
    """Redirect with ordinals in flat index order (minilp.cu:445-515); no hash wrap (n < 4.3 M)."""
    G, D = o2r.shape
    cd = n_combined * D
    L = n_local - cd
    nl = n_group * G * L
    total = by_sm[-1].to(torch.int64)
    p2l = phy2log.to(torch.int64)
    e = torch.arange(nl)
    slot = (e // L) * n_local + e % L
    original = torch.full((nl,), -1, dtype=torch.int64)
    original[p2l[slot]] = slot
    replica = torch.full((nl,), -1, dtype=torch.int64)
    expected = total.clone()
    i = torch.arange(n_group * G * cd)
    ep_rank, place = i // max(cd, 1), i % max(cd, 1)
    le = p2l[ep_rank * n_local + place]
    share = o_weight.reshape(-1)[ep_rank * D + place % D]
    expected[le] = (share * total[le].to(torch.float32)).to(torch.int32).to(torch.int64)   # truncation toward zero
    host = o2r.to(torch.int64)[ep_rank % G, place % D]
    replica[le] = ((ep_rank // G) * G + host + 1) * n_local - cd + place
    flat = idx.reshape(-1)
    valid = (flat >= 0) & (flat < nl)
    ev = torch.where(valid, flat, torch.zeros_like(flat))
    # ordinal = number of earlier tokens of the same expert: position inside the expert's run of a stable sort
    order = torch.argsort(torch.where(valid, flat, torch.full_like(flat, nl)), stable=True)
    sorted_e = torch.where(valid, flat, torch.full_like(flat, nl))[order]
    run_start = torch.searchsorted(sorted_e, torch.arange(nl + 1))
    k = torch.empty_like(flat)
    k[order] = torch.arange(flat.numel()) - run_start[sorted_e]
    t = total[ev].clamp_min(1)
    h = torch.where(total[ev] > 0, (k * 499 + 41) % t, torch.zeros_like(k))
    out = torch.where(h >= expected[ev], replica[ev], original[ev])
    return torch.where(valid, out, torch.full_like(out, -1)).reshape(idx.shape)
