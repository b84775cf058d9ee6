"""ctypes binding of ``liblplb_hip.so`` and the ``CompiledSolver`` facade the planner
talks to.  The facade keeps the method names, argument order, return values and
argument checks of the reference's pybind11 class (csrc/plugin.cpp:459-470,
491-660); underneath it only forwards device pointers and the current stream to
the C ABI declared in ``include/lplb_hip.h``.

There is no CPU or pure-PyTorch fallback: if the shared library is missing or a
tensor is not on a GPU, the call raises.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import torch

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / "liblplb_hip.so"
ABI_VERSION = 7
# limits of lplb_count_totals (LPLB_COUNT_TOTALS_MAX_* of include/lplb_hip.h)
COUNT_TOTALS_MAX_INDICES = 131072
COUNT_TOTALS_MAX_EXPERTS = 1024

STEP_REFERENCE_WINDOW = 0
STEP_FULL_MAX = 1
REFERENCE_STEPS = 5

_lib: ctypes.CDLL | None = None

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64

_SIGNATURES = {
    "lplb_abi_version": (_i, []),
    "lplb_last_error": (ctypes.c_char_p, []),
    "lplb_time_next_launch": (None, [_vp, _vp]),
    "lplb_copy_calibration": (_i, [_vp, _vp, _i64, _vp]),
    "lplb_copy_calibration_series": (_i, [_vp, _vp, _i64, _i, _vp, _vp, _vp]),
    "lplb_slice_histogram_series": (_i, [_vp, _i64, _i, _i, _vp, _i, _vp, _vp, _vp]),
    "lplb_copy_shape_series": (_i, [_vp, _vp, _i64, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "lplb_map_idx_prepared_series": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp]),
    "lplb_count_idx": (_i, [_vp, _i64, _i, _i, _vp, _vp]),
    "lplb_count_totals": (_i, [_vp, _i64, _i, _vp, _vp]),
    "lplb_count_totals_add": (_i, [_vp, _i64, _i, _vp, _vp, _vp]),
    "lplb_solve": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _vp]),
    "lplb_solve_batched": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _vp]),
    "lplb_map_idx": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "lplb_prepared_mapping_bytes": (_i64, [_i, _i, _i, _i, _i]),
    "lplb_prepare_mapping": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _i64, _vp]),
    "lplb_map_idx_prepared": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "lplb_plan_set_cooperative": (_i, [_i]),
    "lplb_plan_forget_captured": (_i, [_vp]),
    "lplb_plan_sync_timeouts": (_i, [_vp]),
    "lplb_plan_poll_timeouts": (_i, [_vp, _vp]),
    "lplb_plan_one_launch_count": (_i, [_vp]),
    "lplb_plan_inject_fault": (_i, [_i, _i]),
    "lplb_plan": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "lplb_plan_noalloc": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
}


def build(verbose: bool = False) -> Path:
    """Compile the HIP library for gfx950 with the Makefile in ``csrc/``."""
    proc = subprocess.run(["make", "-C", str(_PKG / "csrc"), "-B", "-j4"], capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(proc.stdout)
        print(proc.stderr)
    if proc.returncode != 0:
        raise RuntimeError("building liblplb_hip.so failed")
    return LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {_PKG / 'csrc'}` "
            "(hipcc, --offload-arch=gfx950). There is no fallback path.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.lplb_abi_version() != ABI_VERSION:
        raise RuntimeError(f"liblplb_hip.so has ABI {lib.lplb_abi_version()}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def exported_symbols() -> list[str]:
    return list(_SIGNATURES)


def set_plan_cooperative(enabled: bool) -> None:
    """Let ``plan`` run short batches as one kernel launch (default) or always as the chain of kernels."""
    _check(load().lplb_plan_set_cooperative(1 if enabled else 0))


def plan_forget_captured(stream: "torch.cuda.Stream") -> None:
    """Give back the share of the GPU that one-launch plans captured on ``stream`` keep reserved; for callers
    who have destroyed every graph that holds such a plan."""
    _check(load().lplb_plan_forget_captured(stream.cuda_stream))


def plan_sync_timeouts() -> int:
    """Waits between workgroups of the one-launch plan that ran out on the current device (0 when healthy)."""
    count = ctypes.c_int(-1)
    _check(load().lplb_plan_sync_timeouts(ctypes.byref(count)))
    return count.value


def plan_poll_timeouts(dst: torch.Tensor, stream: int | None = None) -> None:
    """Enqueue the health report: dst (two int32, on the GPU or in pinned host memory) receives the number of
    waits that ran out on the current device and the number of blocks of counters switched off."""
    _require(dst.dtype == torch.int32 and dst.numel() >= 2 and dst.is_contiguous() and (dst.is_cuda or dst.is_pinned()),
             "dst: two int32 on the GPU or in pinned host memory")
    _check(load().lplb_plan_poll_timeouts(dst.data_ptr(), stream))


def plan_one_launch_count() -> int:
    """Plans of this process that ran as one kernel launch (the others ran the chain of kernels)."""
    count = ctypes.c_longlong(-1)
    _check(load().lplb_plan_one_launch_count(ctypes.byref(count)))
    return count.value


class UnsupportedShape(RuntimeError):
    """The library has no kernel for this shape (LPLB_EUNSUPPORTED)."""


def _check(rc: int) -> None:
    if rc != 0:
        kind = UnsupportedShape if rc == 2 else RuntimeError
        raise kind(f"lplb_hip error {rc}: {load().lplb_last_error().decode()}")


def _require(cond: bool, what: str) -> None:
    if not cond:
        raise RuntimeError(f"LPLB assertion failed: {what}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """Handle of torch's current stream on t's device (the raw query is ten times cheaper than
    building a torch.cuda.Stream object, which matters at 10 us per plan)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class CompiledSolver:
    """Launches the three planning kernels for one (n_group, G, D, P, C) shape."""

    def __init__(self, *args, **kwargs) -> None:
        """Two ways to construct one.  The reference's own argument list (csrc/plugin.cpp:665-667,
        as lplb/planner.py:26-35 passes it):
            CompiledSolver(resource_path, n_group, group_size, dup_per_rank, block_dim,
                           n_local_experts, n_combined_experts, pg)
        where resource_path (the CUDA templates' folder) and block_dim (every kernel here picks its
        own workgroup size) are accepted and ignored and pg is kept as .pg for the caller; or the
        five numbers that matter:
            CompiledSolver(n_group, group_size, dup_per_rank, n_local_experts, n_combined_experts)"""
        self.pg = None
        if args and isinstance(args[0], (str, bytes)) or "resource_path" in kwargs:
            names = ("resource_path", "n_group", "group_size", "dup_per_rank", "block_dim", "n_local_experts",
                     "n_combined_experts", "pg")
        else:
            names = ("n_group", "group_size", "dup_per_rank", "n_local_experts", "n_combined_experts")
        if len(args) > len(names):
            raise TypeError(f"CompiledSolver takes {len(names)} arguments {names}, got {len(args)}")
        given = dict(zip(names, args))
        for k, v in kwargs.items():
            if k not in names or k in given:
                raise TypeError(f"CompiledSolver: unexpected or repeated argument {k!r}")
            given[k] = v
        missing = [k for k in names if k not in given and k != "pg"]
        if missing:
            raise TypeError(f"CompiledSolver: missing arguments {missing}")
        n_group, group_size, dup_per_rank = int(given["n_group"]), int(given["group_size"]), int(given["dup_per_rank"])
        n_local_experts, n_combined_experts = int(given["n_local_experts"]), int(given["n_combined_experts"])
        self.pg = given.get("pg")
        self.lib = load()
        self.n_group = n_group
        self.group_size = group_size
        self.dup_per_rank = dup_per_rank
        self.n_local_experts = n_local_experts
        self.n_combined_experts = n_combined_experts
        # csrc/plugin.cpp:464-466
        self.n_experts = (n_local_experts - dup_per_rank * n_combined_experts) * group_size * n_group
        self.step_rule = STEP_REFERENCE_WINDOW
        self.n_steps = REFERENCE_STEPS

    # -- csrc/plugin.cpp:491-578 -------------------------------------------------
    def solve(self, local_workload: torch.Tensor, r2o: torch.Tensor, phy2log: torch.Tensor,
              avail_num: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        _require(local_workload.is_cuda, "local_workload on a GPU")
        _require(local_workload.dim() == 3, "local_workload.dim() == 3")
        n_group = local_workload.size(0)
        _require(self.group_size == local_workload.size(1), "group_size == local_workload.size(1)")
        n_logical_per_rank = local_workload.size(2)
        n_pes = n_group * self.group_size
        _require(local_workload.dtype == torch.int32, "local_workload.dtype == int32")
        _require(local_workload.is_contiguous(), "local_workload.is_contiguous()")
        _require(r2o.dim() == 2 and r2o.size(0) == self.group_size and r2o.size(1) == self.dup_per_rank,
                 "r2o is [group_size, dup_per_rank]")
        _require(r2o.dtype == torch.int32, "r2o.dtype == int32")
        _require(phy2log.dim() == 1 and phy2log.size(0) % n_pes == 0, "phy2log is 1-D, a multiple of the EP size")
        _require(phy2log.dtype == torch.int32, "phy2log.dtype == int32")
        n_physical_per_rank = phy2log.size(0) // n_pes
        _require((n_physical_per_rank - n_logical_per_rank) % self.dup_per_rank == 0,
                 "replicas per rank divisible by dup_per_rank")
        n_per_var = (n_physical_per_rank - n_logical_per_rank) // self.dup_per_rank
        n_fixed = n_logical_per_rank - self.dup_per_rank * n_per_var
        _require(avail_num.numel() == 1, "avail_num.numel() == 1")
        _require(avail_num.dtype == torch.int32, "avail_num.dtype == int32")
        _require(r2o.is_cuda and phy2log.is_cuda and avail_num.is_cuda, "all tensors on the GPU")
        r2o = r2o.contiguous()
        phy2log = phy2log.contiguous()
        avail_num = avail_num if avail_num.is_contiguous() else avail_num.contiguous()

        global_workload = torch.empty_like(local_workload, dtype=torch.float32)
        result = torch.empty((n_group, self.group_size, self.dup_per_rank), dtype=torch.float32,
                             device=local_workload.device)
        _check(self.lib.lplb_solve(local_workload.data_ptr(), global_workload.data_ptr(), r2o.data_ptr(),
                                   phy2log.data_ptr(), n_group, self.group_size, self.dup_per_rank,
                                   n_per_var, n_fixed, avail_num.data_ptr(), result.data_ptr(),
                                   self.step_rule, self.n_steps, _stream(local_workload)))
        return result, global_workload

    def solve_batched(self, workloads: torch.Tensor, r2o: torch.Tensor, phy2log: torch.Tensor,
                      avail_num: torch.Tensor, want_global: bool = False):
        """workloads int32 [n_instances, n_group, G, L] -> result fp32 [n_instances, n_group, G, D]."""
        _require(workloads.is_cuda and workloads.dim() == 4 and workloads.dtype == torch.int32
                 and workloads.is_contiguous(), "workloads is a contiguous int32 [N, n_group, G, L] GPU tensor")
        n_inst, n_group, g, n_logical_per_rank = workloads.shape
        _require(g == self.group_size, "group_size == workloads.size(2)")
        n_pes = n_group * g
        _require(phy2log.dtype == torch.int32 and phy2log.dim() == 1 and phy2log.size(0) % n_pes == 0,
                 "phy2log is int32, 1-D, a multiple of the EP size")
        _require(r2o.dtype == torch.int32 and tuple(r2o.shape) == (g, self.dup_per_rank), "r2o is int32 [G, D]")
        _require(avail_num.numel() == 1 and avail_num.dtype == torch.int32, "avail_num is one int32")
        n_per_var = (phy2log.size(0) // n_pes - n_logical_per_rank) // self.dup_per_rank
        n_fixed = n_logical_per_rank - self.dup_per_rank * n_per_var
        result = torch.empty((n_inst, n_group, g, self.dup_per_rank), dtype=torch.float32, device=workloads.device)
        gw = torch.empty_like(workloads, dtype=torch.float32) if want_global else None
        _check(self.lib.lplb_solve_batched(workloads.data_ptr(), gw.data_ptr() if want_global else None,
                                           r2o.contiguous().data_ptr(), phy2log.contiguous().data_ptr(),
                                           n_inst, n_group, g, self.dup_per_rank, n_per_var, n_fixed,
                                           avail_num.data_ptr(), result.data_ptr(), self.step_rule,
                                           self.n_steps, _stream(workloads)))
        return (result, gw) if want_global else result

    # -- csrc/plugin.cpp:580-600 -------------------------------------------------
    def count_idx(self, idx: torch.Tensor, n_sms: int, block_dim: int = 256, *,
                  out: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """out: optional int32 [n_sms, n_experts] table to fill instead of a new one (no counterpart in the
        reference, which allocates on every call)."""
        _require(idx.dtype == torch.int64, "idx.dtype == int64")
        _require(idx.is_cuda, "idx.device().is_cuda()")
        _require(idx.is_contiguous(), "idx.is_contiguous()")
        _require(block_dim == 256, "slices are aligned to 256 indices")
        if out is None:
            out = torch.empty((n_sms, self.n_experts), dtype=torch.int32, device=idx.device)
        else:
            _require(out.dtype == torch.int32 and out.is_cuda and out.is_contiguous() and
                     tuple(out.shape) == (n_sms, self.n_experts), "out: int32 [n_sms, n_experts], contiguous, on the GPU")
        _check(self.lib.lplb_count_idx(idx.data_ptr(), idx.numel(), self.n_experts, n_sms, out.data_ptr(),
                                       _stream(idx)))
        return out[-1], out

    def count_totals(self, idx: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """This GPU's tokens per logical expert (what count_idx returns first) without the table per slice, in
        one kernel launch; short batches only (UnsupportedShape beyond 131072 indices or 1024 experts).  No
        counterpart in the reference."""
        _require(idx.dtype == torch.int64 and idx.is_cuda and idx.is_contiguous(), "idx is a contiguous int64 GPU tensor")
        if out is None:
            out = torch.empty(self.n_experts, dtype=torch.int32, device=idx.device)
        else:
            _require(out.dtype == torch.int32 and out.is_cuda and out.is_contiguous() and out.numel() == self.n_experts,
                     "out: int32 [n_experts], contiguous, on the GPU")
        _check(self.lib.lplb_count_totals(idx.data_ptr(), idx.numel(), self.n_experts, out.data_ptr(), _stream(idx)))
        return out

    def count_totals_add(self, idx: torch.Tensor, totals: torch.Tensor, clear: torch.Tensor | None = None) -> torch.Tensor:
        """Adds this GPU's tokens per logical expert to ``totals`` (which the caller has zeroed), one kernel launch
        of a few workgroups (short batches only: UnsupportedShape beyond 131072 indices); the same launch sets
        ``clear`` to zero, so a caller that swaps two vectors from call to call never zeroes one itself.  No
        counterpart in the reference."""
        _require(idx.dtype == torch.int64 and idx.is_cuda and idx.is_contiguous(), "idx is a contiguous int64 GPU tensor")
        for name, t in (("totals", totals), ("clear", clear)):
            _require(t is None or (t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and
                                   t.numel() == self.n_experts and t.device == idx.device),
                     f"{name}: int32 [n_experts], contiguous, on idx's GPU")
        _check(self.lib.lplb_count_totals_add(idx.data_ptr(), idx.numel(), self.n_experts, totals.data_ptr(),
                                              None if clear is None else clear.data_ptr(), _stream(idx)))
        return totals

    # -- csrc/plugin.cpp:602-660 -------------------------------------------------
    def map_idx(self, mapping_idx: torch.Tensor, o_weight: torch.Tensor, local_workload_split_by_sm: torch.Tensor,
                o2r: torch.Tensor, phy2log: torch.Tensor, n_sms: int, block_dim: int = 256,
                physical_counts: torch.Tensor | None = None, prepared: torch.Tensor | None = None) -> torch.Tensor:
        """prepared: optional table from prepare_mapping(o2r, phy2log) (no counterpart in the reference,
        which rebuilds it in every block); the result is the same with and without it."""
        _require(mapping_idx.dtype == torch.int64, "mapping_idx.dtype == int64")
        _require(mapping_idx.is_cuda, "mapping_idx.device().is_cuda()")
        _require(mapping_idx.is_contiguous(), "mapping_idx.is_contiguous()")
        _require(o_weight.dtype == torch.float32, "o_weight.dtype == float32")
        _require(o_weight.is_cuda and o_weight.is_contiguous(), "o_weight is a contiguous GPU tensor")
        _require(o_weight.dim() == 3 and tuple(o_weight.shape) == (self.n_group, self.group_size, self.dup_per_rank),
                 "o_weight is [n_group, group_size, dup_per_rank]")
        _require(o2r.dtype == torch.int32 and o2r.is_cuda and o2r.is_contiguous(), "o2r is a contiguous int32 GPU tensor")
        _require(o2r.dim() == 2 and tuple(o2r.shape) == (self.group_size, self.dup_per_rank),
                 "o2r is [group_size, dup_per_rank]")
        _require(phy2log.dtype == torch.int32 and phy2log.is_cuda and phy2log.is_contiguous(),
                 "phy2log is a contiguous int32 GPU tensor")
        _require(phy2log.dim() == 1 and phy2log.size(0) == self.group_size * self.n_group * self.n_local_experts,
                 "phy2log.size(0) == group_size * n_group * n_local_experts")
        by_sm = local_workload_split_by_sm
        _require(by_sm.dtype == torch.int32 and by_sm.is_cuda and by_sm.is_contiguous()
                 and tuple(by_sm.shape) == (n_sms, self.n_experts),
                 "local_workload_split_by_sm is a contiguous int32 [n_sms, n_experts] GPU tensor")
        _require(block_dim == 256, "slices are aligned to 256 indices")
        self._check_physical_counts(physical_counts)
        out = torch.empty_like(mapping_idx)
        if prepared is not None:
            _require(prepared.dtype == torch.int32 and prepared.is_cuda and prepared.is_contiguous()
                     and prepared.numel() * 4 >= self.prepared_mapping_bytes(), "prepared is a table from prepare_mapping")
            _check(self.lib.lplb_map_idx_prepared(mapping_idx.data_ptr(), o_weight.data_ptr(), by_sm.data_ptr(),
                                                  prepared.data_ptr(), mapping_idx.numel(), self.n_group,
                                                  self.group_size, self.dup_per_rank, self.n_combined_experts,
                                                  self.n_local_experts, n_sms, out.data_ptr(),
                                                  physical_counts.data_ptr() if physical_counts is not None else None,
                                                  _stream(mapping_idx)))
            return out
        _check(self.lib.lplb_map_idx(mapping_idx.data_ptr(), o_weight.data_ptr(), by_sm.data_ptr(), o2r.data_ptr(),
                                     phy2log.data_ptr(), mapping_idx.numel(), self.n_group, self.group_size,
                                     self.dup_per_rank, self.n_combined_experts, self.n_local_experts, n_sms,
                                     out.data_ptr(),
                                     physical_counts.data_ptr() if physical_counts is not None else None,
                                     _stream(mapping_idx)))
        return out

    def prepared_mapping_bytes(self) -> int:
        n = self.lib.lplb_prepared_mapping_bytes(self.n_group, self.group_size, self.dup_per_rank,
                                                 self.n_combined_experts, self.n_local_experts)
        _require(n > 0, "a shape the prepared table can describe")
        return n

    def prepare_mapping(self, o2r: torch.Tensor, phy2log: torch.Tensor) -> torch.Tensor:
        """The mapping-only part of the redirect's tables as an opaque int32 tensor for map_idx(prepared=...);
        valid until phy2log or o2r change."""
        _require(o2r.dtype == torch.int32 and o2r.is_cuda and o2r.is_contiguous()
                 and tuple(o2r.shape) == (self.group_size, self.dup_per_rank), "o2r is a contiguous int32 [G, D] GPU tensor")
        _require(phy2log.dtype == torch.int32 and phy2log.is_cuda and phy2log.is_contiguous() and phy2log.dim() == 1
                 and phy2log.size(0) == self.group_size * self.n_group * self.n_local_experts,
                 "phy2log is a contiguous int32 [n_group * group_size * n_local_experts] GPU tensor")
        n_bytes = self.prepared_mapping_bytes()
        table = torch.empty((n_bytes + 3) // 4, dtype=torch.int32, device=phy2log.device)
        _check(self.lib.lplb_prepare_mapping(o2r.data_ptr(), phy2log.data_ptr(), self.n_group, self.group_size,
                                             self.dup_per_rank, self.n_combined_experts, self.n_local_experts,
                                             table.data_ptr(), n_bytes, _stream(phy2log)))
        return table

    def _check_physical_counts(self, t: torch.Tensor | None) -> None:
        """Optional output of map_idx / plan: tokens per physical expert (the bincount of the result)."""
        if t is not None:
            _require(t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
                     and t.numel() == self.n_group * self.group_size * self.n_local_experts,
                     "physical_counts is a contiguous int32 [n_group * group_size * n_local_experts] GPU tensor")

    # -- lplb/planner.py:245-266 in one library call -----------------------------
    def plan(self, idx: torch.Tensor, r2o: torch.Tensor, o2r: torch.Tensor, phy2log: torch.Tensor,
             avail_num: torch.Tensor, n_sms: int, global_counts: torch.Tensor | None = None,
             workspace: dict | None = None,
             physical_counts: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Histogram, LP solve and redirect of one batch.  Returns (physical indices, o_weight,
        workspace table whose last row holds this GPU's tokens per logical expert).  ``global_counts`` (int32 [n_logical]) replaces this GPU's own histogram
        as the LP's workload.  ``workspace`` may carry preallocated ``out``, ``by_sm``, ``o_weight``
        and ``global_workload`` tensors to reuse; the last three are stored into it for the next call."""
        _require(idx.dtype == torch.int64 and idx.is_cuda and idx.is_contiguous(),
                 "idx is a contiguous int64 GPU tensor")
        for name, t in (("r2o", r2o), ("o2r", o2r)):
            _require(t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
                     and tuple(t.shape) == (self.group_size, self.dup_per_rank),
                     f"{name} is a contiguous int32 [group_size, dup_per_rank] GPU tensor")
        _require(phy2log.dtype == torch.int32 and phy2log.is_cuda and phy2log.is_contiguous()
                 and phy2log.dim() == 1 and phy2log.size(0) == self.group_size * self.n_group * self.n_local_experts,
                 "phy2log is a contiguous int32 [n_group * group_size * n_local_experts] GPU tensor")
        _require(avail_num.numel() == 1 and avail_num.dtype == torch.int32 and avail_num.is_cuda,
                 "avail_num is one int32 on the GPU")
        if global_counts is not None:
            _require(global_counts.dtype == torch.int32 and global_counts.is_cuda and global_counts.is_contiguous()
                     and global_counts.numel() == self.n_experts, "global_counts is a contiguous int32 [n_experts] GPU tensor")
        self._check_physical_counts(physical_counts)
        ws = workspace if workspace is not None else {}
        dev = idx.device
        out = ws.get("out")
        if out is None or out.shape != idx.shape:
            out = torch.empty_like(idx)
        by_sm = ws.get("by_sm")
        if by_sm is None or tuple(by_sm.shape) != (n_sms, self.n_experts):
            by_sm = torch.empty((n_sms, self.n_experts), dtype=torch.int32, device=dev)
        o_weight = ws.get("o_weight")
        if o_weight is None:
            o_weight = torch.empty((self.n_group, self.group_size, self.dup_per_rank), dtype=torch.float32, device=dev)
        gw = ws.get("global_workload")
        if gw is None:
            gw = torch.empty(self.n_experts, dtype=torch.float32, device=dev)
        if workspace is not None:   # kept for the caller's next batch (never `out`: that is the result)
            workspace.update(by_sm=by_sm, o_weight=o_weight, global_workload=gw)
        _check(self.lib.lplb_plan(idx.data_ptr(), idx.numel(),
                                  global_counts.data_ptr() if global_counts is not None else None,
                                  r2o.data_ptr(), o2r.data_ptr(), phy2log.data_ptr(), self.n_group,
                                  self.group_size, self.dup_per_rank, self.n_combined_experts,
                                  self.n_local_experts, n_sms, by_sm.data_ptr(), gw.data_ptr(),
                                  o_weight.data_ptr(), avail_num.data_ptr(), out.data_ptr(),
                                  physical_counts.data_ptr() if physical_counts is not None else None,
                                  self.step_rule, self.n_steps, _stream(idx)))
        return out, o_weight, by_sm
