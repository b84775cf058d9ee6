"""Per-batch token planner for expert-parallel MoE on MI355X.

``Planner`` is a drop-in for the reference's ``lplb.Planner`` (lplb/planner.py:38-266):
same constructor, attributes and methods, same tensors in and out.  ``run`` chains
three HIP launches on the current stream -- histogram, LP solve, redirect -- without
any host synchronisation.
"""
from __future__ import annotations

import functools
import warnings

import numpy as np
import torch

from . import _native
from ._native import CompiledSolver, UnsupportedShape, _stream
from .mapping import build_redundancy_mapping


@functools.lru_cache(maxsize=None)
def _get_solver(n_group: int, group_size: int, dup_per_rank: int, n_local_experts: int,
                n_combined_experts: int) -> CompiledSolver:
    return CompiledSolver(n_group, group_size, dup_per_rank, n_local_experts, n_combined_experts)


class Planner:
    def __init__(
        self,
        redundant_to_original: torch.Tensor,
        n_routed_experts: int,
        n_logical_routed_experts: int,
        ep_size: int | None = None,
        group: "torch.distributed.ProcessGroup | None" = None,
        *,
        device: str | torch.device = "cuda",
        gpus_per_node: int | None = None,
    ) -> None:
        """
        :param redundant_to_original: [group_size, num_redundants]; entry (i, d) is the group-rank
            whose d-th replicated expert set is copied into replica slot d of group-rank i.  Every
            column must be a permutation, so that each replica joins exactly two ranks.  A rank may
            hold a multiple of ``num_redundants`` replicas; they are pooled per slot for the LP.
        :param n_routed_experts: physical routed experts (originals + replicas) over all ranks.
        :param n_logical_routed_experts: logical routed experts.
        :param ep_size: number of EP ranks; defaults to ``group.size()``.
        :param group: EP process group; ``None`` means the workload handed to ``solve_probs`` is
            already global and no reduction is done.
        :param device: where the planner's tensors live.  Everything except the redundancy-mapping
            bookkeeping needs a GPU.
        :param gpus_per_node: GPUs per node for EPLB's node-aware packing; defaults to the number
            of visible GPUs (lplb/planner.py:132).
        """
        self.device = torch.device(device)
        r2o = torch.as_tensor(redundant_to_original)
        assert r2o.dim() == 2, "redundant_to_original must be [group_size, num_redundants]"
        self.r2o = r2o.to(dtype=torch.int32, device=self.device).contiguous()
        self.o2r = self.r2o.argsort(dim=0).to(torch.int32).contiguous()
        self.group_size, self.num_redundants = int(r2o.shape[0]), int(r2o.shape[1])
        self._r2o_host = self.r2o.cpu().numpy()

        self.n_routed_experts = n_routed_experts
        self.n_logical_routed_experts = n_logical_routed_experts
        if ep_size is not None:
            self.ep_size = ep_size
        else:
            assert group is not None, "ep_size must be provided when group is None"
            self.ep_size = group.size()
        self.n_group = self.ep_size // self.group_size

        self.n_local_routed_experts = self.n_routed_experts // self.ep_size
        self.n_local_logical_routed_experts = self.n_logical_routed_experts // self.ep_size
        self.combined_redundant_experts = (
            self.n_local_routed_experts - self.n_local_logical_routed_experts
        ) // self.num_redundants

        if gpus_per_node is None:
            gpus_per_node = torch.cuda.device_count() or 1
        self.gpus_per_node = gpus_per_node

        self.phy2log: torch.Tensor
        self.update_redundancy_mapping()

        self.ep_group = group
        self.deep_ep_initialized = False
        self._solver: CompiledSolver | None = None
        self._run_buffers: dict = {}
        self._prepared: tuple | None = None   # (key of the mapping it was built from, table or None)
        # health of the one-launch plan (see _look_at_plan_health)
        self.health_check_every = 64
        self.plan_timeouts = 0                # waits between workgroups that ran out on this device, as last seen
        self._health: torch.Tensor | None = None
        self._calls_since_health = 0

    @property
    def solver(self) -> CompiledSolver:
        if self._solver is None:
            if self.device.type != "cuda":
                raise RuntimeError("the planning kernels need a GPU: construct the Planner with device='cuda'")
            self._solver = _get_solver(self.n_group, self.group_size, self.num_redundants,
                                       self.n_local_routed_experts, self.combined_redundant_experts)
        return self._solver

    def init_from_deep_ep(self, buffer) -> None:
        """The reference can take its workload reduction from a DeepEP buffer's NVSHMEM team
        (lplb/planner.py:104-113).  There is no such transport here."""
        raise NotImplementedError(
            "in-kernel workload reduction through a DeepEP buffer is not available; "
            "pass `group` to reduce with torch.distributed, or hand solve_probs a global workload")

    def update_redundancy_mapping(
        self, workload: torch.Tensor | None = None
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Choose which experts get replicas (lplb/planner.py:115-182).

        :param workload: per-logical-expert history; ``None`` keeps experts in index order.
        :return: ``(phy2log [n_routed], log2phy [n_logical, 2], logcnt [n_logical])``, int32.
        """
        host = None if workload is None else workload.detach().cpu().numpy()
        phy2log, log2phy, logcnt = build_redundancy_mapping(
            self._r2o_host, self.ep_size, self.n_logical_routed_experts, self.n_routed_experts,
            host, n_nodes=max(1, self.ep_size // self.gpus_per_node))
        to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(self.device)  # noqa: E731
        self.phy2log = to_dev(phy2log)
        return self.phy2log, to_dev(log2phy), to_dev(logcnt)

    def count_workload(self, idx: torch.Tensor, n_sms: int) -> tuple[torch.Tensor, torch.Tensor]:
        """Histogram of ``idx`` (values in [-1, n_logical), -1 ignored) over ``n_sms`` slices.

        :return: (counts [n_logical], running counts per slice [n_sms, n_logical]), int32.
        """
        return self.solver.count_idx(idx, n_sms, 256)

    def solve_probs(self, workload: torch.Tensor, avail_counter: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """Solve the balancing LP of every EP group.

        :param workload: int32 per-logical-expert counts (numel = n_logical).
        :param avail_counter: int32, numel 1; incremented once per feasible group.
        :return: (share kept on the original rank, fp32 [n_group, group_size, num_redundants];
                  normalised global workload, fp32 [n_group, group_size, L]).
        """
        workload = workload.view(self.n_group, self.group_size, self.n_local_logical_routed_experts)
        if self.ep_group is not None and not self.deep_ep_initialized:
            workload = workload.clone()
            torch.distributed.all_reduce(workload, group=self.ep_group)
        return self.solver.solve(workload, self.r2o, self.phy2log, avail_counter)

    def _prepared_mapping(self) -> torch.Tensor | None:
        """The redirect's mapping-only tables (which the reference rebuilds in every block of every launch,
        minilp.cu:466-496), built once per phy2log; None for shapes the prepared form does not cover."""
        key = (self.phy2log.data_ptr(), self.phy2log._version, self.o2r.data_ptr(), self.o2r._version)
        if self._prepared is None or self._prepared[0] != key:
            try:
                table = self.solver.prepare_mapping(self.o2r, self.phy2log)
            except UnsupportedShape:
                table = None
            self._prepared = (key, table)
        return self._prepared[1]

    def weighted_select_target(self, idx: torch.Tensor, o_weight: torch.Tensor,
                               local_workload_by_sm: torch.Tensor, n_sms: int) -> torch.Tensor:
        """Map logical expert ids to physical ones according to ``o_weight``.

        :return: int64, same shape as ``idx``, values in [-1, n_routed_experts).
        """
        return self.solver.map_idx(idx, o_weight, local_workload_by_sm, self.o2r, self.phy2log, n_sms, 256,
                                   prepared=self._prepared_mapping())

    def _look_at_plan_health(self, idx: torch.Tensor) -> None:
        """Every ``health_check_every`` calls: read what the report enqueued that many calls ago wrote into pinned
        host memory (no synchronisation: it has long been written) and enqueue the next report."""
        self._calls_since_health += 1
        if self._calls_since_health < self.health_check_every:
            return
        self._calls_since_health = 0
        if self._health is None:
            self._health = torch.zeros(2, dtype=torch.int32).pin_memory()
        else:
            self._handle_plan_health(int(self._health[0]), int(self._health[1]))
        _native.plan_poll_timeouts(self._health, _stream(idx))

    def _handle_plan_health(self, timeouts: int, switched_off: int) -> None:
        """A wait between the workgroups of a one-launch plan ran out (a multi-second stall of the GPU, or kernels
        of the caller's that keep the plan's workgroups from being resident together): such plans leave their
        tokens on the original slots and do not raise ``avail_counter``; plans on that stream stay that way until
        the block of counters is switched on again, which is done here (it waits for the device once)."""
        if timeouts > self.plan_timeouts or switched_off:
            warnings.warn(f"lplb_amd: {timeouts - self.plan_timeouts} wait(s) between the workgroups of a one-launch plan ran "
                          f"out since the last look ({switched_off} block(s) of counters switched off); the batches "
                          "concerned were not balanced (avail_counter was not raised for them); switching the "
                          "one-launch form on again", RuntimeWarning, stacklevel=3)
            self.plan_timeouts = timeouts
            if switched_off:
                self.plan_timeouts = _native.plan_sync_timeouts()

    def run(self, idx: torch.Tensor, avail_counter: torch.Tensor, n_sms: int | None = None, *,
            physical_counts: torch.Tensor | None = None) -> torch.Tensor:
        """Assign a physical expert to every selected logical expert.

        :param idx: int64 logical expert ids, any shape, contiguous, values in [-1, n_logical).
        :param avail_counter: int32 tensor with one element, counts feasible LP solves.
        :param n_sms: number of slices / workgroups; defaults to the GPU's compute-unit count.
        :param physical_counts: optional int32 [n_routed_experts] output: tokens per physical expert
            (the bincount of the result, which the reference leaves to the caller).
        """
        if n_sms is None:
            n_sms = torch.cuda.get_device_properties(idx.device).multi_processor_count
        # run() hands out only the redirected indices, so the plan's other buffers (slice table,
        # shares, normalised counts) are kept per stream and slice count instead of being
        # allocated for every batch; work on one stream is ordered, so reuse is safe there
        capturing = torch.cuda.is_current_stream_capturing()
        key = (_stream(idx), n_sms)
        ws = self._run_buffers.get(key)
        if ws is None:
            if len(self._run_buffers) >= 16:
                # drop the oldest set of buffers that no captured graph can still be pointing at
                for old_key, old_ws in self._run_buffers.items():
                    if not old_ws.get("captured"):
                        del self._run_buffers[old_key]
                        break
            ws = self._run_buffers[key] = {}
        if capturing:
            ws["captured"] = True
        else:
            self._look_at_plan_health(idx)
        if self.ep_group is None:
            # count_workload -> solve_probs -> weighted_select_target in one library call
            out, _o_weight, _by_sm = self.solver.plan(idx, self.r2o, self.o2r, self.phy2log, avail_counter, n_sms,
                                                      workspace=ws, physical_counts=physical_counts)
            return out
        # With a process group the counts have to be summed over the ranks between histogram and
        # LP (lplb/planner.py:214-216); LP and redirect then run as one plan on the summed counts.
        # (the histogram's table is kept per stream like the plan's other buffers)
        # (The reference copies the counts before it reduces them, lplb/planner.py:215, because its redirect
        # reads the same table afterwards.  Here nothing reads them again -- the plan counts its slices
        # itself -- so the sum replaces them, and no table per slice is made at all.)
        n_experts = self.solver.n_experts
        short = idx.numel() <= _native.COUNT_TOTALS_MAX_INDICES
        if not capturing and short and n_experts * 4 <= 64 * 1024:
            # one launch adds the batch's counts to a zeroed vector and zeroes the vector of the call before
            pair = ws.get("group_totals_pair")
            if pair is None or pair[0].device != idx.device:
                pair = ws["group_totals_pair"] = [torch.zeros(n_experts, dtype=torch.int32, device=idx.device)
                                                  for _ in range(2)]
                ws["group_totals_turn"] = 0
            turn = ws["group_totals_turn"]
            workload = self.solver.count_totals_add(idx, pair[turn], clear=pair[1 - turn])
            ws["group_totals_turn"] = 1 - turn
        elif short and n_experts <= _native.COUNT_TOTALS_MAX_EXPERTS:
            # (a captured call replays with the vectors as the last replay left them: it takes the launch in
            # which every workgroup owns four experts and nothing has to be zero beforehand)
            totals = ws.get("group_totals")
            if totals is None or totals.device != idx.device:
                totals = ws["group_totals"] = torch.empty(n_experts, dtype=torch.int32, device=idx.device)
            workload = self.solver.count_totals(idx, out=totals)
        else:                                        # a long batch: histogram and scan
            table = ws.get("group_counts")
            if table is None or table.device != idx.device:
                table = ws["group_counts"] = torch.empty((n_sms, n_experts), dtype=torch.int32, device=idx.device)
            workload, _by_sm = self.solver.count_idx(idx, n_sms, 256, out=table)
        if not self.deep_ep_initialized:
            torch.distributed.all_reduce(workload, group=self.ep_group)
        out, _o_weight, _by_sm = self.solver.plan(idx, self.r2o, self.o2r, self.phy2log, avail_counter, n_sms,
                                                  global_counts=workload, workspace=ws,
                                                  physical_counts=physical_counts)
        return out
