"""Host logic that needs no GPU: topologies, the redundancy mapping, the EPLB
reorder (against vectors written by the reference's own eplb.py), the Planner's
derived state, the synthetic workloads, and the C-ABI surface of the HIP library."""
import ctypes
import hashlib
import json
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from lplb_amd import Planner, _native, eplb, synth, topology
from lplb_amd.mapping import build_redundancy_mapping
from tests.helpers import REFERENCE_SOLVE_CASES

ROOT = Path(__file__).resolve().parent.parent
GOLDEN = ROOT / "tests" / "golden"


# --------------------------------------------------------------- topologies
def test_topologies_are_column_permutations():
    for r2o in (topology.CUBE_8P2E, topology.RING_8P, topology.HYPERCUBE_16P2E, topology.torus_2d(8, 4),
                topology.torus_2d(4, 4)):
        assert topology.is_valid_r2o(r2o)
        assert not np.any(r2o == np.arange(r2o.shape[0])[:, None])        # no replica on its own rank
    assert not topology.is_valid_r2o(np.array([[0, 1], [0, 0]]))
    t = topology.torus_2d(8, 4)
    assert t.shape == (32, 2) and t[0].tolist() == [4, 1] and t[31].tolist() == [3, 28]


# ------------------------------------------------------------- EPLB reorder
def test_eplb_matches_reference_vectors():
    """Vectors written by tests/golden/make_eplb_vectors.py from the reference's eplb.py
    (tie-free weights)."""
    for c in json.loads((GOLDEN / "eplb_vectors.json").read_text()):
        w = np.array(c["weight"])
        phy2log, log2phy, logcnt = eplb.rebalance_experts(w, c["num_replicas"], c["num_groups"], c["num_nodes"],
                                                          c["num_gpus"])
        np.testing.assert_array_equal(phy2log, c["phy2log"])
        np.testing.assert_array_equal(logcnt, c["logcnt"])
        want = np.array(c["log2phy"])
        if c["num_replicas"] == c["n_logical"]:
            np.testing.assert_array_equal(log2phy, want)
        else:
            # replicas of one expert carry equal loads, so which of them is "replica 0" is a tie
            np.testing.assert_array_equal(np.sort(log2phy, axis=-1), np.sort(want, axis=-1))


def test_balanced_packing_properties():
    rng = np.random.default_rng(0)
    w = rng.random((3, 24)).astype(np.float32)
    pack, rank = eplb.balanced_packing(w, 6)
    for layer in range(3):
        assert sorted(np.bincount(pack[layer], minlength=6)) == [4] * 6
        for p in range(6):
            assert sorted(rank[layer][pack[layer] == p]) == [0, 1, 2, 3]
    # heaviest-first greedy never does worse than putting the 4 heaviest together
    loads = np.array([[w[l][pack[l] == p].sum() for p in range(6)] for l in range(3)])
    assert np.all(loads.max(1) <= np.sort(w, axis=1)[:, -4:].sum(1))
    pack1, rank1 = eplb.balanced_packing(w[:, :6], 6)
    assert np.array_equal(pack1, np.broadcast_to(np.arange(6), (3, 6))) and not rank1.any()


# ------------------------------------------------------ redundancy mapping
@pytest.mark.parametrize("case", REFERENCE_SOLVE_CASES, ids=[c[0] for c in REFERENCE_SOLVE_CASES])
@pytest.mark.parametrize("with_history", [False, True])
def test_redundancy_mapping_layout(case, with_history):
    _, r2o, nl, ep, red, _, _ = case
    r2o = np.asarray(r2o)
    G, D = r2o.shape
    n_phys = nl + red * ep
    L, P = nl // ep, n_phys // ep
    C = (P - L) // D
    rng = np.random.default_rng(1)
    hist = rng.integers(1, 1 << 20, size=nl) if with_history else None
    phy2log, log2phy, logcnt = build_redundancy_mapping(r2o, ep, nl, n_phys, hist, n_nodes=max(1, ep // 8))
    assert phy2log.shape == (n_phys,) and phy2log.dtype == np.int32
    per_rank = phy2log.reshape(ep // G, G, P)
    # the first L slots of all ranks are a permutation of the logical experts
    assert sorted(per_rank[:, :, :L].reshape(-1)) == list(range(nl))
    # replica (c, d) of group-rank i copies slot (c, d) of group-rank r2o[i, d]
    for g in range(ep // G):
        for i in range(G):
            for c in range(C):
                for d in range(D):
                    assert per_rank[g, i, L + c * D + d] == per_rank[g, r2o[i, d], c * D + d]
    if with_history:
        # every rank keeps its experts heaviest first, so its replicated ones are its heaviest
        h = hist[per_rank[:, :, :L]]
        assert np.all(np.diff(h, axis=-1) <= 0)
    else:
        assert np.array_equal(per_rank[:, :, :L].reshape(-1), np.arange(nl))
    # log2phy: original first, then the replica; at most one replica each (lplb/planner.py:165-178)
    assert logcnt.max() == 2 and logcnt.sum() == n_phys
    for e in range(nl):
        slots = [s for s in log2phy[e] if s >= 0]
        assert len(slots) == logcnt[e] and all(phy2log[s] == e for s in slots)
        assert slots[0] % P < L and all(s % P >= L for s in slots[1:])


def test_redundancy_mapping_rejects_doubly_replicated_experts():
    bad = np.array([[1, 1], [0, 0]]).T            # both ranks copy rank 1's slot-0 expert
    with pytest.raises(AssertionError):
        build_redundancy_mapping(np.array([[1], [1]]), 2, 4, 6)
    del bad


# ------------------------------------------------------------------ Planner
def test_planner_derived_state_on_cpu():
    p = Planner(torch.from_numpy(topology.CUBE_8P2E), 256 + 2 * 32, 256, 32, device="cpu")
    assert (p.group_size, p.num_redundants, p.n_group, p.ep_size) == (8, 2, 4, 32)
    assert (p.n_local_routed_experts, p.n_local_logical_routed_experts, p.combined_redundant_experts) == (10, 8, 1)
    assert p.r2o.dtype == torch.int32 and p.o2r.dtype == torch.int32 and p.o2r.is_contiguous()
    r2o, o2r = p.r2o.numpy(), p.o2r.numpy()
    for d in range(2):
        assert np.array_equal(r2o[o2r[:, d], d], np.arange(8))             # o2r inverts r2o column-wise
    assert p.phy2log.shape == (320,) and p.phy2log.dtype == torch.int32
    phy2log, log2phy, logcnt = p.update_redundancy_mapping(torch.arange(256, 0, -1) * 1000)
    assert phy2log is p.phy2log and log2phy.shape == (256, 2) and int(logcnt.max()) == 2
    assert all(t.dtype == torch.int32 for t in (phy2log, log2phy, logcnt))
    # ep_size defaults to the group size (needs a group), combined replicas
    with pytest.raises(AssertionError):
        Planner(torch.from_numpy(topology.CUBE_8P2E), 320, 256, device="cpu")
    p4 = Planner(torch.from_numpy(topology.CUBE_8P2E), 256 + 4 * 32, 256, 32, device="cpu")
    assert p4.combined_redundant_experts == 2 and p4.phy2log.numel() == 384


def test_planner_needs_a_gpu_for_the_kernels():
    p = Planner(torch.from_numpy(topology.RING_8P), 64 + 8, 64, 8, device="cpu")
    idx = torch.zeros(16, dtype=torch.int64)
    with pytest.raises(RuntimeError):
        p.run(idx, torch.zeros(1, dtype=torch.int32), 4)
    with pytest.raises(NotImplementedError):
        p.init_from_deep_ep(None)


def test_planner_surfaces_waits_that_ran_out(monkeypatch):
    """Planner.run looks at the one-launch plan's health report every few calls; a non-zero count must reach the
    user (a warning, the attribute) and switch the one-launch form on again.  The report itself needs a GPU;
    what is done with it does not."""
    from lplb_amd import _native as native
    p = Planner(torch.from_numpy(topology.RING_8P), 64 + 8, 64, 8, device="cpu")
    rearmed = []
    monkeypatch.setattr(native, "plan_sync_timeouts", lambda: rearmed.append(1) or 5)
    import warnings as w
    with w.catch_warnings():
        w.simplefilter("error")
        p._handle_plan_health(0, 0)                    # healthy: silent
    assert p.plan_timeouts == 0 and not rearmed
    with pytest.warns(RuntimeWarning, match="not balanced"):
        p._handle_plan_health(3, 1)
    assert rearmed == [1] and p.plan_timeouts == 5     # the synchronous call's own count after re-arming
    with pytest.warns(RuntimeWarning):
        p._handle_plan_health(7, 0)                    # counted since, but no block is off: nothing to re-arm
    assert rearmed == [1] and p.plan_timeouts == 7
    with w.catch_warnings():
        w.simplefilter("error")
        p._handle_plan_health(7, 0)                    # nothing new
    # the look itself is spaced out and never happens on a CPU planner before the kernels are needed
    calls = []
    monkeypatch.setattr(native, "plan_poll_timeouts", lambda dst, stream=None: calls.append(dst))
    monkeypatch.setattr(torch.Tensor, "pin_memory", lambda self: self)
    monkeypatch.setattr("lplb_amd.planner._stream", lambda t: 0)
    p.health_check_every = 4
    for _ in range(9):
        p._look_at_plan_health(torch.zeros(1))
    assert len(calls) == 2 and calls[0] is calls[1] and calls[0].dtype == torch.int32


def test_compiled_solver_argument_checks():
    """Same refusals as the reference's extension (csrc/plugin.cpp:494-530, 582-584, 605-628)."""
    s = _native.CompiledSolver(1, 8, 2, 34, 1)
    assert s.n_experts == 256
    idx = torch.zeros(16, dtype=torch.int64)
    with pytest.raises(RuntimeError):
        s.count_idx(idx, 4)                       # not on a GPU
    with pytest.raises(RuntimeError):
        s.count_idx(idx.int(), 4)                 # wrong dtype
    with pytest.raises(RuntimeError):
        s.solve(torch.zeros(1, 8, 32, dtype=torch.int32), torch.zeros(8, 2, dtype=torch.int32),
                torch.zeros(272, dtype=torch.int32), torch.zeros(1, dtype=torch.int32))
    with pytest.raises(RuntimeError):
        s.map_idx(idx, torch.zeros(1, 8, 2), torch.zeros(4, 256, dtype=torch.int32), torch.zeros(8, 2, dtype=torch.int32),
                  torch.zeros(272, dtype=torch.int32), 4)


# ---------------------------------------------------------------- workloads
def test_synthetic_inputs_are_deterministic_and_well_formed():
    digests = {}
    for name in ("cpu_ref_ep8", "v3_ep8_cube", "ep16_hypercube", "ep32_torus"):
        a, b = synth.make_inputs(name, tokens=512), synth.make_inputs(name, tokens=512)
        for x, y in ((a.indices, b.indices), (a.global_counts, b.global_counts), (a.phy2log, b.phy2log)):
            assert np.array_equal(x, y)
        c = a.cfg
        assert a.indices.shape == (512, c.topk) and a.indices.dtype == np.int64
        assert a.indices.min() >= 0 and a.indices.max() < c.n_logical
        assert all(len(set(row)) == c.topk for row in a.indices[:64])      # distinct experts per token
        assert a.global_counts.dtype == np.int32 and a.global_counts.sum() == c.ep_size * c.tokens * c.topk
        assert abs(a.popularity.sum() - 1) < 1e-12
        digests[name] = hashlib.sha256(a.indices.tobytes() + a.global_counts.tobytes()).hexdigest()
    assert len(set(digests.values())) == 4
    m = synth.make_inputs("cpu_ref_ep8", mask_fraction=0.25)
    assert 0.15 < (m.indices == -1).mean() < 0.35
    sc = synth.sweep_counts(4)
    assert sc.shape == (4, 256) and not np.array_equal(sc[0], sc[1])
    hot = synth.make_inputs("ep32_torus", tokens=8).popularity
    assert (hot > 5.0 / 256).sum() >= 3


# ------------------------------------------------------------------- C ABI
def _declared_symbols():
    text = (ROOT / "include" / "lplb_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lplb_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _native.load()
    declared = _declared_symbols()
    assert "lplb_count_idx" in declared and "lplb_solve" in declared and "lplb_map_idx" in declared
    for name in declared:
        assert getattr(lib, name) is not None
    assert sorted(_native.exported_symbols()) == declared
    assert lib.lplb_abi_version() == _native.ABI_VERSION == 7
    header = (ROOT / "include" / "lplb_hip.h").read_text()
    assert f"#define LPLB_ABI_VERSION {_native.ABI_VERSION}" in header
    assert f"#define LPLB_COUNT_TOTALS_MAX_INDICES {_native.COUNT_TOTALS_MAX_INDICES}\n" in header
    assert f"#define LPLB_COUNT_TOTALS_MAX_EXPERTS {_native.COUNT_TOTALS_MAX_EXPERTS}\n" in header


def test_entry_points_reject_bad_arguments_before_touching_the_gpu():
    lib = _native.load()
    buf = (ctypes.c_int64 * 4)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.lplb_count_idx(p, 4, 0, 4, p, None) == 1
    assert b"n_experts" in lib.lplb_last_error()
    assert lib.lplb_count_idx(p, -1, 8, 4, p, None) == 1
    assert lib.lplb_count_idx(p, 4, 8, 4, None, None) == 1
    assert lib.lplb_count_idx(p, 4, 1 << 20, 4, p, None) == 2           # histogram does not fit LDS
    assert lib.lplb_count_totals(p, 4, 0, p, None) == 1
    assert lib.lplb_count_totals(p, 4, 8, None, None) == 1
    assert lib.lplb_count_totals(p, 1 << 20, 8, p, None) == 2          # a long batch: histogram and scan serve it
    assert lib.lplb_count_totals_add(p, 4, 0, p, None, None) == 1
    assert lib.lplb_count_totals_add(p, 4, 8, None, None, None) == 1
    assert lib.lplb_count_totals_add(p, 4, 8, p, p, None) == 1            # totals and clear are one vector
    assert b"same vector" in lib.lplb_last_error()
    assert lib.lplb_count_totals_add(p, 4, 1 << 20, p, None, None) == 2   # histogram does not fit LDS
    assert lib.lplb_count_totals_add(p, 1 << 20, 8, p, None, None) == 2   # a long batch
    assert lib.lplb_solve(p, p, p, p, 1, 16, 9, 1, 2, p, p, 0, 5, None) == 2   # 144 edges > two per lane of a wave
    assert b"128 replica edges" in lib.lplb_last_error()
    assert lib.lplb_solve(p, p, p, p, 1, 4, 17, 1, 2, p, p, 0, 5, None) == 2   # more than 16 slots per rank
    assert lib.lplb_solve(p, p, p, p, 1, 65, 1, 1, 2, p, p, 0, 5, None) == 2   # more ranks than lanes
    assert lib.lplb_solve(p, p, p, p, 1, 8, 2, 1, 2, p, p, 7, 5, None) == 1    # unknown step rule
    assert lib.lplb_solve(p, None, p, p, 1, 8, 2, 1, 2, p, p, 0, 5, None) == 1
    assert lib.lplb_solve_batched(p, None, p, p, 0, 1, 8, 2, 1, 2, p, p, 0, 5, None) == 1
    assert lib.lplb_map_idx(p, p, p, p, p, 4, 1, 8, 2, 1, 2, 4, p, None, None) == 1  # 2 slots per rank cannot hold 2 replicas
    assert lib.lplb_map_idx(p, p, p, p, None, 4, 1, 8, 2, 1, 34, 4, p, None, None) == 1
    assert lib.lplb_plan(p, 4, None, p, p, p, 1, 8, 2, 1, 34, 0, p, p, p, p, p, None, 0, 5, None) == 1
    assert lib.lplb_copy_calibration(p, p, 3, None) == 1
    # an index array needs its natural alignment only; 4 bytes off is refused
    odd = ctypes.c_void_p(p.value + 4)
    assert lib.lplb_count_idx(odd, 4, 8, 4, p, None) == 1 and b"8-byte" in lib.lplb_last_error()
    assert lib.lplb_plan(odd, 4, None, p, p, p, 1, 8, 2, 1, 34, 4, p, p, p, p, p, None, 0, 5, None) == 1
    # tokens per physical expert come from a closed form that assumes 499 k + 41 does not wrap
    assert lib.lplb_plan(p, 5_000_000, None, p, p, p, 1, 8, 2, 1, 34, 256, p, p, p, p, p, p, 0, 5, None) == 2
    assert b"physical_counts" in lib.lplb_last_error()
    assert lib.lplb_map_idx(p, p, p, p, p, 5_000_000, 1, 8, 2, 1, 34, 256, p, p, None) == 2


def test_cross_workgroup_helpers_compile_to_the_forms_the_plan_relies_on(tmp_path):
    """The workgroups of the one-launch plan exchange data through agent-scope atomics
    (lplb_amd/csrc/plan_sync.h).  That works across the GPU's eight L2 caches because those
    atomics bypass the L2 (sc1 bit) and s_waitcnt vmcnt(0) waits for the stores' acknowledgement; nothing
    invalidates a cache (the L2 holds the batch's indices while the workgroups talk).  Compile the helpers on their own
    and look at what the compiler makes of them, so that a toolchain that lowers them
    differently fails here and not silently on the GPU."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(hipcc).exists():
        pytest.skip("no hipcc")
    probe = tmp_path / "probe.hip"
    probe.write_text('''
#include "plan_sync.h"
using namespace lplb;
extern "C" __global__ void publish(int *row, unsigned long long *word, int *counter) {
  agent_store(row + threadIdx.x, 7);
  agent_add(word, (5ull << 32) | 1ull);
  stores_have_landed();
  __syncthreads();
  if (threadIdx.x < 64)
    announce_arrival(counter, 4, blockIdx.x);
}
extern "C" __global__ void consume(int *counter, const int *row, const unsigned long long *word, int *out) {
  if (threadIdx.x < 64)
    out[64] = wait_for_arrivals(counter, 3, 1000);
  __syncthreads();
  out[threadIdx.x] = agent_load(row + threadIdx.x) + (int)(agent_load(word) >> 32);
}
''')
    asm = tmp_path / "probe.s"
    subprocess.run([hipcc, "-O3", "-std=c++17", "--offload-arch=gfx950", "--cuda-device-only", "-S",
                    f"-I{ROOT / 'lplb_amd' / 'csrc'}", str(probe), "-o", str(asm)], check=True, capture_output=True)
    text = asm.read_text()
    publish, consume = text.split("consume:")[0], text.split("consume:")[1]
    assert re.search(r"global_store_dword .* sc1", publish), "agent-scope store does not write through"
    # read-modify-writes are carried out by the atomic unit behind the caches (no cached copy to go stale)
    assert "global_atomic_add_x2" in publish and re.search(r"global_atomic_add v", publish)
    # the row's stores are acknowledged before the barrier that precedes the counter update
    body = publish[publish.index("global_store_dword"):]
    assert body.index("s_waitcnt vmcnt(0)") < body.index("s_barrier") < body.rindex("global_atomic_add v")
    assert "buffer_inv" not in text and "buffer_wbl2" not in text, "a cache is invalidated or written back"
    polls, after_wait = consume.split("s_barrier")[0], consume.split("s_barrier")[1]
    assert "s_sleep" in polls and re.search(r"global_load_dword .* sc1", polls), "a poll may hit a stale L2 line"
    assert re.search(r"global_load_dword v\d+, v\d+, s\[\d+:\d+\] sc1", after_wait), "the row is not read past the L2"
    assert re.search(r"global_load_dwordx2 .* sc1", after_wait), "the tagged word is read past the L2"


def test_no_kernel_spills_vector_registers():
    """The build leaves the compiler's per-kernel resource report next to each object
    (lplb_amd/csrc/*.resources.txt).  No kernel may spill vector registers: besides being slow,
    a spill placed where only part of a wave is active (seen with this compiler in a variant of the
    one-launch plan, between a divergent loop and the instruction that restores the execution mask) loses
    the value in the inactive lanes.  The variants are sized so that none spills; this keeps it so."""
    reports = sorted((Path(__file__).parent.parent / "lplb_amd" / "csrc").glob("*.resources.txt"))
    if not reports:
        pytest.skip("no resource reports: the library was not built here")
    n_kernels, spilling = 0, []
    for report in reports:
        name = None
        for line in report.read_text().splitlines():
            m = re.search(r"Function Name: (\S+)", line)
            if m:
                name, n_kernels = m.group(1), n_kernels + 1
            m = re.search(r"VGPRs Spill: (\d+)", line)
            if m and int(m.group(1)) > 0:
                spilling.append((report.name, name, int(m.group(1))))
    assert n_kernels > 100, n_kernels
    assert not spilling, spilling


def test_compiled_solver_takes_the_reference_argument_list():
    """csrc/plugin.cpp:665-667 / lplb/planner.py:26-35: (resource_path, n_group, group_size, dup_per_rank,
    block_dim, n_local_experts, n_combined_experts, pg)."""
    from lplb_amd import _native
    short = _native.CompiledSolver(2, 8, 2, 34, 1)
    ref = _native.CompiledSolver("/somewhere/resources", 2, 8, 2, 256, 34, 1, None)
    kw = _native.CompiledSolver(resource_path="x", n_group=2, group_size=8, dup_per_rank=2, block_dim=256,
                                n_local_experts=34, n_combined_experts=1, pg="a group")
    for s_ in (ref, kw):
        assert (s_.n_group, s_.group_size, s_.dup_per_rank, s_.n_local_experts, s_.n_combined_experts, s_.n_experts) == \
               (short.n_group, short.group_size, short.dup_per_rank, short.n_local_experts, short.n_combined_experts,
                short.n_experts)
    assert kw.pg == "a group" and ref.pg is None
    with pytest.raises(TypeError):
        _native.CompiledSolver("/somewhere/resources", 2, 8, 2, 256, 34)
    with pytest.raises(TypeError):
        _native.CompiledSolver(2, 8, 2, 34, 1, None)
