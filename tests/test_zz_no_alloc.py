"""lplb_plan_noalloc (the plan for callers that cannot allocate device memory) against
lplb_plan, through the raw C ABI: same inputs, every output compared bit for bit, on two
calls in a row that share the library's built-in slice table, the second on a smaller
batch.  Needs an MI355X.
"""
import ctypes

import numpy as np
import pytest
import torch

from lplb_amd import _native, synth
from oracle import oracle
from tests.helpers import Shape

pytestmark = pytest.mark.gpu

VP = ctypes.c_void_p


def _dev(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def _ptr(t):
    return VP(t.data_ptr()) if t is not None else None


class _Outputs:
    """Caller-owned outputs of one plan, allocated before the calls under test."""

    def __init__(self, n, shape, cuda):
        self.out = torch.full((n,), -7, dtype=torch.int64, device=cuda)
        self.o_weight = torch.full((shape.n_group, shape.G, shape.D), -7.0, dtype=torch.float32, device=cuda)
        self.gw = torch.full((shape.n_logical,), -7.0, dtype=torch.float32, device=cuda)
        self.avail = torch.zeros(1, dtype=torch.int32, device=cuda)
        self.physical = torch.full((shape.n_physical,), -7, dtype=torch.int32, device=cuda)
        self.local = torch.full((shape.n_logical,), -7, dtype=torch.int32, device=cuda)


def _both_plans(lib, cuda, inp, n_tokens, n_blocks, use_global):
    """Runs lplb_plan and lplb_plan_noalloc on the first n_tokens rows; returns their outputs."""
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    idx_host = np.ascontiguousarray(inp.indices[:n_tokens].reshape(-1))
    idx = _dev(idx_host, cuda)
    r2o, o2r, p2l = _dev(shape.r2o, cuda), _dev(shape.o2r, cuda), _dev(inp.phy2log, cuda)
    counts = _dev(inp.global_counts, cuda) if use_global else None
    n = idx.numel()
    ref, got = _Outputs(n, shape, cuda), _Outputs(n, shape, cuda)
    table = torch.empty((n_blocks, shape.n_logical), dtype=torch.int32, device=cuda)
    shape_args = (shape.n_group, shape.G, shape.D, shape.C, shape.P, n_blocks)
    stream = VP(torch.cuda.current_stream().cuda_stream)
    print(f"plan vs plan_noalloc: cfg={c.name} n={n} n_blocks={n_blocks} global={use_global}", flush=True)
    rc = lib.lplb_plan(_ptr(idx), n, _ptr(counts), _ptr(r2o), _ptr(o2r), _ptr(p2l), *shape_args, _ptr(table),
                       _ptr(ref.gw), _ptr(ref.o_weight), _ptr(ref.avail), _ptr(ref.out), _ptr(ref.physical), 0, 5, stream)
    assert rc == 0, lib.lplb_last_error()
    rc = lib.lplb_plan_noalloc(_ptr(idx), n, _ptr(counts), _ptr(r2o), _ptr(o2r), _ptr(p2l), *shape_args,
                               _ptr(got.local), _ptr(got.gw), _ptr(got.o_weight), _ptr(got.avail), _ptr(got.out),
                               _ptr(got.physical), 0, 5, stream)
    assert rc == 0, lib.lplb_last_error()
    torch.cuda.synchronize()
    ref.local = table[-1].clone()
    return shape, idx_host, ref, got


def _assert_same(shape, idx_host, ref, got):
    assert torch.equal(got.out, ref.out)
    assert torch.equal(got.o_weight, ref.o_weight)          # same kernels, same bits
    assert torch.equal(got.gw, ref.gw)
    assert torch.equal(got.physical, ref.physical)
    assert torch.equal(got.local, ref.local)
    assert int(got.avail[0]) == int(ref.avail[0]) == shape.n_group
    # and both are right: totals and bincount against the CPU checker
    want_local = oracle.count_idx(idx_host, shape.n_logical, 1)[-1]
    np.testing.assert_array_equal(got.local.cpu().numpy(), want_local)
    out = got.out.cpu().numpy()
    np.testing.assert_array_equal(got.physical.cpu().numpy(),
                                  np.bincount(out[out >= 0], minlength=shape.n_physical))


@pytest.mark.parametrize("use_global", [True, False])
def test_plan_noalloc_matches_plan_on_two_calls_in_a_row(cuda, use_global):
    lib = _native.load()
    inp = synth.make_inputs("v3_ep8_cube", mask_fraction=0.05)
    # first call: the whole [8192 x 8] batch (one kernel launch); second: a smaller batch that
    # reuses the table the first one left behind
    for n_tokens, n_blocks in ((8192, 256), (1000, 40)):
        _assert_same(*_both_plans(lib, cuda, inp, n_tokens, n_blocks, use_global))


def test_plan_noalloc_long_batch_then_short_batch(cuda):
    """A batch long enough for the chain of kernels (the full prefix table is then used), then a
    short one with fewer slices on the same table; a second topology for the LP shape."""
    lib = _native.load()
    inp = synth.make_inputs("sweep_redirect", tokens=100000, mask_fraction=0.02)
    _assert_same(*_both_plans(lib, cuda, inp, 100000, 256, False))
    _assert_same(*_both_plans(lib, cuda, inp, 300, 256, False))
    torus = synth.make_inputs("ep32_torus", mask_fraction=0.05)
    _assert_same(*_both_plans(lib, cuda, torus, 16384, 200, True))
    _assert_same(*_both_plans(lib, cuda, torus, 77, 3, True))


def test_plan_noalloc_refuses_what_its_table_cannot_hold(cuda):
    lib = _native.load()
    inp = synth.make_inputs("v3_ep8_cube")
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    idx = _dev(inp.indices.reshape(-1), cuda)
    r2o, o2r, p2l = _dev(shape.r2o, cuda), _dev(shape.o2r, cuda), _dev(inp.phy2log, cuda)
    o = _Outputs(idx.numel(), shape, cuda)
    args = lambda n_blocks: (_ptr(idx), idx.numel(), None, _ptr(r2o), _ptr(o2r), _ptr(p2l), shape.n_group, shape.G,  # noqa: E731
                             shape.D, shape.C, shape.P, n_blocks, _ptr(o.local), _ptr(o.gw), _ptr(o.o_weight),
                             _ptr(o.avail), _ptr(o.out), None, 0, 5, None)
    assert lib.lplb_plan_noalloc(*args(1025)) == 2            # 1025 x 256 counters > 262144
    assert b"slice table" in lib.lplb_last_error()
    torch.cuda.synchronize()
    assert int(o.avail[0]) == 0 and int(o.out[0]) == -7       # nothing was enqueued
    assert lib.lplb_plan_noalloc(*args(1024)) == 0            # exactly the limit
    torch.cuda.synchronize()
    want = oracle.count_idx(inp.indices.reshape(-1), shape.n_logical, 1)[-1]
    np.testing.assert_array_equal(o.local.cpu().numpy(), want)


def test_plan_noalloc_allocates_nothing_and_replays_from_a_graph(cuda):
    """What the entry point is for: after a first call (which looks up addresses and attributes), a call
    leaves torch's allocator as it found it, and a call captured into a HIP graph replays with the same
    result as the eager call, several times, with other work in between."""
    lib = _native.load()
    inp = synth.make_inputs("v3_ep8_cube", mask_fraction=0.05)
    c = inp.cfg
    shape = Shape(c.r2o, c.ep_size, c.n_logical, c.n_physical)
    idx = _dev(inp.indices.reshape(-1), cuda)
    r2o, o2r, p2l = _dev(shape.r2o, cuda), _dev(shape.o2r, cuda), _dev(inp.phy2log, cuda)
    counts = _dev(inp.global_counts, cuda)
    eager, replayed = _Outputs(idx.numel(), shape, cuda), _Outputs(idx.numel(), shape, cuda)

    def call(o, stream):
        rc = lib.lplb_plan_noalloc(_ptr(idx), idx.numel(), _ptr(counts), _ptr(r2o), _ptr(o2r), _ptr(p2l), shape.n_group,
                                   shape.G, shape.D, shape.C, shape.P, 256, _ptr(o.local), _ptr(o.gw), _ptr(o.o_weight),
                                   _ptr(o.avail), _ptr(o.out), _ptr(o.physical), 0, 5, VP(stream))
        assert rc == 0, lib.lplb_last_error()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(eager, side.cuda_stream)                       # warm-up on the stream that will be captured
        torch.cuda.synchronize()
        allocated, reserved = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        free_before = torch.cuda.mem_get_info()[0]
        eager.avail.zero_()
        call(eager, side.cuda_stream)
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (allocated, reserved)
        assert torch.cuda.mem_get_info()[0] == free_before  # nothing taken from the device behind torch's back either
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):              # (the stream that used the table last: see the header)
        call(replayed, side.cuda_stream)
    for replay in range(3):
        replayed.out.fill_(-7)
        replayed.physical.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(replayed.out, eager.out) and torch.equal(replayed.physical, eager.physical)
        assert torch.equal(replayed.o_weight, eager.o_weight) and torch.equal(replayed.local, eager.local)
        _ = (idx + replay).sum().item()                      # eager work and a synchronisation between replays
    assert int(replayed.avail[0]) == 3
    # the captured call keeps the table: another stream is told so instead of racing on it
    other = torch.cuda.Stream()
    rc = lib.lplb_plan_noalloc(_ptr(idx), idx.numel(), _ptr(counts), _ptr(r2o), _ptr(o2r), _ptr(p2l), shape.n_group,
                               shape.G, shape.D, shape.C, shape.P, 256, None, _ptr(eager.gw), _ptr(eager.o_weight),
                               _ptr(eager.avail), _ptr(eager.out), None, 0, 5, VP(other.cuda_stream))
    assert rc == 4 and b"another stream" in lib.lplb_last_error()
