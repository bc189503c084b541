"""bp_sort_by_expert_static (the entry point that allocates nothing: its histograms live in a fixed device array
inside the library) against bp_sort_by_expert with a caller workspace, through the C ABI: order and offsets
bit-identical, on two calls in a row, the second with a smaller input (the array keeps the first call's contents)."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _sort_both(lib, ids, E):
    from deepseekternarized_amd.kernels import _lib

    n = ids.numel()
    stream = _lib.stream_ptr(ids.device)
    need = lib.bp_sort_workspace_ints(n, E)
    assert need > 0 and n > 128, "the case must be one that uses the histogram memory"
    ws = torch.empty(need, dtype=torch.int32, device="cuda")
    want_order = torch.full((n,), -1, dtype=torch.int64, device="cuda")
    want_offsets = torch.full((E + 1,), -1, dtype=torch.int64, device="cuda")
    _lib.check(lib.bp_sort_by_expert(want_order.data_ptr(), want_offsets.data_ptr(), ids.data_ptr(), n, E, ws.data_ptr(), None, stream))
    got_order = torch.full((n,), -2, dtype=torch.int64, device="cuda")
    got_offsets = torch.full((E + 1,), -2, dtype=torch.int64, device="cuda")
    bad = torch.zeros(1, dtype=torch.int32, device="cuda")
    _lib.check(lib.bp_sort_by_expert_static(got_order.data_ptr(), got_offsets.data_ptr(), ids.data_ptr(), n, E, bad.data_ptr(), stream))
    torch.cuda.synchronize()
    return want_order.cpu().numpy(), want_offsets.cpu().numpy(), got_order.cpu().numpy(), got_offsets.cpu().numpy(), int(bad.item())


def test_static_sort_matches_workspace_sort_on_two_calls_in_a_row():
    from deepseekternarized_amd.kernels import _lib

    lib = _lib.load()
    rng = np.random.default_rng(11)
    for n, E in ((70000, 5000), (3000, 4000)):  # the second call is smaller: stale counters of the first must not show
        ids_np = rng.integers(0, E, n).astype(np.int64)
        ids = torch.from_numpy(ids_np).cuda()
        want_order, want_offsets, got_order, got_offsets, bad = _sort_both(lib, ids, E)
        assert bad == 0
        assert np.array_equal(got_offsets, want_offsets)
        assert np.array_equal(got_order, want_order)
        # ... and both equal the definition: stable argsort, offsets = [0, cumsum(bincount)]
        assert np.array_equal(got_order, np.argsort(ids_np, kind="stable"))
        assert np.array_equal(got_offsets, np.concatenate([[0], np.cumsum(np.bincount(ids_np, minlength=E))]))


def test_static_sort_rejects_more_experts_than_its_array_holds():
    from deepseekternarized_amd.kernels import _lib

    lib = _lib.load()
    ids = torch.zeros(200, dtype=torch.int64, device="cuda")
    out = torch.zeros(200, dtype=torch.int64, device="cuda")
    offs = torch.zeros(65538, dtype=torch.int64, device="cuda")
    assert lib.bp_sort_by_expert_static(out.data_ptr(), offs.data_ptr(), ids.data_ptr(), 200, 65537, None, None) == 1
    assert b"at most 65536" in lib.bp_last_error()


def test_static_sort_captured_in_a_graph_after_a_first_eager_call():
    """The first call per device resolves the array's address outside any capture; a later call is plain launches and
    can be captured: replayed three times with eager work in between, each replay equal to bp_sort_by_expert."""
    from deepseekternarized_amd.kernels import _lib

    lib = _lib.load()
    n, E = 9000, 3000
    g = torch.Generator(device="cuda").manual_seed(3)
    ids = torch.randint(0, E, (n,), device="cuda", generator=g)
    order = torch.empty(n, dtype=torch.int64, device="cuda")
    offsets = torch.empty(E + 1, dtype=torch.int64, device="cuda")
    _lib.check(lib.bp_sort_by_expert_static(order.data_ptr(), offsets.data_ptr(), ids.data_ptr(), n, E, None, _lib.stream_ptr(ids.device)))
    torch.cuda.synchronize()
    assert lib.bp_last_error() == b""
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(lib.bp_sort_by_expert_static(order.data_ptr(), offsets.data_ptr(), ids.data_ptr(), n, E, None, _lib.stream_ptr(ids.device)))
    ws = torch.empty(lib.bp_sort_workspace_ints(n, E), dtype=torch.int32, device="cuda")
    want_order, want_offsets = torch.empty_like(order), torch.empty_like(offsets)
    for rep in range(3):
        ids.copy_(torch.randint(0, E, (n,), device="cuda", generator=g))
        order.fill_(-1)
        graph.replay()
        _lib.check(lib.bp_sort_by_expert(want_order.data_ptr(), want_offsets.data_ptr(), ids.data_ptr(), n, E, ws.data_ptr(), None,
                                         _lib.stream_ptr(ids.device)))
        torch.cuda.synchronize()
        assert torch.equal(order, want_order) and torch.equal(offsets, want_offsets), rep
