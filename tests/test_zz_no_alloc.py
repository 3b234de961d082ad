"""The plan entry point that allocates nothing (``picomoe_permute_plan_static``) against ``picomoe_permute_plan``.

Called through the C ABI with caller-owned inputs and outputs only; its block histograms live in the library's fixed
1 MiB device array.  Two calls in a row, the second with a smaller input (the array then still holds the first call's
numbers past the part the second call uses), every output bit-identical to the workspace variant's and to the CPU
oracle's stable sort; with a capacity window and a later round; refused with its own error code beyond the fixed size;
captured into a HIP graph on a side stream after ``picomoe_permute_plan_static_init`` and replayed on changing inputs.
"""

import ctypes

import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _plan(lib, _lib, idx, E, capacity, round_index, static):
    R = idx.numel()
    dev = idx.device
    order = torch.full((R,), -7, dtype=torch.int32, device=dev)
    inv = torch.full((R,), -7, dtype=torch.int32, device=dev)
    counts = torch.full((E,), -7, dtype=torch.int64, device=dev)
    kept = torch.full((E,), -7, dtype=torch.int64, device=dev)
    within = torch.full((R,), -7, dtype=torch.int32, device=dev)
    P = _lib.ptr
    if static:
        rc = lib.picomoe_permute_plan_static(P(idx), R, E, capacity, round_index, P(order), P(inv), P(counts), P(kept), P(within),
                                             _lib.stream_ptr())
    else:
        ws = torch.empty(max(lib.picomoe_permute_workspace_bytes(R, E), 4), dtype=torch.uint8, device=dev)
        rc = lib.picomoe_permute_plan(P(idx), R, E, capacity, round_index, P(order), P(inv), P(counts), P(kept), P(within), P(ws),
                                      _lib.stream_ptr())
    torch.cuda.synchronize()
    return rc, (order, inv, counts, kept, within)


def test_static_plan_matches_workspace_plan_on_consecutive_calls(gpu):
    from picotron_amd import _lib

    lib = _lib.load()
    assert lib.picomoe_permute_plan_static_max_bytes() == 1 << 20
    g = torch.Generator().manual_seed(5)
    # (rows, experts, capacity, round): large first, then smaller ones that reuse the front of the same array
    cases = [(98304, 64, 0, 0), (5000, 64, 0, 0), (16384, 8, 0, 0), (3000, 8, 300, 1), (777, 1000, 0, 0), (1, 1, 0, 0), (0, 4, 0, 0)]
    for R, E, cap, rnd in cases:
        pr = 1.0 / torch.arange(1, E + 1, dtype=torch.float32) ** 1.1
        idx = torch.multinomial(pr, max(R, 1), replacement=True, generator=g)[:R].to(gpu)
        print(f"static plan: rows {R} experts {E} capacity {cap} round {rnd}", flush=True)
        rc_s, got = _plan(lib, _lib, idx, E, cap, rnd, static=True)
        rc_w, want = _plan(lib, _lib, idx, E, cap, rnd, static=False)
        assert rc_s == 0 and rc_w == 0, (rc_s, rc_w)
        for name, a, b in zip(("order", "inv_order", "counts", "kept_counts", "within"), got, want):
            assert torch.equal(a, b), (R, E, name)
        assert int(want[2].sum()) == R
        # and against the oracle's stable sort by expert (uncapped plans keep every row)
        o_order, o_inv, o_counts = O.permute_plan_fast(idx.cpu(), E)
        assert torch.equal(got[2].cpu(), o_counts), (R, E)
        if cap == 0:
            assert torch.equal(got[0].cpu().long(), o_order) and torch.equal(got[1].cpu().long(), o_inv), (R, E)
        else:  # round `rnd` of capacity `cap`: the rows whose rank inside their expert lies in [rnd * cap, (rnd + 1) * cap)
            o_within, _ = O.slot_assignment(idx.cpu(), E)
            keep = (o_within >= rnd * cap) & (o_within < (rnd + 1) * cap)
            assert torch.equal(got[4].cpu().long(), o_within)
            assert torch.equal(got[1].cpu() >= 0, keep)
            assert torch.equal(got[3].cpu(), torch.bincount(idx.cpu()[keep], minlength=E))
            kept_rows = got[0].cpu()[: int(keep.sum())].long()
            # kept rows lie expert after expert, ascending row order inside an expert: the stable sort of the kept rows
            assert torch.equal(kept_rows, torch.nonzero(keep).flatten()[torch.sort(idx.cpu()[keep], stable=True).indices])
    # and once more through the Python wrapper
    from picotron_amd import _ops

    idx = torch.randint(0, 8, (4096,), generator=g).to(gpu)
    a, b = _ops.permute_plan(idx, 8, static_scratch=True), _ops.permute_plan(idx, 8)
    assert torch.equal(a.order, b.order) and torch.equal(a.inv_order, b.inv_order) and torch.equal(a.counts, b.counts)


def test_static_plan_refuses_what_does_not_fit(gpu):
    from picotron_amd import _lib

    lib = _lib.load()
    R, E = 300000, 1024    # (293 + 1) x 1024 ints = 1.15 MiB
    assert lib.picomoe_permute_workspace_bytes(R, E) > lib.picomoe_permute_plan_static_max_bytes()
    idx = torch.zeros(R, dtype=torch.int64, device=gpu)
    rc, _ = _plan(lib, _lib, idx, E, 0, 0, static=True)
    assert rc == 2 and b"exceeds the fixed scratch" in lib.picomoe_error_string(rc)
    with pytest.raises(_lib.PicomoeError):
        _lib.check(rc, "picomoe_permute_plan_static")
    # the largest plan that fits: 255 blocks x 1024 experts
    R = 255 * 1024
    assert lib.picomoe_permute_workspace_bytes(R, E) == lib.picomoe_permute_plan_static_max_bytes()
    idx = (torch.arange(R, dtype=torch.int64) * 7919 % E).to(gpu)
    rc_s, got = _plan(lib, _lib, idx, E, 0, 0, static=True)
    rc_w, want = _plan(lib, _lib, idx, E, 0, 0, static=False)
    assert rc_s == 0 and rc_w == 0
    assert all(torch.equal(a, b) for a, b in zip(got, want))


def test_static_plan_captured_on_a_side_stream(gpu):
    """The caller the entry point is for: after one ``picomoe_permute_plan_static_init`` on the device, the plan is
    captured into a HIP graph on a side stream (no allocation, no symbol lookup inside the capture) and replayed three
    times on inputs that change between the replays, with eager work and synchronisations in between; every replay must
    equal the workspace variant run eagerly on the same input."""
    from picotron_amd import _lib

    lib = _lib.load()
    assert lib.picomoe_permute_plan_static_init() == 0
    assert lib.picomoe_permute_plan_static_init() == 0     # again: free
    R, E = 20000, 16
    g = torch.Generator().manual_seed(11)
    idx = torch.randint(0, E, (R,), generator=g).to(gpu)
    order = torch.empty(R, dtype=torch.int32, device=gpu)
    inv = torch.empty(R, dtype=torch.int32, device=gpu)
    counts = torch.empty(E, dtype=torch.int64, device=gpu)
    kept = torch.empty(E, dtype=torch.int64, device=gpu)
    within = torch.empty(R, dtype=torch.int32, device=gpu)
    P = _lib.ptr
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        rc = lib.picomoe_permute_plan_static(P(idx), R, E, 0, 0, P(order), P(inv), P(counts), P(kept), P(within), _lib.stream_ptr())
    assert rc == 0
    for replay in range(3):
        idx.copy_(torch.randint(0, E, (R,), generator=g))
        for t in (order, inv, within):
            t.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rc_w, want = _plan(lib, _lib, idx, E, 0, 0, static=False)
        assert rc_w == 0
        for name, a, b in zip(("order", "inv_order", "counts", "kept_counts", "within"), (order, inv, counts, kept, within), want):
            assert torch.equal(a, b), (replay, name)
