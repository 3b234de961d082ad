"""The plan entry point that allocates nothing (``picomoe_permute_plan_static``) against ``picomoe_permute_plan``.

Called through the C ABI with caller-owned inputs and outputs only; its block histograms live in the library's fixed
1 MiB device array.  Two calls in a row, the second with a smaller input (the array then still holds the first call's
numbers past the part the second call uses), every output bit-identical to the workspace variant's; with a capacity
window and a later round; refused with its own error code beyond the fixed size.
"""

import ctypes

import pytest
import torch

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
    assert rc == 2 and b"larger than the fixed scratch" in lib.picomoe_error_string(rc)
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
