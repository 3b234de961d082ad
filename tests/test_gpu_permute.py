"""GPU parity of the permutation plan (stable counting sort, capacity slots), the gather and the
combine kernels against the CPU oracle: permutation, drop set and counts bit-exact."""

import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _zipf_idx(T, k, E, skew, seed):
    g = torch.Generator().manual_seed(seed)
    rank_w = 1.0 / torch.arange(1, E + 1, dtype=torch.float32) ** skew
    probs = (rank_w / rank_w.sum()).expand(T, E)
    return torch.multinomial(probs, k, replacement=False, generator=g)


@pytest.mark.parametrize("R,E", [(0, 4), (1, 1), (17, 4), (1000, 8), (1024, 8), (1025, 3), (16384, 8), (98304, 64), (5000, 1000), (70000, 1024)])
def test_plan_is_the_stable_sort(gpu, R, E):
    from picotron_amd import _ops

    g = torch.Generator().manual_seed(R + E)
    e = torch.randint(0, E, (R,), generator=g)
    if R > 10 and E > 2:
        e[e == 1] = 0                               # an empty expert
    plan = _ops.permute_plan(e.cuda(), E, want_within=True)
    order, inv, counts = O.permute_plan_fast(e, E)
    within, _ = O.slot_assignment(e, E)
    assert torch.equal(plan.order.cpu().long(), order)
    assert torch.equal(plan.inv_order.cpu().long(), inv)
    assert torch.equal(plan.counts.cpu(), counts) and torch.equal(plan.kept_counts.cpu(), counts)
    assert torch.equal(plan.within.cpu().long(), within)


@pytest.mark.parametrize("T,k,E,skew,factor", [(512, 2, 8, 1.0, 1.0), (512, 2, 8, 2.0, 0.5), (16384, 6, 64, 1.1, 1.25), (300, 2, 4, 0.0, 0.3)])
def test_capacity_drop_set_bit_exact(gpu, T, k, E, skew, factor):
    from picotron_amd import _ops
    from picotron_amd.expert_parallel.capacity_moe import compute_capacity

    idx = _zipf_idx(T, k, E, skew, seed=7).reshape(-1)
    C = compute_capacity(T, k, E, factor)
    assert C == O.compute_capacity(T, k, E, factor)
    within, counts = O.slot_assignment(idx, E)
    plan = _ops.permute_plan(idx.cuda(), E, capacity=C, want_within=True)
    keep = plan.inv_order.cpu() >= 0
    assert torch.equal(keep, within < C)                              # the drop set
    assert torch.equal(plan.counts.cpu(), counts)
    assert torch.equal(plan.kept_counts.cpu(), counts.clamp(max=C))
    # kept rows: compact layout, expert after expert, ascending original row inside an expert
    kept_rows = torch.nonzero(keep).squeeze(1)
    want_order = kept_rows[torch.argsort(idx[kept_rows], stable=True)]
    n_kept = int(keep.sum())
    assert torch.equal(plan.order.cpu()[:n_kept].long(), want_order)
    assert torch.all(plan.order.cpu()[n_kept:] == -1)
    # later rounds of the dropless loop keep the next window of ranks
    for r in (1, 2):
        pr = _ops.permute_plan(idx.cuda(), E, capacity=C, round_index=r)
        keep_r = pr.inv_order.cpu() >= 0
        assert torch.equal(keep_r, (within >= r * C) & (within < (r + 1) * C))
        assert torch.equal(pr.kept_counts.cpu(), (counts - r * C).clamp(min=0, max=C))


def test_capacity_tables_of_the_reference_on_gpu(gpu):
    """Drop percentages of the reference's README table (tests/golden/capacity_tables.json) from the GPU plan."""
    import json
    import os

    from picotron_amd import _ops

    gold = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "capacity_tables.json")))
    E, k, T = gold["num_experts"], gold["top_k"], gold["num_tokens"]
    for row in gold["vary_skew_factor_1"]:
        idx = _zipf_idx(T, k, E, row["skew"], seed=100 + int(row["skew"] * 10)).reshape(-1)
        plan = _ops.permute_plan(idx.cuda(), E, capacity=row["capacity"])
        drop = 100.0 * float((plan.inv_order < 0).sum()) / idx.numel()
        assert round(drop, 1) == row["drop_pct"]
        assert int(plan.counts.max()) == row["worst_buf"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [256, 100, 4096])
def test_gather_and_combine_match_oracle(gpu, dtype, H):
    from picotron_amd import _ops

    T, k, E = 333, 3, 8
    g = torch.Generator().manual_seed(H)
    tokens = torch.randn(T, H, generator=g).to(dtype)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    w = torch.softmax(torch.randn(T, k, generator=g), -1).to(dtype)
    plan = _ops.permute_plan(idx.reshape(-1).cuda(), E)
    xs = _ops.expand_permute(tokens.cuda(), plan.order, plan.inv_order, k, T * k)
    routed, eidx, wf, _ = O.expand_routed(tokens, idx, w)
    order, inv, _ = O.permute_plan_fast(eidx, E)
    assert torch.equal(xs.cpu(), routed[order])                       # pure data movement: bit-exact
    y = torch.randn(T * k, H, generator=g).to(dtype)                  # stand-in expert output, sorted order
    out = _ops.unpermute_combine(y.cuda(), w.cuda(), plan.inv_order, plan.order, T, k)
    want = O.combine_topk(y[inv], wf, T, k)
    if dtype == torch.float32:
        assert torch.allclose(out.cpu(), want, rtol=1e-6, atol=1e-7)
    else:
        assert torch.equal(out.cpu(), want)                           # same rounding points as the reference ops
    # with dropped rows (capacity mode) == the reference's weighted index_add into zeros in the tensor dtype
    keep = torch.rand(T * k, generator=g) > 0.3
    inv_drop = torch.where(keep, inv, torch.full_like(inv, -1)).int()
    out_seq = _ops.unpermute_combine(y.cuda(), w.cuda(), inv_drop.cuda(), plan.order, T, k)
    tok = torch.arange(T).repeat_interleave(k)
    contrib = y[inv[keep]] * wf[keep].unsqueeze(-1)
    want_seq = torch.zeros(T, H, dtype=dtype).index_add(0, tok[keep], contrib)
    if dtype == torch.float32:
        assert torch.allclose(out_seq.cpu(), want_seq, rtol=1e-6, atol=1e-7)
    else:
        assert torch.equal(out_seq.cpu(), want_seq)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_permute_combine_backward(gpu, dtype):
    from picotron_amd import _ops

    T, k, E, H = 100, 2, 4, 64
    g = torch.Generator().manual_seed(1)
    tokens = torch.randn(T, H, generator=g).to(dtype)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    w = torch.softmax(torch.randn(T, k, generator=g), -1).to(dtype)
    gout = torch.randn(T, H, generator=g).to(dtype)
    # GPU: expand+permute -> (identity expert) -> combine
    tg, wg = tokens.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    plan = _ops.permute_plan(idx.reshape(-1).cuda(), E)
    xs = _ops.expand_permute(tg, plan.order, plan.inv_order, k, T * k)
    out = _ops.unpermute_combine(xs * 1.0, wg, plan.inv_order, plan.order, T, k)
    out.backward(gout.cuda())
    # oracle: autograd through the reference's indexing ops
    tr, wr = tokens.clone().requires_grad_(True), w.clone().requires_grad_(True)
    routed, eidx, wf, _ = O.expand_routed(tr, idx, wr)
    order, inv, _ = O.permute_plan_fast(eidx, E)
    ref = O.combine_topk((routed[order] * 1.0)[inv], wf, T, k)
    ref.backward(gout)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    assert torch.allclose(out.detach().cpu().float(), ref.detach().float(), **tol)
    assert torch.allclose(tg.grad.cpu().float(), tr.grad.float(), **tol)
    if dtype == torch.float32:
        assert torch.allclose(wg.grad.cpu().float(), wr.grad.float(), rtol=1e-5, atol=1e-5)
    else:  # bf16 gradients: within 1e-2 of the tensor's magnitude
        assert (wg.grad.cpu().float() - wr.grad.float()).abs().max() <= 1e-2 * wr.grad.float().abs().max()


@pytest.mark.parametrize("k", [1, 2, 6, 12])
def test_combine_every_top_k_width(gpu, k):
    """Forward and backward of the combine for each compile-time bound of k the kernels are built for (2, 8, 16)."""
    from picotron_amd import _ops

    T, E, H = 70, 16, 264
    g = torch.Generator().manual_seed(k)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    w = torch.softmax(torch.randn(T, k, generator=g), -1).bfloat16()
    y = torch.randn(T * k, H, generator=g).bfloat16()                  # expert outputs in sorted order
    gout = torch.randn(T, H, generator=g).bfloat16()
    plan = _ops.permute_plan(idx.reshape(-1).cuda(), E)
    yg, wg = y.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    out = _ops.unpermute_combine(yg, wg, plan.inv_order, plan.order, T, k)
    out.backward(gout.cuda())
    order, inv, _ = O.permute_plan_fast(idx.reshape(-1), E)
    yr, wr = y.clone().requires_grad_(True), w.clone().requires_grad_(True)
    want = O.combine_topk(yr[inv], wr.reshape(-1), T, k)
    want.backward(gout)
    assert torch.equal(out.detach().cpu(), want.detach())              # same rounding points as the reference ops
    assert torch.allclose(yg.grad.cpu().float(), yr.grad.float(), rtol=1e-2, atol=1e-2)
    assert (wg.grad.cpu().float() - wr.grad.float()).abs().max() <= 1e-2 * wr.grad.float().abs().max()
