"""GPU parity of the whole MoELayer against the CPU oracle, following the recipes of the reference's
own layer tests (tests/test_expert_parallel.py:51-71, tests/test_capacity_moe.py:41-111,
tests/test_load_balance.py:31-99) plus the tiny-config benchmark case (512 tokens, H256, I512, E8, top-2, fp32)."""

import types

import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def make_config(hidden=16, inter=32, num_experts=4, top_k=2, n_shared=0, latent=0, **kw):
    return types.SimpleNamespace(hidden_size=hidden, intermediate_size=inter, num_experts=num_experts, num_experts_per_tok=top_k,
                                 num_shared_experts=n_shared, norm_topk_prob=True, moe_latent_dim=latent, **kw)


def oracle_weights(moe):
    """Copy a layer's parameters into the oracle's container (CPU)."""
    c = lambda t: t.detach().cpu().clone()
    w = O.LayerWeights(
        c(moe.gate.weight),
        torch.stack([c(e.gate_proj.weight) for e in moe.local_experts]),
        torch.stack([c(e.up_proj.weight) for e in moe.local_experts]),
        torch.stack([c(e.down_proj.weight) for e in moe.local_experts]),
        router_b=c(moe.gate.bias) if moe.gate.bias is not None else None,
        expert_bias=c(moe.expert_bias).float(),
    )
    if moe.shared_expert is not None:
        s = moe.shared_expert
        w.shared = (c(s.gate_proj.weight), c(s.up_proj.weight), c(s.down_proj.weight))
    if moe.latent:
        w.latent = (c(moe.down_proj_latent.weight), c(moe.up_proj_latent.weight))
    return w


def layer_grads(moe):
    """The layer's parameter gradients in the order of ``LayerWeights.tensors()``."""
    gs = [moe.gate.weight.grad] + [torch.stack([getattr(e, n).weight.grad for e in moe.local_experts])
                                   for n in ("gate_proj", "up_proj", "down_proj")]
    if moe.gate.bias is not None:
        gs.append(moe.gate.bias.grad)
    if moe.shared_expert is not None:
        gs += [getattr(moe.shared_expert, n).weight.grad for n in ("gate_proj", "up_proj", "down_proj")]
    if moe.latent:
        gs += [moe.down_proj_latent.weight.grad, moe.up_proj_latent.weight.grad]
    return [g.detach().cpu().float() for g in gs]


def given_logits(x, w, logits_gpu):
    """Router logits with the VALUES the GPU computed and the gradient of the oracle's own gate Linear: the GPU's GEMM
    and the CPU's round a bf16 logit differently now and then, which flips near-tie picks; scoring the GPU's logits
    with the oracle's selection rule keeps the comparison about the kernels.  a + (b - a) is exact in fp32 for two
    nearby low-precision values."""
    own = torch.nn.functional.linear(x, w.router_w, w.router_b)
    return (own.float() + (logits_gpu.float() - own.float()).detach()).to(own.dtype)


def assert_close(got, want, rtol, what=""):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    err, scale = (got - want).abs().max().item(), want.abs().max().item()
    assert err <= rtol * scale, f"{what}: max |err| {err:.3e} > {rtol} x {scale:.3e}"


def build(cfg, seed=0, std=None, dtype=torch.float32):
    from picotron_amd.expert_parallel.expert_parallel import MoELayer

    torch.manual_seed(seed)
    moe = MoELayer(cfg)
    if std is not None:
        g = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            for p in moe.parameters():
                p.copy_(std * torch.randn(p.shape, generator=g))
    return moe.to(dtype).cuda()


def test_local_ep1_recipe(gpu):
    cfg = make_config(n_shared=1)
    moe = build(cfg)
    tokens = torch.randn(8, cfg.hidden_size, generator=torch.Generator().manual_seed(1))
    out = moe(tokens.view(2, 4, -1).cuda()).view(-1, cfg.hidden_size)
    w = oracle_weights(moe)
    assert torch.allclose(out.cpu(), O.moe_brute_force(tokens, w, cfg.num_experts_per_tok), atol=1e-5)
    out.sum().backward()
    assert moe.gate.weight.grad is not None
    assert all(e.up_proj.weight.grad is not None for e in moe.local_experts)


def test_tiny_config_fp32_forward_parity(gpu):
    """512 tokens (2 x 256), hidden 256, FFN 512, 8 experts, top-2, softmax router, no capacity cap, N(0, 0.02) weights."""
    cfg = make_config(hidden=256, inter=512, num_experts=8, top_k=2)
    moe = build(cfg, seed=0, std=0.02)
    x = torch.randn(2, 256, 256, generator=torch.Generator().manual_seed(0))
    out = moe(x.cuda()).cpu().view(-1, 256)
    ref, info = O.moe_forward(x.view(-1, 256), oracle_weights(moe), 2)
    idx, wts = moe._route(x.view(-1, 256).cuda())
    assert not O.tie_rows(info["logits"], 2).any()
    assert torch.equal(idx.cpu(), info["topk_idx"])                               # routing indices bit-exact
    assert torch.allclose(wts.cpu(), info["topk_w"], rtol=1e-5)
    assert (out - ref).abs().max() <= 1e-5 * ref.abs().max()                      # fp32 outputs within 1e-5 relative
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5 * ref.abs().max().item())


@pytest.mark.parametrize("latent", [0, 8])
def test_gradients_match_oracle_autograd(gpu, latent):
    cfg = make_config(hidden=32, inter=48, num_experts=4, top_k=2, n_shared=1, latent=latent)
    moe = build(cfg, seed=3, std=0.2)
    x = torch.randn(2, 9, 32, generator=torch.Generator().manual_seed(4))
    xg = x.cuda().requires_grad_(True)
    out = moe(xg)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5))
    out.backward(gout.cuda())
    w = oracle_weights(moe)
    assert (w.latent is not None) == bool(latent) and w.gate_w.shape[2] == (latent or 32)
    for t in w.tensors():
        t.requires_grad_(True)
    xr = x.view(-1, 32).clone().requires_grad_(True)
    ref, _ = O.moe_forward(xr, w, 2)
    ref.backward(gout.view(-1, 32))
    assert torch.allclose(out.detach().cpu().view(-1, 32), ref.detach(), atol=1e-5)
    assert torch.allclose(xg.grad.cpu().view(-1, 32), xr.grad, atol=1e-5)
    for got, want in zip(layer_grads(moe), w.tensors()):   # router, experts, shared expert, latent projections
        assert torch.allclose(got, want.grad, atol=1e-5)


@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
def test_latent_layer_matches_oracle(gpu, dtype, rtol):
    """LatentMoE (reference expert_parallel.py:59-69, 226-228, 250-252) at a size the MFMA kernels tile: hidden 512,
    latent 256, with the FP8 dispatch on the latent rows in the bf16 case; forward and every gradient."""
    fp8 = dtype == torch.bfloat16
    cfg = make_config(hidden=512, inter=256, num_experts=4, top_k=2, n_shared=1, latent=256, ep_fp8_dispatch=fp8)
    moe = build(cfg, seed=6, std=0.06, dtype=dtype)
    x = torch.randn(3, 50, 512, generator=torch.Generator().manual_seed(7)).to(dtype)
    gout = torch.randn(150, 512, generator=torch.Generator().manual_seed(8)).to(dtype)
    xg = x.cuda().requires_grad_(True)
    out = moe(xg)
    out.backward(gout.view_as(out).cuda())
    w = oracle_weights(moe)
    for t in w.tensors():
        t.requires_grad_(True)
    xr = x.view(-1, 512).clone().requires_grad_(True)
    logits = given_logits(xr, w, moe.gate(xg.detach().view(-1, 512)).detach().cpu())
    ref, info = O.moe_forward(xr, w, 2, logits=logits, fp8_dispatch=fp8)
    ref.backward(gout)
    assert info["y_routed"].shape[1] == 256
    assert_close(out.view(-1, 512), ref, rtol, "out")
    assert_close(xg.grad.view(-1, 512), xr.grad, rtol, "d x")
    names = ["router", "gate", "up", "down", "shared gate", "shared up", "shared down", "latent down", "latent up"]
    for name, got, want in zip(names, layer_grads(moe), w.tensors()):
        assert_close(got, want.grad, rtol, "d " + name)


def _run(moe, x):
    moe.zero_grad(set_to_none=True)
    out = moe(x).view(-1, moe.hidden_size)
    out.sum().backward()
    return out.detach().clone(), {n: p.grad.detach().clone() for n, p in moe.named_parameters() if p.grad is not None}


@pytest.mark.parametrize("latent", [0, 8])
def test_capacity_dropless_matches_naive(gpu, latent):
    moe = build(make_config(num_experts=4, top_k=2, n_shared=1, latent=latent))
    x = torch.randn(2, 8, 16, generator=torch.Generator().manual_seed(123)).cuda()
    moe.ep_capacity_factor = 0.0
    out_base, g_base = _run(moe, x)
    moe.ep_capacity_factor, moe.ep_capacity_dropless, moe.ep_max_rounds = 1.0, True, 64
    out_cap, g_cap = _run(moe, x)
    assert (out_base - out_cap).abs().max().item() < 1e-5
    assert max((g_base[n] - g_cap[n]).abs().max().item() for n in g_base) < 1e-5


def test_capacity_capped_drops_matches_oracle(gpu):
    moe = build(make_config(num_experts=4, top_k=2, n_shared=1))
    x = torch.randn(2, 8, 16, generator=torch.Generator().manual_seed(123))
    moe.ep_capacity_factor = 0.0
    out_base, _ = _run(moe, x.cuda())
    moe.ep_capacity_factor, moe.ep_capacity_dropless = 0.5, False
    out_capped, g_capped = _run(moe, x.cuda())
    assert torch.isfinite(out_capped).all() and all(torch.isfinite(g).all() for g in g_capped.values())
    assert (out_base - out_capped).abs().max().item() > 0
    ref, info = O.moe_forward(x.view(-1, 16), oracle_weights(moe), 2, capacity_factor=0.5, capacity_dropless=False)
    assert torch.allclose(out_capped.cpu(), ref, atol=1e-5)


def _zipf_layer(dtype, max_rounds, dropless=True, cap=0.25):
    """8 experts, top-2, a Zipf bias on the gate so the first experts overflow their capacity several times over."""
    cfg = make_config(hidden=256, inter=128, num_experts=8, top_k=2, n_shared=1, ep_capacity_factor=cap,
                      ep_capacity_dropless=dropless, ep_max_rounds=max_rounds)
    moe = build(cfg, seed=21, std=0.08, dtype=torch.float32)
    moe.gate.bias = torch.nn.Parameter(-1.5 * torch.log(torch.arange(1, 9, dtype=torch.float32)).cuda())
    return moe.to(dtype)


@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("max_rounds", [64, 2])
def test_dropless_rounds_match_oracle(gpu, dtype, rtol, max_rounds):
    """Static-memory dropless capacity (reference capacity_moe.py:96-120) under a skewed router that needs at least
    three rounds: outputs and gradients against the oracle's rounds, with enough rounds (nothing lost) and with
    ``ep_max_rounds`` = 2, smaller than needed (rows of rank >= 2C are lost, and get no gradient)."""
    moe = _zipf_layer(dtype, max_rounds)
    T, H = 384, 256
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(22)).to(dtype)
    gout = torch.randn(T, H, generator=torch.Generator().manual_seed(23)).to(dtype)
    xg = x.cuda().requires_grad_(True)
    out = moe(xg.view(2, T // 2, H))
    out.backward(gout.view_as(out).cuda())
    w = oracle_weights(moe)
    for t in w.tensors():
        t.requires_grad_(True)
    xr = x.clone().requires_grad_(True)
    logits = given_logits(xr, w, moe.gate(xg.detach()).detach().cpu())
    ref, info = O.moe_forward(xr, w, 2, logits=logits, capacity_factor=0.25, capacity_dropless=True, max_rounds=max_rounds)
    ref.backward(gout)
    C = info["capacity"]
    need = -(-int(info["counts"].max()) // C)
    assert C == 24 and need >= 3, (C, need)
    assert info["rounds"] == min(need, max_rounds)
    assert bool(info["keep"].all()) == (max_rounds >= need)
    assert_close(out.view(T, H), ref, rtol, "out")
    assert_close(xg.grad, xr.grad, rtol, "d x")
    names = ["router", "gate", "up", "down", "router bias", "shared gate", "shared up", "shared down"]
    for name, got, want in zip(names, layer_grads(moe), w.tensors()):
        assert_close(got, want.grad, rtol, "d " + name)
    if max_rounds < need:   # the cut really lost rows: the uncapped layer differs
        base, _ = O.moe_forward(x, w, 2, logits=logits.detach())
        assert (base.float() - ref.detach().float()).abs().max() > 10 * rtol * ref.detach().float().abs().max()


def test_aux_loss_and_loss_free_bias(gpu):
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss

    moe = build(make_config(num_experts=8, top_k=2, router_aux_loss_coef=0.01))
    moe.train()
    x = torch.randn(4, 8, 16, generator=torch.Generator().manual_seed(1))
    out = moe(x.cuda())
    aux = collect_aux_loss(moe)
    assert aux is not None and aux.item() > 0 and collect_aux_loss(moe) is None      # drained once
    _, info = O.moe_forward(x.view(-1, 16), oracle_weights(moe), 2, aux_coef=0.01, training=True)
    assert abs(aux.item() - info["aux"].item()) < 1e-6
    (out.float().pow(2).mean() + aux).backward()
    assert moe.gate.weight.grad is not None
    moe.eval()
    moe(x.cuda())
    assert collect_aux_loss(moe) is None                                             # eval: nothing stashed
    moe2 = build(make_config(num_experts=8, top_k=2))
    moe2.train()
    moe2(x.cuda())
    assert collect_aux_loss(moe2) is None                                            # coef = 0

    # loss-free bias: one step moves the most loaded expert below the least loaded one
    moe3 = build(make_config(num_experts=8, top_k=2, router_bias_update_rate=0.01))
    moe3.train()
    assert moe3.use_loss_free
    xb = torch.randn(8, 16, 16, generator=torch.Generator().manual_seed(2))
    _, info3 = O.moe_forward(xb.view(-1, 16), oracle_weights(moe3), 2, use_loss_free=True, bias_rate=0.01, training=True)
    load0 = torch.bincount(info3["topk_idx"].reshape(-1), minlength=8)
    moe3(xb.cuda())
    assert torch.allclose(moe3.expert_bias.cpu(), info3["new_bias"], atol=1e-8)
    assert moe3.expert_bias[load0.argmax()] < moe3.expert_bias[load0.argmin()]

    def cumulative(rate):
        m = build(make_config(num_experts=8, top_k=2, router_bias_update_rate=rate))
        m.train()
        total = torch.zeros(8)
        for _ in range(300):
            idx, _ = m._route(xb.view(-1, 16).cuda())
            total += torch.bincount(idx.reshape(-1).cpu(), minlength=8).float()
        return total

    off, on = cumulative(0.0), cumulative(0.01)
    assert on.std() < 0.5 * off.std()


def test_fp8_dispatch_bf16(gpu):
    cfg = make_config(hidden=256, inter=512, num_experts=8, top_k=2, n_shared=1)
    moe = build(cfg, seed=0, std=0.05, dtype=torch.bfloat16)
    x = torch.randn(8, 64, 256, generator=torch.Generator().manual_seed(123)).bfloat16()
    moe.ep_fp8_dispatch = False
    out_bf16 = moe(x.cuda()).float()
    moe.ep_fp8_dispatch = True
    out_fp8 = moe(x.cuda())
    out_fp8.float().sum().backward()
    rel = ((out_bf16 - out_fp8.float()).norm() / out_bf16.norm()).item()
    assert 0 < rel < 0.05
    g = moe.local_experts[0].up_proj.weight.grad
    assert g is not None and torch.isfinite(g).all()
    w = oracle_weights(moe)
    ref, info = O.moe_forward(x.view(-1, 256), w, 2, fp8_dispatch=True)
    got = out_fp8.detach().cpu().float().view(-1, 256)
    assert (got - ref.float()).abs().max() <= 1e-2 * ref.float().abs().max()


@pytest.mark.parametrize("arith", ["bf16", "fp32"])
def test_fp8_dispatch_aux_forward_backward_small(gpu, arith):
    """The headline configuration in small (hidden 256, FFN 512, 8 experts, top-2, bf16, FP8 dispatch, aux-loss
    coefficient 0.01, training mode, loss = <out, g> + aux): output, aux and every gradient within 1e-2 of the oracle
    -- once with the oracle in the layer's own bf16 (the reference's rounding points), once with the same weights
    and inputs evaluated in fp32 arithmetic (the rows still quantised as bf16 rows)."""
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss

    cfg = make_config(hidden=256, inter=512, num_experts=8, top_k=2, ep_fp8_dispatch=True, router_aux_loss_coef=0.01)
    moe = build(cfg, seed=0, std=0.05, dtype=torch.bfloat16).train()
    T, H = 1024, 256
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(31)).bfloat16()
    gout = torch.randn(T, H, generator=torch.Generator().manual_seed(32)).bfloat16()
    xg = x.cuda().requires_grad_(True)
    out = moe(xg.view(4, 256, H))
    aux = collect_aux_loss(moe)
    torch.autograd.backward([out, aux], [gout.view_as(out).cuda(), torch.ones_like(aux)])
    wide = torch.float32 if arith == "fp32" else torch.bfloat16
    w = oracle_weights(moe)
    w.router_w, w.gate_w, w.up_w, w.down_w = (t.to(wide) for t in (w.router_w, w.gate_w, w.up_w, w.down_w))
    for t in w.tensors():
        t.requires_grad_(True)
    xr = x.to(wide).requires_grad_(True)
    logits = given_logits(xr, w, moe.gate(xg.detach()).detach().cpu())
    ref, info = O.moe_forward(xr, w, 2, logits=logits, fp8_dispatch=True, aux_coef=0.01, training=True,
                              dispatch_dtype=torch.bfloat16)
    torch.autograd.backward([ref, info["aux"]], [gout.to(wide), torch.ones(())])
    assert abs(aux.item() - info["aux"].item()) <= 1e-5 * abs(info["aux"].item())
    assert_close(out.view(T, H), ref, 1e-2, "out")
    assert_close(xg.grad, xr.grad, 1e-2, "d x")
    for name, got, want in zip(["router", "gate", "up", "down"], layer_grads(moe), w.tensors()):
        assert_close(got, want.grad, 1e-2, "d " + name)


def test_state_dict_names_and_weight_stacking(gpu):
    cfg = make_config(hidden=32, inter=64, num_experts=4, top_k=2, n_shared=1)
    moe = build(cfg, seed=1)
    keys = set(moe.state_dict().keys())
    want = {"gate.weight", "expert_bias"} | {f"local_experts.{i}.{p}_proj.weight" for i in range(4) for p in ("gate", "up", "down")}
    want |= {f"shared_expert.{p}_proj.weight" for p in ("gate", "up", "down")}
    assert keys == want
    x = torch.randn(1, 12, 32, generator=torch.Generator().manual_seed(2))
    y0 = moe(x.cuda()).detach().cpu()
    # after the first forward every expert parameter is a slice of one stacked buffer
    gw = moe._stacks[0]
    assert all(e.gate_proj.weight.data_ptr() == gw[i].data_ptr() for i, e in enumerate(moe.local_experts))
    # in-place updates (optimizer steps, load_state_dict) are seen without re-stacking
    sd = {k: v.clone() for k, v in moe.state_dict().items()}
    with torch.no_grad():
        moe.local_experts[2].gate_proj.weight.mul_(2.0)
    y1 = moe(x.cuda()).detach().cpu()
    assert moe._stacks[0] is gw and not torch.equal(y0, y1)
    moe.load_state_dict(sd)
    assert torch.equal(moe(x.cuda()).detach().cpu(), y0)
    # re-assigning a parameter's storage or casting the module triggers one re-stack
    moe.local_experts[1].up_proj.weight.data = moe.local_experts[1].up_proj.weight.data.clone() * 0
    y2 = moe(x.cuda()).detach().cpu()
    assert not torch.equal(y2, y0)
    ref, _ = O.moe_forward(x.view(-1, 32), oracle_weights(moe), 2)
    assert torch.allclose(y2.view(-1, 32), ref, atol=1e-5)
    moe_bf = moe.to(torch.bfloat16)
    yb = moe_bf(x.cuda().bfloat16())
    assert yb.dtype == torch.bfloat16 and moe_bf._stacks[0].dtype == torch.bfloat16


def test_private_helpers_keep_their_contracts(gpu):
    cfg = make_config(hidden=32, inter=64, num_experts=4, top_k=2)
    moe = build(cfg, seed=2, std=0.2)
    T = 20
    tokens = torch.randn(T, 32, generator=torch.Generator().manual_seed(3))
    w = oracle_weights(moe)
    idx, wt = moe._route(tokens.cuda())
    routed, eidx, wflat = moe._expand_routed(tokens.cuda(), idx, wt)
    r_routed, r_eidx, r_w, _ = O.expand_routed(tokens, idx.cpu(), wt.cpu())
    assert torch.equal(routed.cpu(), r_routed) and torch.equal(eidx.cpu(), r_eidx) and torch.equal(wflat.cpu(), r_w)
    y = moe._run_local_experts(routed, eidx)
    ry, (order, inv, counts) = O.run_local_experts(r_routed, r_eidx, w)
    assert torch.allclose(y.cpu(), ry, atol=1e-5)
    out = moe._combine_topk(y, wflat, T)
    assert torch.allclose(out.cpu(), O.combine_topk(ry, r_w, T, 2), atol=1e-5)
    ys = moe._grouped_experts(routed[order.cuda()], counts.cuda())
    assert torch.allclose(ys.cpu(), O.expert_ffn(r_routed[order], counts, w.gate_w, w.up_w, w.down_w), atol=1e-5)
    # externally supplied routing through the private paths (as the reference's ablation does)
    ext_idx = torch.stack([torch.randperm(4)[:2] for _ in range(T)])
    ext_w = torch.softmax(torch.rand(T, 2), -1)
    naive = moe._moe_naive(tokens.cuda(), ext_idx.cuda(), ext_w.cuda())
    ref, _ = O.moe_forward(tokens, w, 2, routing=(ext_idx, ext_w))
    assert torch.allclose(naive.cpu(), ref, atol=1e-5)
    moe.ep_capacity_factor, moe.ep_capacity_dropless, moe.ep_max_rounds = 1.0, True, 64
    capped = moe._moe_capped(tokens.cuda(), ext_idx.cuda(), ext_w.cuda())
    assert (naive - capped).abs().max().item() < 1e-5


def test_capacity_moe_function_signature(gpu):
    from picotron_amd.expert_parallel.capacity_moe import _slot_assignment, capacity_moe, compute_capacity

    cfg = make_config(hidden=32, inter=64, num_experts=4, top_k=2)
    moe = build(cfg, seed=5, std=0.2)
    T, k, E = 24, 2, 4
    tokens = torch.randn(T, 32, generator=torch.Generator().manual_seed(6))
    idx = torch.stack([torch.randperm(E)[:k] for _ in range(T)])
    wt = torch.softmax(torch.rand(T, k), -1)
    token_idx = torch.arange(T).repeat_interleave(k)
    C = compute_capacity(T, k, E, 0.5)
    out = capacity_moe(tokens[token_idx].cuda(), idx.reshape(-1).cuda(), wt.reshape(-1).cuda(), token_idx.cuda(), T, 32, E, E, 1, None,
                       moe._grouped_experts, C, False, 8)
    ref, _ = O.moe_forward(tokens, oracle_weights(moe), k, routing=(idx, wt), capacity_factor=0.5, capacity_dropless=False)
    assert torch.allclose(out.cpu(), ref, atol=1e-5)
    within, counts = _slot_assignment(idx.reshape(-1).cuda(), E)
    rw, rc = O.slot_assignment(idx.reshape(-1), E)
    assert torch.equal(within.cpu(), rw) and torch.equal(counts.cpu(), rc)


def _sample_check(moe, x_tokens, out, idx, wts, keep, sample, rtol):
    """Per-token brute force on the CPU for a sample of tokens: each kept (token, expert) pick goes through that
    expert's MLP alone, products rounded to the tensor dtype, fp32 sum rounded once, plus the shared expert."""
    k = idx.shape[1]
    scale = out.float().abs().max().item()
    cache = {}

    def expert_w(e):
        if e not in cache:
            ex = moe.local_experts[e]
            cache[e] = tuple(t.weight.detach().cpu() for t in (ex.gate_proj, ex.up_proj, ex.down_proj))
        return cache[e]

    shared = None
    if moe.shared_expert is not None:
        s = moe.shared_expert
        shared = tuple(t.weight.detach().cpu() for t in (s.gate_proj, s.up_proj, s.down_proj))
    worst = 0.0
    for t in sample:
        row = x_tokens[t : t + 1]
        acc = torch.zeros(1, row.shape[1], dtype=torch.float32)
        for j in range(k):
            if keep is not None and not bool(keep[t * k + j]):
                continue
            y = O.mlp(row, *expert_w(int(idx[t, j])))
            acc += (y * wts[t, j]).float()
        ref = acc.to(row.dtype)
        if shared is not None:
            ref = ref + O.mlp(row, *shared)
        worst = max(worst, (out[t].float() - ref[0].float()).abs().max().item())
    assert worst <= rtol * scale, (worst, scale)


def test_mixtral_shape_forward_full_size(gpu):
    """8192 tokens, hidden 4096, FFN 14336, 8 experts, top-2, bf16 (the grouped-GEMM benchmark shape): routing
    bit-exact against the oracle on the same logits, permutation bit-exact, outputs of sampled tokens within 1e-2."""
    import bench
    from picotron_amd import _ops

    w = bench.WORKLOADS["c3"]
    moe = bench.build_layer(w, gpu, torch.bfloat16)
    x = torch.randn(w["T"], w["H"], generator=torch.Generator().manual_seed(0)).bfloat16()
    with torch.no_grad():
        xg = x.to(gpu)
        out = moe(xg.view(1, w["T"], w["H"])).view(w["T"], w["H"]).cpu()
        logits = moe.gate(xg).cpu()
        idx, wts = moe._route(xg)
        plan = _ops.permute_plan(idx.reshape(-1), w["E"])
    ridx, rw, _ = O.softmax_topk_route(logits, w["k"])
    assert torch.equal(idx.cpu(), ridx)                                    # incl. the tie rows of bf16 logits
    assert int(O.tie_rows(logits, w["k"]).sum()) > 0
    order, inv, counts = O.permute_plan_fast(ridx.reshape(-1), w["E"])
    assert torch.equal(plan.order.cpu().long(), order) and torch.equal(plan.counts.cpu(), counts)
    _sample_check(moe, x, out, ridx, wts.cpu(), None, range(0, w["T"], w["T"] // 24), rtol=1e-2)


def test_fine_grained_skewed_capacity_full_size(gpu):
    """16384 tokens, hidden 2048, 64 experts of FFN 1408, top-6, shared expert 2816, Zipf(1.1) router bias,
    capacity factor 1.25 with drops: drop set bit-exact, outputs of sampled tokens within 1e-2."""
    import bench
    from picotron_amd import _ops
    from picotron_amd.expert_parallel.capacity_moe import compute_capacity

    w = bench.WORKLOADS["c4"]
    moe = bench.build_layer(w, gpu, torch.bfloat16)
    x = torch.randn(w["T"], w["H"], generator=torch.Generator().manual_seed(0)).bfloat16()
    with torch.no_grad():
        xg = x.to(gpu)
        out = moe(xg.view(1, w["T"], w["H"])).view(w["T"], w["H"]).cpu()
        logits = moe.gate(xg).cpu()
        idx, wts = moe._route(xg)
    ridx, rw, _ = O.softmax_topk_route(logits, w["k"])
    ties = O.tie_rows(logits, w["k"])
    assert torch.equal(idx.cpu(), ridx)
    C = compute_capacity(w["T"], w["k"], w["E"], w["cap"])
    assert C == 1920
    within, counts = O.slot_assignment(ridx.reshape(-1), w["E"])
    keep = within < C
    plan = _ops.permute_plan(idx.reshape(-1), w["E"], capacity=C)
    assert torch.equal(plan.inv_order.cpu() >= 0, keep)                    # the drop set
    assert 0 < int((~keep).sum()) < keep.numel() and int(counts.max()) > C  # the skew really overflows experts
    assert torch.equal(plan.kept_counts.cpu(), counts.clamp(max=C))
    sample = list(range(0, w["T"], w["T"] // 24))
    dropped_tokens = torch.nonzero((~keep).view(-1, w["k"]).any(1)).squeeze(1)[:8].tolist()
    _sample_check(moe, x, out, ridx, wts.cpu(), keep, sample + dropped_tokens, rtol=1e-2)
    assert int(ties.sum()) >= 0


def test_training_steps_follow_the_oracle(gpu):
    """Two residual MoE blocks (routed + shared experts, aux loss 0.01) trained for four SGD steps, fp32: the loss of
    every step and the final parameters follow the same loop run on the CPU through the oracle with torch autograd
    (how the layer sits in picotron's DecoderLayer, model.py:329-331, and train step, train.py:73), the per-expert
    parameters keep receiving their gradients through the stacked buffers, and the state dict round-trips."""
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss

    cfg = make_config(hidden=32, inter=64, num_experts=4, top_k=2, n_shared=1, router_aux_loss_coef=0.01)
    blocks = torch.nn.ModuleList([build(cfg, seed=s, std=0.15) for s in (1, 2)])
    blocks.train()
    ws = [oracle_weights(b) for b in blocks]
    for w in ws:
        for t in w.tensors():
            t.requires_grad_(True)
    gen = torch.Generator().manual_seed(9)
    x = torch.randn(2, 48, 32, generator=gen)
    target = torch.randn(2, 48, 32, generator=gen)
    lr = 0.02
    opt = torch.optim.SGD(blocks.parameters(), lr=lr)
    losses = []
    for step in range(4):
        # device
        opt.zero_grad(set_to_none=True)
        h = x.cuda()
        for b in blocks:
            h = h + b(h)
        loss = (h - target.cuda()).pow(2).mean() + collect_aux_loss(blocks)
        loss.backward()
        opt.step()
        # oracle
        ho = x.view(-1, 32)
        aux = 0.0
        for w in ws:
            out, info = O.moe_forward(ho, w, 2, aux_coef=0.01, training=True)
            ho = ho + out
            aux = aux + info["aux"]
        loss_o = (ho - target.view(-1, 32)).pow(2).mean() + aux
        grads = torch.autograd.grad(loss_o, [t for w in ws for t in w.tensors()])
        with torch.no_grad():
            for t, g in zip([t for w in ws for t in w.tensors()], grads):
                t -= lr * g
        assert abs(loss.item() - loss_o.item()) <= 2e-5 * abs(loss_o.item()), (step, loss.item(), loss_o.item())
        losses.append(loss.item())
    assert losses[-1] < losses[0] - 0.1                                              # and it trains
    for b, w in zip(blocks, ws):
        got = oracle_weights(b)
        for a, r in zip(got.tensors(), w.tensors()):
            assert (a - r.detach()).abs().max().item() <= 1e-4 * r.detach().abs().max().item() + 1e-6
    # every per-expert parameter moved (its .grad came through the stacked buffer) and the state dict round-trips
    sd = blocks[0].state_dict()
    assert {"gate.weight", "local_experts.3.down_proj.weight", "shared_expert.up_proj.weight", "expert_bias"} <= set(sd)
    fresh = build(cfg, seed=5, std=0.15)
    fresh.load_state_dict(sd)
    fresh.eval(); blocks[0].eval()
    with torch.no_grad():
        assert torch.equal(fresh(x.cuda()), blocks[0](x.cuda()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_shared_expert_on_a_second_stream_changes_nothing(gpu, dtype):
    """``ep_overlap`` runs the shared expert on a second stream beside the routed path where the launches leave CUs idle
    (every shape of this size): outputs and every gradient must equal, bit for bit, the run on one stream, for two
    steps in a row (the second reuses memory the first released on either stream) and with work queued on the launch
    stream right behind the layer."""
    cfg = make_config(hidden=256, inter=128, num_experts=4, top_k=2, n_shared=1)
    moe = build(cfg, seed=3, std=0.05, dtype=dtype)
    assert moe._launches_leave_cus_idle(200) and not moe._launches_leave_cus_idle(10 ** 6)
    g = torch.Generator().manual_seed(4)
    xs = [torch.randn(2, 100, 256, generator=g).to(dtype) for _ in range(2)]
    ups = [torch.randn(2, 100, 256, generator=g).to(dtype) for _ in range(2)]

    def run(overlap):
        moe.ep_overlap = overlap
        results = []
        for x, up in zip(xs, ups):
            moe.zero_grad(set_to_none=True)
            xin = x.cuda().requires_grad_(True)
            out = moe(xin)
            tail = out * 2.0 + 1.0                      # consumer queued on the launch stream right behind the layer
            out.backward(up.cuda())
            results.append([tail.detach().clone(), xin.grad.clone()] + [p.grad.clone() for p in moe.parameters()])
        torch.cuda.synchronize()
        return results

    serial, overlapped = run(False), run(True)
    for step_s, step_o in zip(serial, overlapped):
        assert len(step_s) == len(step_o)
        for a, b in zip(step_s, step_o):
            assert torch.equal(a, b)


@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("n_shared", [0, 1])
def test_fused_gate_gradient_equals_the_gate_as_a_plain_linear(gpu, dtype, rtol, n_shared):
    """The token gradient written by one kernel (expert path + router path) against the same layer with its gate run as a
    plain ``nn.Linear`` node (a forward hook on the gate switches the fused node off): same output and expert
    gradients bit for bit -- the forward is the same launches -- and d x and d gate.weight within the dtype's bar; with a shared expert
    the tokens have a third reader."""
    cfg = make_config(hidden=256, inter=128, num_experts=8, top_k=2, n_shared=n_shared)
    moe = build(cfg, seed=11, std=0.05, dtype=dtype)
    moe.ep_overlap = False
    g = torch.Generator().manual_seed(12)
    x = torch.randn(3, 50, 256, generator=g).to(dtype)
    up = torch.randn(3, 50, 256, generator=g).to(dtype)

    def run():
        moe.zero_grad(set_to_none=True)
        xin = x.cuda().requires_grad_(True)
        out = moe(xin)
        out.backward(up.cuda())
        return out.detach().clone(), xin.grad.clone(), {n: p.grad.clone() for n, p in moe.named_parameters()}

    import picotron_amd._ops as _ops
    calls = []
    real = _ops.gate_tap
    _ops.gate_tap = lambda *a: (calls.append(1), real(*a))[1]
    try:
        out_f, dx_f, grads_f = run()
        assert calls == [1]
        handle = moe.gate.register_forward_hook(lambda m, i, o: None)
        out_p, dx_p, grads_p = run()
        handle.remove()
        assert calls == [1]
    finally:
        _ops.gate_tap = real
    assert torch.equal(out_f, out_p)
    for name in grads_f:
        if name == "gate.weight":                 # d_logits.T @ x as a GEMM of the library's choosing on either side
            assert_close(grads_f[name], grads_p[name], rtol, name)
        else:
            assert torch.equal(grads_f[name], grads_p[name]), name
    assert_close(dx_f, dx_p, rtol, "d x")
