"""Pins the expert-FFN, backward and whole-layer parts of the CPU oracle.

Checks: a per-token brute force, finite differences, autograd, the dropless-capacity == naive
identity the reference tests (tests/test_capacity_moe.py:41-72), and the ragged / empty-expert case
of the reference's own kernel test (tests/test_megakernel.py:35-61).
"""

import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


def _weights(E, H, I, seed=0, shared=0, dtype=torch.float32, std=0.02, router_bias=False):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: (std * torch.randn(*s, generator=g)).to(dtype)
    w = O.LayerWeights(r(E, H), r(E, I, H), r(E, I, H), r(E, H, I))
    if shared:
        w.shared = (r(shared * I, H), r(shared * I, H), r(H, shared * I))
    if router_bias:
        w.router_b = r(E)
    return w


def test_expert_ffn_ragged_matches_row_by_row():
    torch.manual_seed(0)
    E, H, I = 4, 48, 96
    counts = torch.tensor([5, 0, 130, 17])
    N = int(counts.sum())
    x = torch.randn(N, H)
    gw, uw, dw = (torch.randn(E, I, H) * 0.1, torch.randn(E, I, H) * 0.1, torch.randn(E, H, I) * 0.1)
    y = O.expert_ffn(x, counts, gw, uw, dw)
    owner = torch.repeat_interleave(torch.arange(E), counts)
    for r in range(0, N, 7):
        e = int(owner[r])
        g = gw[e] @ x[r]
        want = dw[e] @ ((g * torch.sigmoid(g)) * (uw[e] @ x[r]))
        assert torch.allclose(y[r], want, atol=1e-5, rtol=1e-5)
    rw = torch.rand(N)
    assert torch.allclose(O.expert_ffn(x, counts, gw, uw, dw, rw), y * rw[:, None])
    assert O.expert_ffn(x[:0], torch.zeros(E, dtype=torch.int64), gw, uw, dw).shape == (0, H)


def test_silu_mul_bwd_finite_differences_and_autograd():
    torch.manual_seed(1)
    N, I = 6, 10
    z = torch.randn(N, 2 * I, dtype=torch.float64, requires_grad=True)
    da = torch.randn(N, I, dtype=torch.float64)
    a = F.silu(z[:, :I]) * z[:, I:]
    (want,) = torch.autograd.grad(a, z, da)
    got = O.silu_and_mul_bwd(z.detach().float(), da.float())
    assert torch.allclose(got.double(), want, atol=1e-5)
    eps = 1e-6
    zz = z.detach().clone()
    for (r, c) in [(0, 0), (2, 3), (5, I + 4), (3, 2 * I - 1)]:
        zp, zm = zz.clone(), zz.clone()
        zp[r, c] += eps
        zm[r, c] -= eps
        f = lambda t: ((F.silu(t[:, :I]) * t[:, I:]) * da).sum()
        fd = (f(zp) - f(zm)) / (2 * eps)
        assert abs(fd.item() - got[r, c].item()) < 1e-4


def test_expert_ffn_backward_matches_manual_chain():
    torch.manual_seed(2)
    E, H, I = 3, 8, 12
    counts = torch.tensor([4, 0, 5])
    x = torch.randn(9, H, dtype=torch.float64)
    gw, uw, dw = torch.randn(E, I, H, dtype=torch.float64), torch.randn(E, I, H, dtype=torch.float64), torch.randn(E, H, I, dtype=torch.float64)
    dy = torch.randn(9, H, dtype=torch.float64)
    dx, dg, du, dd = O.expert_ffn_backward(x, counts, gw, uw, dw, dy)
    # manual chain rule for expert 2 (rows 4..9): the explicit dgrad / wgrad contract of the kernels
    xs, dys = x[4:], dy[4:]
    g, u = xs @ gw[2].T, xs @ uw[2].T
    a = F.silu(g) * u
    da = dys @ dw[2]
    d13 = O.silu_and_mul_bwd(torch.cat([g, u], 1), da)
    assert torch.allclose(dd[2], dys.T @ a)
    assert torch.allclose(dg[2], d13[:, :I].T @ xs)
    assert torch.allclose(du[2], d13[:, I:].T @ xs)
    assert torch.allclose(dx[4:], d13 @ torch.cat([gw[2], uw[2]], 0))
    assert torch.all(dg[1] == 0) and torch.all(dd[1] == 0)     # empty expert: zero weight grads


def test_layer_matches_per_token_brute_force():
    for (T, H, I, E, k, shared) in [(8, 16, 32, 4, 2, 1), (37, 32, 24, 8, 3, 0), (16, 16, 32, 4, 1, 2)]:
        w = _weights(E, H, I, seed=T, shared=shared, std=0.3)
        x = torch.randn(T, H, generator=torch.Generator().manual_seed(5))
        out, info = O.moe_forward(x, w, k)
        assert torch.allclose(out, O.moe_brute_force(x, w, k), atol=1e-5)
        assert int(info["counts"].sum()) == T * k


def test_dropless_capacity_equals_naive_and_capped_drops():
    T, H, I, E, k = 16, 16, 32, 4, 2
    w = _weights(E, H, I, seed=0, shared=1, std=0.3)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(123))
    base, _ = O.moe_forward(x, w, k)
    cap, info = O.moe_forward(x, w, k, capacity_factor=1.0, capacity_dropless=True, max_rounds=64)
    assert (base - cap).abs().max().item() < 1e-5
    assert bool(info["keep"].all())
    capped, info2 = O.moe_forward(x, w, k, capacity_factor=0.5, capacity_dropless=False)
    assert torch.isfinite(capped).all() and (base - capped).abs().max().item() > 0
    C = info2["capacity"]
    assert C == 4 and int(info2["keep"].sum()) == int(torch.clamp(info2["counts"], max=C).sum())
    # a dropped (token, expert) pair contributes exactly nothing: removing it from the routing changes nothing
    idx, wt = info2["topk_idx"], info2["topk_w"]
    keep = info2["keep"].view(T, k)
    wt2 = torch.where(keep, wt, torch.zeros_like(wt))
    again, _ = O.moe_forward(x, w, k, routing=(idx, wt2))
    assert torch.allclose(again, capped, atol=1e-6)


def test_fp8_dispatch_layer_semantics():
    T, H, I, E, k = 32, 64, 48, 4, 2
    w = _weights(E, H, I, seed=3, std=0.2, dtype=torch.bfloat16)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(7)).bfloat16().requires_grad_(True)
    plain, _ = O.moe_forward(x, w, k)
    fp8, info = O.moe_forward(x, w, k, fp8_dispatch=True)
    rel = ((fp8.float() - plain.float()).norm() / plain.float().norm()).item()
    assert 0 < rel < 0.05                          # the bound the reference's own FP8 test uses
    # routed row r = t*k+j carries token t's codes: one quantisation per token is enough
    cq, cs = O.quant_fp8(x.detach())
    assert torch.equal(info["fp8_codes"], cq.repeat_interleave(k, 0)) and torch.equal(info["fp8_scale"], cs.repeat_interleave(k))
    fp8.float().sum().backward()                   # straight-through: gradient reaches x
    assert x.grad is not None and torch.isfinite(x.grad).all()
