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


def test_explicit_backward_is_autograd_in_exact_arithmetic():
    """The reference's explicit dgrad / wgrad formulas (megakernel.py:332-357) and autograd over its torch FFN (:321-329)
    are the same mathematics: equal to 1e-12 in float64 on ragged counts with an empty expert; in bf16 they differ
    only by where they round; through the layer (``ffn_backward="explicit"``) every gradient agrees as well."""
    g = torch.Generator().manual_seed(3)
    E, H, I = 4, 10, 14
    counts = torch.tensor([5, 0, 9, 1])
    x = torch.randn(15, H, generator=g, dtype=torch.float64)
    gw, uw, dw = (torch.randn(E, I, H, generator=g, dtype=torch.float64), torch.randn(E, I, H, generator=g, dtype=torch.float64),
                  torch.randn(E, H, I, generator=g, dtype=torch.float64))
    dy = torch.randn(15, H, generator=g, dtype=torch.float64)
    for a, b in zip(O.expert_ffn_backward_explicit(x, counts, gw, uw, dw, dy), O.expert_ffn_backward(x, counts, gw, uw, dw, dy)):
        assert a.shape == b.shape and (a - b).abs().max() < 1e-12
    lo = [t.bfloat16() for t in (x, gw * 0.2, uw * 0.2, dw * 0.2, dy)]
    for a, b in zip(O.expert_ffn_backward_explicit(lo[0], counts, *lo[1:]), O.expert_ffn_backward(lo[0], counts, *lo[1:])):
        assert (a.float() - b.float()).abs().max() <= 2e-2 * b.float().abs().max()
    w = _weights(4, 16, 24, seed=2, shared=1, std=0.3)
    xs = torch.randn(20, 16, generator=g)
    grads = []
    for mode in ("autograd", "explicit"):
        for t in w.tensors():
            t.requires_grad_(True)
            t.grad = None
        xr = xs.clone().requires_grad_(True)
        O.moe_forward(xr, w, 2, ffn_backward=mode)[0].pow(2).sum().backward()
        grads.append([xr.grad] + [t.grad.clone() for t in w.tensors()])
    for a, b in zip(*grads):
        assert torch.allclose(a, b, atol=1e-5, rtol=1e-4)


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


def test_latent_layer_is_the_plain_layer_between_two_matmuls():
    """LatentMoE (expert_parallel.py:59-69, 226-228, 250-252): the routed path of a latent layer is the plain layer run
    on ``tokens @ W_down^T`` with the routing decided on the full-width tokens, followed by ``@ W_up^T``; the shared
    expert sees the full-width tokens.  Checked with two library matmuls around the already pinned plain layer, and
    against a per-token loop that never calls moe_forward."""
    T, H, L, I, E, k = 24, 32, 12, 20, 4, 2
    g = torch.Generator().manual_seed(11)
    r = lambda *s: 0.3 * torch.randn(*s, generator=g)
    w = O.LayerWeights(r(E, H), r(E, I, L), r(E, I, L), r(E, L, I), shared=(r(2 * I, H), r(2 * I, H), r(H, 2 * I)),
                       latent=(r(L, H), r(H, L)))
    x = torch.randn(T, H, generator=g)
    out, info = O.moe_forward(x, w, k)
    assert out.shape == (T, H) and info["y_routed"].shape == (T * k, L)
    plain = O.LayerWeights(w.router_w, w.gate_w, w.up_w, w.down_w)
    inner, _ = O.moe_forward(x @ w.latent[0].T, plain, k, routing=(info["topk_idx"], info["topk_w"]))
    want = inner @ w.latent[1].T + O.mlp(x, *w.shared)
    assert torch.allclose(out, want, atol=1e-5)
    # per-token loop: token -> latent row -> each picked expert alone -> weighted sum -> up projection (+ shared)
    p = torch.softmax(x @ w.router_w.T, -1)
    for t in range(0, T, 5):
        picks = sorted(range(E), key=lambda e: (-float(p[t, e]), e))[:k]
        pw = torch.stack([p[t, e] for e in picks])
        pw = pw / pw.sum()
        z = w.latent[0] @ x[t]
        acc = sum(pw[j] * (w.down_w[e] @ (F.silu(w.gate_w[e] @ z) * (w.up_w[e] @ z))) for j, e in enumerate(picks))
        ref = w.latent[1] @ acc + O.mlp(x[t : t + 1], *w.shared)[0]
        assert torch.allclose(out[t], ref, atol=1e-5)
    # a wrong operand order or a swapped projection changes the shape or the value
    assert not torch.allclose(out, inner @ w.latent[1].T, atol=1e-3)
    # the capped paths work in the latent width too
    cap, _ = O.moe_forward(x, w, k, capacity_factor=1.0, capacity_dropless=True, max_rounds=64)
    assert torch.allclose(cap, out, atol=1e-5)
    # and gradients reach both projections
    for t_ in w.latent:
        t_.requires_grad_(True)
    O.moe_forward(x, w, k)[0].sum().backward()
    assert all(t_.grad is not None and t_.grad.abs().sum() > 0 for t_ in w.latent)


def _zipf_routing(T, E, k, seed):
    """Distinct picks per token, expert e drawn with weight 1/(e+1)^1.5: the first experts overflow several times."""
    g = torch.Generator().manual_seed(seed)
    pr = 1.0 / torch.arange(1, E + 1, dtype=torch.float32) ** 1.5
    idx = torch.multinomial(pr.expand(T, E), k, replacement=False, generator=g)
    wt = torch.softmax(torch.rand(T, k, generator=g), -1)
    return idx, wt


def test_dropless_rounds_partition_the_rows_and_max_rounds_cuts_them():
    """capacity_moe.py:96-120.  Round r keeps the rows whose rank inside their expert lies in [r*C, (r+1)*C), so
    (a) with enough rounds every row is processed exactly once and the result is the uncapped layer's;
    (b) with max_rounds = R smaller than needed exactly the rows of rank >= R*C are lost, i.e. the kept set is the
        drop mode's at capacity R*C -- two statements the rounds' loop cannot satisfy with an off-by-one in the
        window, a wrong round count or a missing clamp to max_rounds."""
    T, H, I, E, k = 96, 16, 24, 8, 2
    w = _weights(E, H, I, seed=4, shared=1, std=0.3)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(8))
    routing = _zipf_routing(T, E, k, seed=9)
    base, _ = O.moe_forward(x, w, k, routing=routing)
    full, info = O.moe_forward(x, w, k, routing=routing, capacity_factor=0.25, capacity_dropless=True, max_rounds=64)
    C = info["capacity"]
    need = -(-int(info["counts"].max()) // C)
    assert C == 6 and need >= 4 and info["rounds"] == need and bool(info["keep"].all())
    assert torch.allclose(full, base, atol=1e-5)
    for R in (1, 2, need - 1):
        cut, ci = O.moe_forward(x, w, k, routing=routing, capacity_factor=0.25, capacity_dropless=True, max_rounds=R)
        assert ci["rounds"] == R
        want_keep = ci["within"] < R * C
        assert torch.equal(ci["keep"], want_keep) and not bool(want_keep.all())
        # the same rows kept through the routing instead of the capacity: weights of the lost picks set to zero
        wt0 = torch.where(want_keep.view(T, k), routing[1], torch.zeros_like(routing[1]))
        same, _ = O.moe_forward(x, w, k, routing=(routing[0], wt0))
        assert torch.allclose(cut, same, atol=1e-5)
        assert (cut - base).abs().max() > 1e-3
