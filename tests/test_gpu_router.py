"""GPU parity of the router kernels (softmax top-k, gate weights, aux loss, loss-free bias, backward)
against the CPU oracle: indices bit-exact on tie-free rows, equal scores on tie rows, fp32 values 1e-5."""

import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

RTOL_F32 = 1e-5


def _route_gpu(logits, k, bias=None, norm=True, **kw):
    from picotron_amd import _ops

    b = bias.cuda().float() if bias is not None else None
    idx, w, aux = _ops.route(logits.cuda(), b, k, norm, **kw)
    return idx.cpu(), w.cpu(), aux.cpu(), (b.cpu() if b is not None else None)


@pytest.mark.parametrize("T,E,k", [(512, 8, 2), (1000, 64, 6), (37, 4, 1), (129, 3, 3), (300, 16, 4), (64, 160, 8), (50, 1024, 16), (0, 8, 2)])
@pytest.mark.parametrize("use_bias", [False, True])
@pytest.mark.parametrize("norm", [True, False])
def test_route_fp32_matches_oracle(gpu, T, E, k, use_bias, norm):
    g = torch.Generator().manual_seed(T * 1000 + E)
    logits = torch.randn(T, E, generator=g) * 2
    bias = 0.02 * torch.randn(E, generator=g) if use_bias else None
    idx, w, _, _ = _route_gpu(logits, k, bias, norm)
    ridx, rw, rp = O.softmax_topk_route(logits, k, bias, norm)
    assert idx.dtype == torch.int64 and idx.shape == (T, k)
    ties = O.tie_rows(logits, k, bias)
    assert not ties.any()
    assert torch.equal(idx, ridx)
    assert torch.allclose(w, rw, rtol=RTOL_F32, atol=1e-8)


def test_route_bf16_logits_with_ties(gpu):
    """bf16 router logits at the Mixtral shape tie on ~0.4% of rows: indices must match on tie-free rows,
    and on tie rows the selected scores must be equal (torch.topk's own tie order is unspecified)."""
    g = torch.Generator().manual_seed(0)
    T, H, E, k = 8192, 4096, 8, 2
    x = torch.randn(T, H, generator=g).bfloat16()
    wr = (0.02 * torch.randn(E, H, generator=g)).bfloat16()
    logits = torch.nn.functional.linear(x, wr)
    idx, w, _, _ = _route_gpu(logits, k)
    ridx, rw, rp = O.softmax_topk_route(logits, k)
    ties = O.tie_rows(logits, k)
    assert int(ties.sum()) > 0                      # the case exists in this data
    assert torch.equal(idx, ridx)                   # same canonical rule -> equal everywhere, ties included
    tk = torch.topk(rp, k, dim=-1).indices          # library top-k: equal on tie-free rows, equal scores on tie rows
    assert torch.equal(idx[~ties], tk[~ties])
    assert torch.equal(rp[ties].gather(-1, idx[ties]), rp[ties].gather(-1, tk[ties]))
    assert w.dtype == torch.bfloat16
    assert torch.allclose(w.float(), rw.float(), rtol=1e-2)
    assert (w.view(torch.int16) != rw.view(torch.int16)).float().mean() < 0.02   # bf16 rounding of near-identical fp32


def test_route_explicit_ties(gpu):
    logits = torch.tensor([[1.0, 3.0, 3.0, 1.0], [0.0, 0.0, 0.0, 0.0], [2.0, 1.0, 2.0, 2.0], [5.0, 5.0, 1.0, 5.0]])
    idx, w, _, _ = _route_gpu(logits, 2)
    assert idx.tolist() == [[1, 2], [0, 1], [0, 2], [0, 1]]
    assert torch.allclose(w, torch.full((4, 2), 0.5))
    idx3, _, _, _ = _route_gpu(logits, 3)
    assert idx3.tolist() == [[1, 2, 0], [0, 1, 2], [0, 2, 3], [0, 1, 3]]


def test_bias_changes_picks_not_weights(gpu):
    logits = torch.tensor([[1.0, 3.0, 3.0, 1.0]])
    bias = torch.tensor([10.0, 0.0, 0.0, 0.0])
    idx, w, _, _ = _route_gpu(logits, 2, bias, norm=False)
    p = torch.softmax(logits, -1)
    assert idx.tolist() == [[0, 1]]
    assert torch.allclose(w[0], p[0, [0, 1]], rtol=RTOL_F32)


@pytest.mark.parametrize("T,E,k", [(512, 8, 2), (4096, 64, 6), (300, 160, 4)])
def test_balance_aux_and_bias_step(gpu, T, E, k):
    g = torch.Generator().manual_seed(E)
    logits = torch.randn(T, E, generator=g)
    bias0 = 0.01 * torch.randn(E, generator=g)
    idx, w, aux, bias1 = _route_gpu(logits, k, bias0, True, balance=True, aux_coef=0.01, bias_rate=0.001)
    ridx, _, rp = O.softmax_topk_route(logits, k, bias0, True)
    raux, rbias, rcounts = O.balance(rp, ridx, E, k, 0.01, 0.001, bias0)
    assert torch.equal(idx, ridx)
    assert abs(aux.item() - raux.item()) <= RTOL_F32 * abs(raux.item())
    assert torch.allclose(bias1, rbias, rtol=0, atol=1e-9)
    # closed form: a uniform router with balanced picks gives aux == coef
    from picotron_amd import _ops

    ul = torch.zeros(E * 8, E)
    ul[torch.arange(E * 8), torch.arange(E * 8) % E] = 1e-3   # tiny preference -> balanced top-1
    _, _, aux_u = _ops.route(ul.cuda(), None, 1, True, True, 0.5, 0.0)
    assert abs(aux_u.item() - 0.5) < 1e-3


@pytest.mark.parametrize("E,k,norm", [(8, 2, True), (64, 6, True), (16, 1, True), (8, 3, False), (160, 4, True)])
def test_route_backward_matches_autograd(gpu, E, k, norm):
    from picotron_amd import _ops

    T = 257
    g = torch.Generator().manual_seed(E + k)
    logits = torch.randn(T, E, generator=g)
    dw = torch.randn(T, k, generator=g)
    # oracle: autograd through softmax -> gather -> renorm, plus the aux term
    lr = logits.clone().requires_grad_(True)
    ridx, rw, rp = O.softmax_topk_route(lr, k, None, norm)
    raux, _, _ = O.balance(rp, ridx, E, k, 0.01, 0.0)
    ((rw * dw).sum() + 3.0 * raux).backward()
    lg = logits.cuda().requires_grad_(True)
    idx, w, aux = _ops.route(lg, None, k, norm, True, 0.01, 0.0)
    ((w * dw.cuda()).sum() + 3.0 * aux).backward()
    assert torch.equal(idx.cpu(), ridx)
    err = (lg.grad.cpu() - lr.grad).abs().max().item()
    assert err <= 1e-5 * lr.grad.abs().max().item() + 1e-9, err
    # without aux
    lg2 = logits.cuda().requires_grad_(True)
    _, w2, _ = _ops.route(lg2, None, k, norm)
    (w2 * dw.cuda()).sum().backward()
    lr2 = logits.clone().requires_grad_(True)
    _, rw2, _ = O.softmax_topk_route(lr2, k, None, norm)
    (rw2 * dw).sum().backward()
    assert (lg2.grad.cpu() - lr2.grad).abs().max().item() <= 1e-5 * lr2.grad.abs().max().item() + 1e-9


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,H", [(700, 8, 4096), (2100, 8, 264), (5, 3, 72), (1, 1, 8), (600, 16, 2048), (33, 9, 520), (0, 8, 64),
                                   (8192, 8, 2048)])
@pytest.mark.parametrize("with_addend", [True, False])
@pytest.mark.parametrize("with_weight_grad", [True, False])
def test_gate_bwd_is_the_linear_backward_plus_the_addend(gpu, dtype, T, E, H, with_addend, with_weight_grad):
    """d_x = addend + d_logits @ W against float64 arithmetic with the kernel's two roundings (product, then sum) and
    d_W = d_logits.T @ x against float64 rounded once: fp32 within 1e-5 of the largest element, bf16 within 1e-2 (one
    rounding step of either).  Token counts above and below the grid, more than four tokens per wavefront, widths that
    leave lanes without columns, 1..16 experts (the weight gradient is fused up to 8; above, None comes back)."""
    from picotron_amd import _ops

    g = torch.Generator().manual_seed(T * 31 + E * 7 + H)
    d_logits = torch.randn(T, E, generator=g).to(dtype)
    w = torch.randn(E, H, generator=g).to(dtype)
    x = torch.randn(T, H, generator=g).to(dtype)
    addend = (3 * torch.randn(T, H, generator=g)).to(dtype) if with_addend else None
    d_x, d_w = _ops.gate_bwd(d_logits.cuda(), w.cuda(), addend.cuda() if with_addend else None, x.cuda(), with_weight_grad)
    torch.cuda.synchronize()
    ref = (d_logits.double() @ w.double()).to(dtype).double()
    if with_addend:
        ref = (ref + addend.double()).to(dtype).double()
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    got = d_x.cpu().double()
    assert got.shape == (T, H) and torch.isfinite(got).all()
    if T:
        assert (got - ref).abs().max() <= tol * ref.abs().amax()
    assert (d_w is not None) == (with_weight_grad and E <= 8)
    if d_w is not None:
        ref_w = (d_logits.double().t() @ x.double()).to(dtype).double()
        got_w = d_w.cpu().double()
        assert got_w.shape == (E, H) and torch.isfinite(got_w).all()
        assert (got_w - ref_w).abs().max() <= tol * max(float(ref_w.abs().amax()), 1e-30)
        if T == 0:
            assert not got_w.any()


def test_gate_weight_gradient_has_one_fixed_summation_order(gpu):
    """Two launches on the same inputs give the same bits (block sums are added in block order, no atomics)."""
    from picotron_amd import _ops

    g = torch.Generator(device="cuda").manual_seed(3)
    T, E, H = 5000, 8, 1024
    dl = torch.randn(T, E, generator=g, device="cuda").bfloat16()
    w = torch.randn(E, H, generator=g, device="cuda").bfloat16()
    x = torch.randn(T, H, generator=g, device="cuda").bfloat16()
    a = _ops.gate_bwd(dl, w, None, x, True)
    b = _ops.gate_bwd(dl, w, None, x, True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_gate_tap_gradients_equal_the_linear_beside_its_readers(gpu):
    """The autograd node that hands the tokens through gives the gradients of `linear(x, W)` with a second reader of x:
    d x and d W against float64 autograd of the same graph (fp32: 1e-5 of the largest element)."""
    from picotron_amd import _ops

    g = torch.Generator().manual_seed(5)
    T, E, H = 300, 8, 512
    x = torch.randn(T, H, generator=g)
    w = 0.1 * torch.randn(E, H, generator=g)
    m = torch.randn(T, H, generator=g)
    c = torch.randn(T, E, generator=g)
    xd, wd = x.cuda().requires_grad_(), w.cuda().requires_grad_()
    assert _ops.gate_dgrad_supported(xd, wd)
    logits, tap = _ops.gate_tap(xd, wd)
    ((logits * c.cuda()).sum() + (tap * m.cuda()).sum()).backward()
    x64, w64 = x.double().requires_grad_(), w.double().requires_grad_()
    ((torch.nn.functional.linear(x64, w64) * c.double()).sum() + (x64 * m.double()).sum()).backward()
    for got, ref in ((xd.grad, x64.grad), (wd.grad, w64.grad)):
        assert (got.cpu().double() - ref).abs().max() <= 1e-5 * ref.abs().max()
    # only the logits read: the gradient is the plain product; only the tokens read: it is handed through
    xd.grad = None
    logits, tap = _ops.gate_tap(xd, wd)
    (logits * c.cuda()).sum().backward()
    assert (xd.grad.cpu().double() - c.double() @ w.double()).abs().max() <= 1e-5 * 10
    xd.grad = None
    logits, tap = _ops.gate_tap(xd, wd)
    (tap * m.cuda()).sum().backward()
    assert torch.equal(xd.grad.cpu(), m)
