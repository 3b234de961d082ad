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
