"""Pins the router / balance part of the CPU oracle by brute force, closed forms and torch.topk."""

import math

import torch

from oracle import moe_oracle as O


def _brute_route(logits, k, bias, norm):
    T, E = logits.shape
    idx, w = [], []
    for t in range(T):
        row = [float(v) for v in logits[t].float()]
        m = max(row)
        ex = torch.tensor([math.exp(v - m) for v in row], dtype=torch.float64)
        p = (ex / ex.sum()).float()
        s = p + bias if bias is not None else p
        picks = sorted(range(E), key=lambda e: (-float(s[e]), e))[:k]
        pw = torch.stack([p[e] for e in picks])
        if norm and k > 1:
            pw = pw / pw.sum()
        idx.append(picks)
        w.append(pw)
    return torch.tensor(idx), torch.stack(w)


def test_route_matches_brute_force_and_topk():
    g = torch.Generator().manual_seed(0)
    for (T, E, k) in [(64, 8, 2), (33, 64, 6), (5, 4, 1), (7, 3, 3)]:
        logits = torch.randn(T, E, generator=g)
        for bias in (None, 0.05 * torch.randn(E, generator=g)):
            for norm in (True, False):
                idx, w, p = O.softmax_topk_route(logits, k, bias, norm)
                bidx, bw = _brute_route(logits, k, bias, norm)
                assert torch.equal(idx, bidx)
                assert torch.allclose(w, bw, rtol=1e-6, atol=1e-8)
                sel = p + bias if bias is not None else p
                assert torch.equal(idx, torch.topk(sel, k, dim=-1).indices)  # fp32 randn rows are tie-free
                assert not O.tie_rows(logits, k, bias).any()
                if norm and k > 1:
                    assert torch.allclose(w.sum(-1), torch.ones(T), atol=1e-6)
                # picks are distinct, scores non-increasing
                assert all(len(set(r.tolist())) == k for r in idx)
                assert torch.all(sel.gather(-1, idx).diff(dim=-1) <= 0)


def test_route_tie_rule_and_bf16_weights():
    logits = torch.tensor([[1.0, 3.0, 3.0, 1.0], [0.0, 0.0, 0.0, 0.0], [2.0, 1.0, 2.0, 2.0]])
    idx, w, _ = O.softmax_topk_route(logits, 2)
    assert idx.tolist() == [[1, 2], [0, 1], [0, 2]]      # equal scores -> lower expert id first
    assert O.tie_rows(logits, 2).tolist() == [True, True, True]
    assert torch.allclose(w, torch.full((3, 2), 0.5))
    _, wb, _ = O.softmax_topk_route(logits.bfloat16(), 2)
    assert wb.dtype == torch.bfloat16
    # gate weights come from the UNBIASED probabilities even when the bias changes the picks
    bias = torch.tensor([10.0, 0.0, 0.0, 0.0])
    idx2, w2, p2 = O.softmax_topk_route(logits[:1], 2, bias, norm_topk_prob=False)
    assert idx2.tolist() == [[0, 1]]
    assert torch.equal(w2[0], p2[0, [0, 1]])


def test_aux_loss_closed_forms():
    T, E, k = 64, 8, 2
    probs = torch.full((T, E), 1.0 / E)
    idx = torch.stack([torch.arange(T) % E, (torch.arange(T) + 1) % E], dim=1)  # perfectly balanced picks
    aux, nb, counts = O.balance(probs, idx, E, k, aux_coef=0.01, bias_rate=0.0)
    assert counts.tolist() == [T * k / E] * E
    assert abs(aux.item() - 0.01) < 1e-9          # balanced router: sum_e f_e P_e = E * 1 * 1/E = 1
    assert nb is None
    # everything on expert 0 with P concentrated there: f_0 = E/k * ... closed form
    idx0 = torch.zeros(T, 1, dtype=torch.int64)
    p0 = torch.zeros(T, E)
    p0[:, 0] = 1.0
    aux0, _, _ = O.balance(p0, idx0, E, 1, aux_coef=0.5, bias_rate=0.0)
    assert abs(aux0.item() - 0.5 * E) < 1e-6
    # gradient flows only through the mean probability: d aux / d probs[t,e] = coef * f_e / T
    pr = torch.softmax(torch.randn(T, E, generator=torch.Generator().manual_seed(1)), -1).requires_grad_(True)
    ti = torch.topk(pr, k).indices
    a, _, c = O.balance(pr, ti, E, k, aux_coef=0.3, bias_rate=0.0)
    a.backward()
    want = 0.3 * c * (E / (k * T)) / T
    assert torch.allclose(pr.grad, want.expand(T, E), atol=1e-7)
    assert O.balance(pr.detach(), ti, E, k, 0.0, 0.0)[0] is None


def test_bias_step_sign_rule():
    E = 4
    probs = torch.full((6, E), 0.25)
    idx = torch.tensor([[0], [0], [0], [1], [1], [2]])
    _, nb, counts = O.balance(probs, idx, E, 1, 0.0, bias_rate=0.1, expert_bias=torch.zeros(E))
    assert counts.tolist() == [3, 2, 1, 0]                       # mean 1.5
    assert torch.allclose(nb, torch.tensor([-0.1, -0.1, 0.1, 0.1]))
    # most loaded ends below least loaded (the monotonic property the reference tests, test_load_balance.py:76-79)
    assert nb[counts.argmax()] < nb[counts.argmin()]
    idx_eq = torch.tensor([[0], [1], [2], [3]])
    _, nb2, _ = O.balance(probs[:4], idx_eq, E, 1, 0.0, 0.1, torch.ones(E))
    assert torch.equal(nb2, torch.ones(E))                       # sign(0) = 0
