"""The headline configuration at full size, forward AND backward, against the CPU oracle.

Mixtral-shape MoE layer with FP8 dispatch: 8192 tokens, hidden 4096, SwiGLU FFN 14336, 8 experts, top-2, bf16,
E4M3 per-token-scaled rows into the expert FFN, aux load-balance loss coefficient 0.01, upstream gradient ~ N(0,1),
loss = <out, g> + aux.  The oracle runs the reference's naive torch path (expert_parallel.py:168-224, 271-341;
ep_communications.py:63-68, :100; megakernel.py:308-329 through autograd) on the host cores with the same weights in
the same bf16 -- about 17 TFLOP, some tens of seconds on 16 cores.

Compared: routing and FP8 codes bit-exact; the output, d x, d router weight and each expert's three weight
gradients within 1e-2 (bf16 GEMM outputs and gradients).  The reference differentiates the expert FFN in two ways:
op by op through autograd where there is no GPU (megakernel.py:321-329) and with explicit dgrad / wgrad formulas on a
GPU (:332-357).  They are the same mathematics and round to bf16 in different places (autograd: da*u, dg, du and the
two halves of dx one by one; explicit: the SwiGLU backward in fp32 rounded once, dx as one contraction over 2I).
The kernels round where the explicit form does.  Against that form every tensor must be within 1e-2 both norm-wise
and in its largest element difference; against the autograd form norm-wise (two bf16 results that each round a
value once can sit two bf16 steps apart, and two steps of an element in the binade of the largest one are up to
1.6e-2 of it).
"""

import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _rel_l2(got, want):
    return ((got - want).norm() / want.norm()).item()


def test_mixtral_fp8_dispatch_forward_backward_full_size(gpu):
    import bench
    from picotron_amd.expert_parallel.ep_communications import _per_token_quant_fp8
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss

    wl = bench.WORKLOADS["c5"]
    T, H, I, E, k = wl["T"], wl["H"], wl["I"], wl["E"], wl["k"]
    moe = bench.build_layer(wl, gpu, torch.bfloat16)
    assert moe.training and moe.ep_fp8_dispatch and moe.router_aux_loss_coef == 0.01
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(T, H, generator=gen).bfloat16()
    upstream = torch.randn(T, H, generator=gen).bfloat16()

    xg = x.to(gpu).requires_grad_(True)
    out = moe(xg.view(1, T, H))
    aux = collect_aux_loss(moe)
    torch.autograd.backward([out, aux], [upstream.to(gpu).view(1, T, H), torch.ones_like(aux)])
    with torch.no_grad():
        logits_gpu = moe.gate(xg.detach()).cpu()
        idx_gpu, _ = moe._route(xg.detach())       # a second pass of the router in training mode only re-stashes the aux
        moe.aux_loss = None
        codes_gpu, scale_gpu = _per_token_quant_fp8(xg.detach())
    got = {"out": out.detach().view(T, H).cpu().float(), "d x": xg.grad.cpu().float(), "aux": float(aux),
           "d router": moe.gate.weight.grad.cpu().float()}
    for name, proj in (("gate", "gate_proj"), ("up", "up_proj"), ("down", "down_proj")):
        got["d " + name] = torch.stack([getattr(e, proj).weight.grad for e in moe.local_experts]).cpu()
    c = lambda t: t.detach().cpu().clone()
    w16 = O.LayerWeights(c(moe.gate.weight), c(moe._stacks[0]), c(moe._stacks[1]), c(moe._stacks[2]))
    del moe, out, xg
    torch.cuda.empty_cache()

    torch.set_num_threads(16)

    def oracle_run(ffn_backward, wide=torch.bfloat16):
        w = O.LayerWeights(*(t.detach().to(wide) for t in w16.tensors()))
        for t in w.tensors():
            t.requires_grad_(True)
        xr = x.detach().to(wide).clone().requires_grad_(True)
        own = torch.nn.functional.linear(xr, w.router_w)
        # the GPU's logit values (its GEMM rounds a bf16 logit differently from the CPU's now and then, which flips
        # near-tie picks), the oracle's own gate Linear for the gradient: a + (b - a) is exact in fp32 here
        logits = (own.float() + (logits_gpu.float() - own.float()).detach()).to(own.dtype)
        ref, info = O.moe_forward(xr, w, k, logits=logits, fp8_dispatch=True, aux_coef=0.01, training=True,
                                  ffn_backward=ffn_backward, dispatch_dtype=torch.bfloat16)
        torch.autograd.backward([ref, info["aux"]], [upstream.to(wide), torch.ones(())])
        want = {"out": ref.detach().float(), "d x": xr.grad.float(), "d router": w.router_w.grad.float()}
        for name, t in (("gate", w.gate_w), ("up", w.up_w), ("down", w.down_w)):
            want["d " + name] = t.grad.clone()
        return want, info

    def compare(want, label):
        report = []
        for name in ("out", "d x", "d router"):
            err = (got[name] - want[name]).abs().max().item() / want[name].abs().max().item()
            report.append((name, err, _rel_l2(got[name], want[name])))
        for name in ("gate", "up", "down"):
            for e in range(E):
                g, r = got["d " + name][e].float(), want["d " + name][e].float()
                report.append((f"d {name}[{e}]", (g - r).abs().max().item() / r.abs().max().item(), _rel_l2(g, r)))
        for name, err, rel in report:
            print(f"[{label}] {name:12s} max|err|/max|ref| = {err:.2e}   rel-L2 = {rel:.2e}", flush=True)
        return report

    want, info = oracle_run("explicit")
    # integer / byte parts: bit-exact
    assert torch.equal(idx_gpu.cpu(), info["topk_idx"])
    assert torch.equal(codes_gpu.view(torch.uint8).cpu().repeat_interleave(k, 0), info["fp8_codes"])
    assert torch.equal(scale_gpu.cpu().repeat_interleave(k), info["fp8_scale"])
    assert abs(got["aux"] - float(info["aux"])) <= 1e-4 * abs(float(info["aux"]))
    bad = [(n, e, r) for n, e, r in compare(want, "explicit") if e > 1.6e-2 or r > 1e-2]
    assert not bad, bad
    del want
    want, _ = oracle_run("autograd")
    bad = [(n, e, r) for n, e, r in compare(want, "autograd") if r > 1e-2 or e > 1.6e-2]
    assert not bad, bad
    del want
    want, _ = oracle_run("autograd", torch.float32)
    bad = [(n, e, r) for n, e, r in compare(want, "fp32") if r > 1e-2 or e > 1e-2]
    assert not bad, bad
