"""GPU parity of the decoder that calls the MoE layer (picotron_amd.model.Llama) against the CPU oracle
(oracle/llama_oracle.py), with the reference's parameter names (picotron/model.py:363-402) and the training step of
tests/bench_ep_train_step.py:54-60 (cross entropy + the layers' aux losses, AdamW)."""

import types

import pytest
import torch
import torch.nn.functional as F

from oracle import llama_oracle as L

pytestmark = pytest.mark.gpu


def make_config(**kw):
    base = dict(vocab_size=211, hidden_size=64, intermediate_size=96, num_attention_heads=4, num_key_value_heads=2,
                num_hidden_layers=2, max_position_embeddings=64, rms_norm_eps=1e-5, rope_theta=10000.0,
                num_experts=4, num_experts_per_tok=2, num_shared_experts=1, norm_topk_prob=True)
    base.update(kw)
    return types.SimpleNamespace(**base)


def build(cfg, seed, dtype, std=0.08):
    from picotron_amd.model import Llama

    torch.manual_seed(seed)
    model = Llama(cfg)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("layernorm.weight") or name == "final_norm.weight":
                p.copy_(1 + 0.1 * torch.randn(p.shape, generator=g))
            elif name == "embedding.weight":
                p.copy_(torch.randn(p.shape, generator=g))
            else:
                p.copy_(std * torch.randn(p.shape, generator=g))
    return model.to(dtype).cuda()


def cpu_state(model, grad=False):
    sd = {k: v.detach().cpu().clone() for k, v in model.state_dict().items()}
    if grad:
        for k, v in sd.items():
            if v.is_floating_point() and not k.endswith("expert_bias"):
                v.requires_grad_(True)
    return sd


def batch(cfg, B, S, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg.vocab_size, (B, S), generator=g), torch.randint(0, cfg.vocab_size, (B, S), generator=g)


@pytest.mark.parametrize("variant", ["moe", "parallel_block", "dense"])
def test_logits_match_oracle_fp32(gpu, variant):
    cfg = make_config(**{"moe": {}, "parallel_block": dict(parallel_block=True),
                         "dense": dict(num_experts=1, num_shared_experts=0)}[variant])
    model = build(cfg, seed=1, dtype=torch.float32).eval()
    ids, _ = batch(cfg, 2, 48, seed=2)
    with torch.no_grad():
        got = model(ids.cuda()).cpu()
    want, _ = L.llama_forward(cpu_state(model), cfg, ids)
    assert got.shape == (2, 48, cfg.vocab_size)
    assert torch.allclose(got, want, atol=2e-4, rtol=1e-4), (got - want).abs().max().item()


def test_state_dict_round_trip_with_reference_names(gpu):
    """A state_dict keyed like the reference's model loads strictly, and the loaded model computes the same logits."""
    cfg = make_config()
    a = build(cfg, seed=3, dtype=torch.float32).eval()
    b = build(cfg, seed=4, dtype=torch.float32).eval()
    keys = list(a.state_dict().keys())
    assert keys[0] == "embedding.weight" and keys[-2:] == ["final_proj.weight", "final_norm.weight"]
    assert "decoder_layers.1.mlp.local_experts.3.down_proj.weight" in keys and "decoder_layers.0.mlp.expert_bias" in keys
    assert not any("cos" in k or "sin" in k for k in keys)
    b.load_state_dict({k: v.cpu() for k, v in a.state_dict().items()}, strict=True)
    ids, _ = batch(cfg, 1, 32, seed=5)
    with torch.no_grad():
        assert torch.equal(a(ids.cuda()), b(ids.cuda()))


def test_training_steps_follow_the_oracle_fp32(gpu):
    """Three AdamW steps on cross entropy + aux loss: loss values and updated parameters track the CPU oracle's."""
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss

    cfg = make_config(router_aux_loss_coef=0.01)
    model = build(cfg, seed=6, dtype=torch.float32).train()
    sd = cpu_state(model, grad=True)
    leaves = [v for v in sd.values() if v.requires_grad]
    opt_gpu = torch.optim.AdamW(model.parameters(), lr=1e-3)
    opt_cpu = torch.optim.AdamW(leaves, lr=1e-3)
    ids, tgt = batch(cfg, 2, 40, seed=7)
    for step in range(3):
        opt_gpu.zero_grad(set_to_none=True)
        logits = model(ids.cuda())
        loss = F.cross_entropy(logits.view(-1, logits.size(-1)).float(), tgt.cuda().view(-1))
        aux = collect_aux_loss(model)
        assert aux is not None and collect_aux_loss(model) is None   # drained
        (loss + aux.float()).backward()
        opt_gpu.step()

        opt_cpu.zero_grad(set_to_none=True)
        ref = L.train_loss(sd, cfg, ids, tgt)
        ref.backward()
        if step == 0:
            grads = dict(model.named_parameters())
            for k, v in sd.items():
                if v.requires_grad:
                    g, r = grads[k].grad.cpu(), v.grad
                    assert torch.allclose(g, r, atol=2e-5 + 1e-3 * float(r.abs().max())), (k, (g - r).abs().max().item())
        opt_cpu.step()
        assert abs(float((loss + aux).detach()) - float(ref.detach())) < 2e-4 * abs(float(ref.detach())), (step, float((loss + aux).detach()), float(ref.detach()))
    for k, p in model.named_parameters():
        assert torch.allclose(p.detach().cpu(), sd[k].detach(), atol=5e-4), k


def test_bf16_mfma_shapes_forward_backward(gpu):
    """bf16 with expert shapes the MFMA kernels take (H 256, I 128): logits and gradients against the oracle.

    Why the bars are wider than the single layer's 1e-2: the oracle run in bf16 on the CPU is itself one bf16
    evaluation of a 4-layer decoder -- 4 x (attention + MoE) with a rounding after every op, library kernels (attention,
    norms, dense projections) that round in other places on the GPU than on the CPU, a router whose near-tie tokens
    may pick another expert once the hidden state differs in its last bit, and a backward pass through all of it -- so
    two correct bf16 evaluations differ by a few rounding steps per layer.  The test therefore measures both bf16
    evaluations against the same oracle evaluated in fp32 arithmetic on the same bf16 weights (the value both
    approximate) and requires the GPU model to be about as close to it as the CPU's bf16 evaluation is (within a factor
    of 2 plus 5e-3); the direct GPU-vs-CPU-bf16 bars (logits 2e-2, loss 5e-2, gradients 6e-2 relative L2) are kept as
    a gross-error check."""
    cfg = make_config(hidden_size=256, intermediate_size=128, vocab_size=512, max_position_embeddings=128,
                      router_aux_loss_coef=0.01)
    model = build(cfg, seed=8, dtype=torch.bfloat16, std=0.05).train()
    sd = cpu_state(model, grad=True)
    sd32 = {k: v.detach().float().requires_grad_(v.requires_grad) for k, v in sd.items()}
    ids, tgt = batch(cfg, 2, 128, seed=9)
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss

    logits = model(ids.cuda())
    loss = F.cross_entropy(logits.view(-1, logits.size(-1)).float(), tgt.cuda().view(-1))
    (loss + collect_aux_loss(model).float()).backward()
    rel_l2 = lambda a, b: ((a.float() - b.float()).norm() / b.float().norm()).item()
    ref_logits, _ = L.llama_forward({k: v.detach() for k, v in sd.items()}, cfg, ids, training=False)
    true_logits, _ = L.llama_forward({k: v.detach() for k, v in sd32.items()}, cfg, ids, training=False)
    got_logits = logits.detach().cpu()
    rel = rel_l2(got_logits, ref_logits)
    assert rel < 2e-2, rel
    e_gpu, e_cpu = rel_l2(got_logits, true_logits), rel_l2(ref_logits, true_logits)
    print(f"logits vs the fp32 evaluation: GPU bf16 {e_gpu:.2e}, CPU bf16 {e_cpu:.2e}", flush=True)
    assert e_gpu <= 2.0 * e_cpu + 5e-3, (e_gpu, e_cpu)
    ref = L.train_loss(sd, cfg, ids, tgt)
    ref.backward()
    true = L.train_loss(sd32, cfg, ids, tgt)
    true.backward()
    assert abs(float(loss.detach()) - float(ref.detach())) < 5e-2 * abs(float(ref.detach()))
    for k, p in model.named_parameters():
        r = sd[k].grad.float()
        if float(r.norm()) == 0.0:
            continue
        rel = rel_l2(p.grad.cpu(), r)
        assert rel < 6e-2, (k, rel)
        t = sd32[k].grad
        e_gpu, e_cpu = rel_l2(p.grad.cpu(), t), rel_l2(r, t)
        print(f"d {k:48s} vs fp32: GPU bf16 {e_gpu:.2e}, CPU bf16 {e_cpu:.2e}", flush=True)
        assert e_gpu <= 2.0 * e_cpu + 5e-3, (k, e_gpu, e_cpu)
