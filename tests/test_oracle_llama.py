"""Pins the CPU restatement of the decoder around the MoE layer (oracle/llama_oracle.py) without running the reference:
each piece is checked against what the mathematics fixes or against a library routine."""

import math
import types

import torch
import torch.nn.functional as F

from oracle import llama_oracle as L


def _cfg(**kw):
    base = dict(vocab_size=97, hidden_size=32, intermediate_size=48, num_attention_heads=4, num_key_value_heads=2,
                num_hidden_layers=2, max_position_embeddings=24, rms_norm_eps=1e-5, rope_theta=10000.0,
                num_experts=4, num_experts_per_tok=2, num_shared_experts=1, norm_topk_prob=True)
    base.update(kw)
    return types.SimpleNamespace(**base)


def _state(cfg, seed=0, scale=0.2):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    d = H // cfg.num_attention_heads
    r = lambda *s: torch.randn(*s, generator=g) * scale
    sd = {"embedding.weight": r(V, H) / scale, "final_proj.weight": r(V, H), "final_norm.weight": 1 + r(H)}
    for i in range(cfg.num_hidden_layers):
        p = f"decoder_layers.{i}."
        sd[p + "input_layernorm.weight"] = 1 + r(H)
        if not getattr(cfg, "parallel_block", False):
            sd[p + "post_attention_layernorm.weight"] = 1 + r(H)
        sd[p + "attention.q_proj.weight"] = r(H, H)
        sd[p + "attention.k_proj.weight"] = r(cfg.num_key_value_heads * d, H)
        sd[p + "attention.v_proj.weight"] = r(cfg.num_key_value_heads * d, H)
        sd[p + "attention.out_proj.weight"] = r(H, H)
        if getattr(cfg, "num_experts", 1) > 1:
            sd[p + "mlp.gate.weight"] = r(cfg.num_experts, H)
            sd[p + "mlp.expert_bias"] = torch.zeros(cfg.num_experts)
            for e in range(cfg.num_experts):
                sd[p + f"mlp.local_experts.{e}.gate_proj.weight"] = r(I, H)
                sd[p + f"mlp.local_experts.{e}.up_proj.weight"] = r(I, H)
                sd[p + f"mlp.local_experts.{e}.down_proj.weight"] = r(H, I)
            if cfg.num_shared_experts:
                Is = I * cfg.num_shared_experts
                sd[p + "mlp.shared_expert.gate_proj.weight"] = r(Is, H)
                sd[p + "mlp.shared_expert.up_proj.weight"] = r(Is, H)
                sd[p + "mlp.shared_expert.down_proj.weight"] = r(H, Is)
        else:
            sd[p + "mlp.gate_proj.weight"], sd[p + "mlp.up_proj.weight"], sd[p + "mlp.down_proj.weight"] = r(I, H), r(I, H), r(H, I)
    return sd


def test_rope_is_a_rotation_by_position_times_frequency():
    S, d, base = 16, 8, 10000.0
    cos, sin = L.rope_tables(S, d, base)
    x = torch.randn(1, 2, S, d, generator=torch.Generator().manual_seed(1))
    got = L.rotate_half(x, cos, sin)
    # pair j = (x[j], x[j + d/2]) as a complex number, multiplied by exp(i * m * base^(-2j/d))
    z = torch.complex(x[..., : d // 2].double(), x[..., d // 2 :].double())
    m = torch.arange(S, dtype=torch.float64)[:, None]
    theta = base ** (-2.0 * torch.arange(d // 2, dtype=torch.float64) / d)
    w = z * torch.polar(torch.ones(S, d // 2, dtype=torch.float64), m * theta)
    want = torch.cat([w.real, w.imag], dim=-1)
    assert torch.allclose(got.double(), want, atol=1e-5)
    assert torch.allclose(got.norm(dim=-1), x.norm(dim=-1), atol=1e-5)
    # position 0 is the identity
    assert torch.equal(got[..., 0, :], x[..., 0, :])


def test_rope_scores_depend_on_the_distance_only():
    S, d = 20, 16
    cos, sin = L.rope_tables(S, d, 500000.0)
    g = torch.Generator().manual_seed(2)
    q, k = torch.randn(d, generator=g), torch.randn(d, generator=g)
    rq = L.rotate_half(q.expand(S, d), cos, sin)
    rk = L.rotate_half(k.expand(S, d), cos, sin)
    scores = rq @ rk.T
    for delta in (0, 1, 5):
        diag = torch.diagonal(scores, offset=-delta)  # q at m + delta, k at m
        assert torch.allclose(diag, diag[0].expand_as(diag), atol=1e-4)


def test_rms_norm_matches_the_library_routine():
    x = torch.randn(3, 5, 32, generator=torch.Generator().manual_seed(3)) * 4
    w = torch.rand(32, generator=torch.Generator().manual_seed(4)) + 0.5
    got = L.rms_norm(x, w, 1e-5)
    assert torch.allclose(got, F.rms_norm(x, (32,), w, 1e-5), atol=1e-6)
    assert torch.allclose(L.rms_norm(x, torch.ones(32), 0.0).pow(2).mean(-1), torch.ones(3, 5), atol=1e-5)
    # the normalised value is rounded to the input dtype before the weight multiplies it
    xb = x.bfloat16()
    h = xb.float() * torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-5)
    assert torch.equal(L.rms_norm(xb, w.bfloat16(), 1e-5), w.bfloat16() * h.bfloat16())


def test_attention_core_matches_library_and_a_loop():
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(2, 3, 7, 8, generator=g) for _ in range(3))
    got = L.causal_attention_core(q, k, v)
    assert torch.allclose(got, F.scaled_dot_product_attention(q, k, v, is_causal=True), atol=1e-5)
    assert torch.allclose(got[:, :, 0], v[:, :, 0], atol=1e-6)  # the first query sees only itself
    for b in range(2):
        for h in range(3):
            for i in range(7):
                s = torch.tensor([float(q[b, h, i] @ k[b, h, j]) / math.sqrt(8) for j in range(i + 1)])
                p = torch.softmax(s, 0)
                want = sum(p[j] * v[b, h, j] for j in range(i + 1))
                assert torch.allclose(got[b, h, i], want, atol=1e-5)


def test_attention_repeats_kv_heads_in_groups():
    """Grouped-query attention: query head h reads kv head h // group (repeat_interleave, not tile)."""
    cfg = _cfg(num_hidden_layers=1)
    sd = _state(cfg)
    x = torch.randn(1, 6, cfg.hidden_size, generator=torch.Generator().manual_seed(6))
    cos, sin = L.rope_tables(6, 8, cfg.rope_theta)
    got = L.attention(x, sd, "decoder_layers.0.attention.", cfg, cos, sin)
    p = "decoder_layers.0.attention."
    d, nh, nkv = 8, 4, 2
    q = (x @ sd[p + "q_proj.weight"].T).view(1, 6, nh, d)
    k = (x @ sd[p + "k_proj.weight"].T).view(1, 6, nkv, d)
    v = (x @ sd[p + "v_proj.weight"].T).view(1, 6, nkv, d)
    heads = []
    for h in range(nh):
        qh = L.rotate_half(q[:, :, h], cos, sin)
        kh = L.rotate_half(k[:, :, h // (nh // nkv)], cos, sin)
        heads.append(F.scaled_dot_product_attention(qh[:, None], kh[:, None], v[:, None, :, h // (nh // nkv)], is_causal=True)[:, 0])
    want = torch.cat(heads, dim=-1) @ sd[p + "out_proj.weight"].T
    assert torch.allclose(got, want, atol=1e-5)


def test_llama_forward_is_causal_and_matches_a_library_composition():
    for cfg in (_cfg(), _cfg(parallel_block=True), _cfg(num_experts=1, num_shared_experts=0)):
        sd = _state(cfg)
        g = torch.Generator().manual_seed(7)
        ids = torch.randint(0, cfg.vocab_size, (2, 12), generator=g)
        logits, auxes = L.llama_forward(sd, cfg, ids)
        assert logits.shape == (2, 12, cfg.vocab_size) and auxes == []
        ids2 = ids.clone()
        ids2[:, 8:] = (ids2[:, 8:] + 1) % cfg.vocab_size
        logits2, _ = L.llama_forward(sd, cfg, ids2)
        assert torch.allclose(logits[:, :8], logits2[:, :8], atol=1e-5) and not torch.allclose(logits[:, 8:], logits2[:, 8:])
        # a composition written with library routines: F.rms_norm, F.scaled_dot_product_attention
        x = F.embedding(ids, sd["embedding.weight"])
        cos, sin = L.rope_tables(12, 8, cfg.rope_theta)
        for i in range(cfg.num_hidden_layers):
            p = f"decoder_layers.{i}."
            n = F.rms_norm(x, (32,), sd[p + "input_layernorm.weight"], cfg.rms_norm_eps)
            q = (n @ sd[p + "attention.q_proj.weight"].T).view(2, 12, 4, 8).transpose(1, 2)
            k = (n @ sd[p + "attention.k_proj.weight"].T).view(2, 12, 2, 8).transpose(1, 2)
            v = (n @ sd[p + "attention.v_proj.weight"].T).view(2, 12, 2, 8).transpose(1, 2)
            q, k = L.rotate_half(q, cos, sin), L.rotate_half(k, cos, sin)
            a = F.scaled_dot_product_attention(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), is_causal=True)
            a = a.transpose(1, 2).reshape(2, 12, 32) @ sd[p + "attention.out_proj.weight"].T
            if getattr(cfg, "parallel_block", False):
                x = x + a + L.feed_forward(n, sd, p + "mlp.", cfg, False)[0]
            else:
                x = x + a
                n2 = F.rms_norm(x, (32,), sd[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
                x = x + L.feed_forward(n2, sd, p + "mlp.", cfg, False)[0]
        want = F.rms_norm(x, (32,), sd["final_norm.weight"], cfg.rms_norm_eps) @ sd["final_proj.weight"].T
        assert torch.allclose(logits, want, atol=1e-4)


def test_train_loss_adds_one_aux_term_per_moe_layer():
    cfg = _cfg(router_aux_loss_coef=0.01)
    sd = _state(cfg)
    g = torch.Generator().manual_seed(8)
    ids, tgt = torch.randint(0, cfg.vocab_size, (1, 16), generator=g), torch.randint(0, cfg.vocab_size, (1, 16), generator=g)
    logits, auxes = L.llama_forward(sd, cfg, ids, training=True)
    assert len(auxes) == cfg.num_hidden_layers and all(a > 0 for a in auxes)
    ce = F.cross_entropy(logits.view(-1, cfg.vocab_size), tgt.view(-1))
    assert torch.allclose(L.train_loss(sd, cfg, ids, tgt), ce + sum(auxes), atol=1e-6)
    # a uniform random guess costs ln(vocab): the loss of these random weights is of that order
    assert 0.5 * math.log(cfg.vocab_size) < float(ce) < 3 * math.log(cfg.vocab_size)
