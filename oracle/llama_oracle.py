"""CPU oracle for the decoder the MoE layer is called from.  TEST INFRASTRUCTURE ONLY.

Restates, with plain torch on the CPU, the single-device forward of the reference's Llama (embedding, decoder layers of
RMSNorm / rotary causal grouped-query attention / MoE or dense SwiGLU MLP, final norm, vocabulary projection) as a
function of a state_dict that uses the reference's parameter names.  The MoE layers go through
``oracle.moe_oracle.moe_forward``.  Only ``tests/`` may import this file; nothing under ``picotron_amd/`` does.

Reference lines each function follows (paths relative to the reference checkout):

  rope_tables      picotron/model.py:39-52     (get_cos_sin; fp32 angles, table repeated twice along the last axis)
  rotate_half      picotron/model.py:29-36     (apply_rotary_pos_emb)
  rms_norm         picotron/model.py:109-114   (LlamaRMSNorm.forward)
  attention        picotron/model.py:157-233   (the FLASH_ATTEN=0 branch: q/k/v projections, RoPE on q and k,
                                                repeat_interleave of the kv heads, causal softmax(QK^T/sqrt(d))V, out_proj)
  decoder_layer    picotron/model.py:323-340   (sequential and parallel-block residual forms)
  llama_forward    picotron/model.py:393-401
  train_loss       tests/bench_ep_train_step.py:54-60 (cross entropy on fp32 logits) plus the aux losses the MoE layers
                   stash, picotron/expert_parallel/expert_parallel.py:442-454 (collect_aux_loss)

What pins each function (tests/test_oracle_llama.py):
  * rope: the rotation written as a complex multiplication exp(i m theta_j) per pair; norms preserved; the q.k product
    depends only on the distance between the two positions.
  * rms_norm: ``torch.nn.functional.rms_norm`` (a library routine) in fp32; unit mean square of the output.
  * attention core: ``torch.nn.functional.scaled_dot_product_attention(is_causal=True)`` on the CPU in fp32, and a
    per-query Python loop on a tiny case; the first position attends only to itself (output = its own v).
  * decoder_layer / llama_forward: composition only (residual adds); checked for causality (changing a later token leaves
    earlier logits unchanged) and against the library routines end to end.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


def rope_tables(seq_length, head_dim, base):
    theta = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    angle = torch.arange(seq_length).unsqueeze(1).float() * theta
    return torch.cos(angle).repeat(1, 2), torch.sin(angle).repeat(1, 2)


def rotate_half(x, cos, sin):
    d = x.shape[-1]
    x1, x2 = x[..., : d // 2], x[..., d // 2 :]
    return x * cos + torch.cat([-x2, x1], dim=-1) * sin


def rms_norm(x, weight, eps):
    h = x.to(torch.float32)
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    return weight * h.to(x.dtype)


def causal_attention_core(q, k, v):
    """q, k, v [B, heads, S, d] -> [B, heads, S, d]; scores and softmax in fp32."""
    S, d = q.shape[-2], q.shape[-1]
    scores = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(d)
    mask = torch.ones(S, S, dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, float("-inf"))
    return (torch.softmax(scores, dim=-1) @ v.float()).to(q.dtype)


def attention(x, sd, prefix, cfg, cos, sin):
    B, S, H = x.shape
    nh, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    d = H // nh
    q = F.linear(x, sd[prefix + "q_proj.weight"]).view(B, S, nh, d).transpose(1, 2)
    k = F.linear(x, sd[prefix + "k_proj.weight"]).view(B, S, nkv, d).transpose(1, 2)
    v = F.linear(x, sd[prefix + "v_proj.weight"]).view(B, S, nkv, d).transpose(1, 2)
    q, k = rotate_half(q, cos, sin), rotate_half(k, cos, sin)
    k, v = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)
    out = causal_attention_core(q, k, v).transpose(1, 2).reshape(B, S, nh * d)
    return F.linear(out, sd[prefix + "out_proj.weight"])


def moe_weights(sd, prefix, cfg):
    E = cfg.num_experts
    stack = lambda name: torch.stack([sd[f"{prefix}local_experts.{e}.{name}.weight"] for e in range(E)])
    shared = None
    if getattr(cfg, "num_shared_experts", 0) > 0:
        shared = tuple(sd[f"{prefix}shared_expert.{n}.weight"] for n in ("gate_proj", "up_proj", "down_proj"))
    return O.LayerWeights(
        router_w=sd[prefix + "gate.weight"], gate_w=stack("gate_proj"), up_w=stack("up_proj"), down_w=stack("down_proj"),
        shared=shared, expert_bias=sd.get(prefix + "expert_bias"),
    )


def feed_forward(x, sd, prefix, cfg, training):
    """The ``mlp`` slot of a decoder layer: MoE when cfg.num_experts > 1, else the dense SwiGLU MLP.  Returns (y, aux)."""
    if getattr(cfg, "num_experts", 1) > 1:
        B, S, H = x.shape
        out, info = O.moe_forward(
            x.reshape(-1, H), moe_weights(sd, prefix, cfg), cfg.num_experts_per_tok,
            norm_topk_prob=getattr(cfg, "norm_topk_prob", True),
            aux_coef=getattr(cfg, "router_aux_loss_coef", 0.0), training=training,
        )
        return out.view(B, S, H), info.get("aux")
    return O.mlp(x, sd[prefix + "gate_proj.weight"], sd[prefix + "up_proj.weight"], sd[prefix + "down_proj.weight"]), None


def decoder_layer(x, sd, prefix, cfg, cos, sin, training):
    eps = cfg.rms_norm_eps
    if getattr(cfg, "parallel_block", False):
        n = rms_norm(x, sd[prefix + "input_layernorm.weight"], eps)
        y, aux = feed_forward(n, sd, prefix + "mlp.", cfg, training)
        return x + attention(n, sd, prefix + "attention.", cfg, cos, sin) + y, aux
    x = x + attention(rms_norm(x, sd[prefix + "input_layernorm.weight"], eps), sd, prefix + "attention.", cfg, cos, sin)
    y, aux = feed_forward(rms_norm(x, sd[prefix + "post_attention_layernorm.weight"], eps), sd, prefix + "mlp.", cfg, training)
    return x + y, aux


def llama_forward(sd, cfg, input_ids, training=False):
    """logits [B, S, vocab] and the list of aux losses (one per MoE layer that produced one)."""
    x = sd["embedding.weight"][input_ids]
    S = input_ids.shape[1]
    cos, sin = rope_tables(cfg.max_position_embeddings, cfg.hidden_size // cfg.num_attention_heads, cfg.rope_theta)
    cos, sin = cos[:S].to(x.dtype), sin[:S].to(x.dtype)
    auxes = []
    for i in range(cfg.num_hidden_layers):
        x, aux = decoder_layer(x, sd, f"decoder_layers.{i}.", cfg, cos, sin, training)
        if aux is not None:
            auxes.append(aux)
    return F.linear(rms_norm(x, sd["final_norm.weight"], cfg.rms_norm_eps), sd["final_proj.weight"]), auxes


def train_loss(sd, cfg, input_ids, target_ids):
    logits, auxes = llama_forward(sd, cfg, input_ids, training=True)
    loss = F.cross_entropy(logits.view(-1, logits.size(-1)).float(), target_ids.view(-1))
    for aux in auxes:
        loss = loss + aux.float()
    return loss
