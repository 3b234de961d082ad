"""CPU oracle for the single-GPU (EP=1) MoE hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU with plain torch/numpy, the algorithm of the reference's naive torch
MoE path.  It exists to CHECK the HIP kernels; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it.  Nothing under ``picotron_amd/`` imports it.

Reference lines each function follows (paths relative to the reference checkout):

  softmax_topk_route   picotron/expert_parallel/expert_parallel.py:174-184   (_route)
  balance              picotron/expert_parallel/expert_parallel.py:189-212   (_balance)
  expand_routed        picotron/expert_parallel/expert_parallel.py:214-217   (_expand_routed)
  permute_plan         picotron/expert_parallel/expert_parallel.py:30-35, 335-339
  expert_ffn           picotron/expert_parallel/expert_parallel.py:323-329,
                       picotron/expert_parallel/megakernel.py:308-318, picotron/model.py:258
  silu_and_mul_bwd     picotron/expert_parallel/megakernel.py:187-197
  expert_ffn_backward_explicit  picotron/expert_parallel/megakernel.py:332-357 (fused_moe_dgrad / fused_moe_wgrad)
  combine_topk         picotron/expert_parallel/expert_parallel.py:219-224
  compute_capacity     picotron/expert_parallel/capacity_moe.py:33-41
  slot_assignment      picotron/expert_parallel/capacity_moe.py:44-57
  capped_forward       picotron/expert_parallel/capacity_moe.py:93-160 (drop mode and dropless rounds)
  quant_fp8 / dequant  picotron/expert_parallel/ep_communications.py:59-68, :100
  moe_forward          picotron/expert_parallel/expert_parallel.py:144-166, 271-309; the LatentMoE
                       projections around the routed path: :59-69, :226-228 (_maybe_down), :250-252 (_finalize)

What pins each function (see tests/test_oracle_*.py):
  * route: brute-force per-row Python selection, torch.topk on tie-free rows, weights sum to one.
  * balance: a uniform router gives aux == coef exactly; sign rule monotonicity.
  * permute_plan / slot_assignment: torch.argsort(stable=True) + torch.bincount (library routines).
  * capacity: the drop-percentage / round tables the reference README holds (tests/golden/).
  * fp8: closed-form 256-entry decode table; software RNE encoder against
    ``Tensor.to(torch.float8_e4m3fn)`` on every interesting fp32 value; oracle/fp8_e4m3.c.
  * expert_ffn: a per-token brute-force loop; silu_and_mul_bwd: autograd and finite differences;
    expert_ffn_backward_explicit: autograd over expert_ffn in float64 (the two are the same mathematics).
  * moe_forward: a per-token brute-force MoE (each token sent through its experts one at a time);
    latent: equals the plain layer run on ``tokens @ W_down^T`` (same routing) followed by ``@ W_up^T``,
    two library matmuls, plus the shared expert on the full-width tokens; dropless rounds: equal to the
    uncapped layer when ``max_rounds`` covers every row, and to the drop mode at capacity
    ``max_rounds * C`` when it does not (the rounds partition the rows by rank).

Tie rule for top-k (``torch.topk`` leaves the order of equal scores unspecified): higher score
first; among equal scores the lower expert id first.  The HIP router uses the same rule.
"""

from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

E4M3_MAX = 448.0


# ------------------------------------------------------------------------------------------------
# Router
# ------------------------------------------------------------------------------------------------
def softmax_topk_route(logits, top_k, expert_bias=None, norm_topk_prob=True, out_dtype=None):
    """probs = softmax_fp32(logits); pick top_k of (probs + expert_bias); gate weights are the
    UNBIASED probs at the picks, optionally renormalised to sum to one, cast to ``out_dtype``.

    Returns (topk_idx int64 [T,k], topk_w out_dtype [T,k], probs fp32 [T,E]).
    """
    out_dtype = out_dtype or logits.dtype
    probs = F.softmax(logits, dim=-1, dtype=torch.float32)
    sel = probs + expert_bias if expert_bias is not None else probs
    # stable descending sort == "higher score first, lower expert id on equal score"
    topk_idx = torch.sort(sel, dim=-1, descending=True, stable=True).indices[:, :top_k].contiguous()
    topk_w = probs.gather(-1, topk_idx)
    if norm_topk_prob and top_k > 1:
        topk_w = topk_w / topk_w.sum(dim=-1, keepdim=True)
    return topk_idx, topk_w.to(out_dtype), probs


def tie_rows(logits, top_k, expert_bias=None):
    """Rows whose selection score repeats anywhere in the first top_k+1 sorted positions: on those
    rows only the selected *scores* (not the indices) are comparable between implementations."""
    probs = F.softmax(logits, dim=-1, dtype=torch.float32)
    sel = probs + expert_bias if expert_bias is not None else probs
    s = torch.sort(sel, dim=-1, descending=True, stable=True).values
    upto = min(top_k + 1, s.shape[1])
    return (s[:, : upto - 1] == s[:, 1:upto]).any(dim=-1)


def balance(probs, topk_idx, num_experts, top_k, aux_coef, bias_rate, expert_bias=None):
    """Aux loss ``coef * sum_e f_e * P_e`` (f_e = count_e * E/(k*T) detached, P_e = mean_t probs) and
    the loss-free bias step ``bias += rate * sign(mean(load) - load)``.

    Returns (aux or None, new_bias or None, counts fp32 [E]).
    """
    T = probs.shape[0]
    counts = torch.zeros(num_experts, dtype=probs.dtype)
    counts.scatter_add_(0, topk_idx.reshape(-1), torch.ones(topk_idx.numel(), dtype=probs.dtype))
    aux = None
    if aux_coef > 0:
        f = counts * (num_experts / (top_k * T))
        aux = aux_coef * (f * probs.mean(dim=0)).sum()
    new_bias = None
    if bias_rate > 0:
        with torch.no_grad():
            new_bias = expert_bias + bias_rate * torch.sign(counts.mean() - counts)
    return aux, new_bias, counts


# ------------------------------------------------------------------------------------------------
# Permutation (stable counting sort by expert) and capacity slotting
# ------------------------------------------------------------------------------------------------
def expand_routed(tokens, topk_idx, topk_w):
    """One routed row per (token, pick), token-major: flat row r = t*k + j."""
    k = topk_idx.shape[1]
    token_idx = torch.arange(tokens.shape[0]).repeat_interleave(k)
    return tokens[token_idx], topk_idx.reshape(-1), topk_w.reshape(-1), token_idx


def permute_plan(expert_idx, num_experts):
    """Textbook stable counting sort.  order[pos] = flat row that lands at sorted position pos;
    inv_order[r] = sorted position of flat row r; counts[e] = rows of expert e."""
    e = np.asarray(expert_idx, dtype=np.int64)
    counts = np.zeros(num_experts, dtype=np.int64)
    for v in e:
        counts[v] += 1
    cursor = np.concatenate([[0], np.cumsum(counts)[:-1]])
    order = np.empty(e.size, dtype=np.int64)
    inv = np.empty(e.size, dtype=np.int64)
    for r, v in enumerate(e):
        order[cursor[v]] = r
        inv[r] = cursor[v]
        cursor[v] += 1
    return torch.from_numpy(order), torch.from_numpy(inv), torch.from_numpy(counts)


def permute_plan_fast(expert_idx, num_experts):
    """Same result as ``permute_plan`` through library routines (for large inputs)."""
    order = torch.argsort(expert_idx, stable=True)
    inv = torch.empty_like(order)
    inv[order] = torch.arange(order.numel())
    return order, inv, torch.bincount(expert_idx, minlength=num_experts)


def compute_capacity(num_tokens, top_k, num_experts, capacity_factor):
    return max(1, int(capacity_factor * ((num_tokens * top_k) / num_experts) + 0.999))


def slot_assignment(expert_idx, num_experts):
    """within[r] = how many earlier flat rows chose the same expert as row r."""
    _, inv, counts = permute_plan_fast(expert_idx, num_experts)
    starts = torch.cumsum(counts, 0) - counts
    return inv - starts[expert_idx], counts


def capacity_rounds(counts, capacity, dropless, max_rounds):
    if not dropless:
        return 1
    need = int((int(counts.max()) + capacity - 1) // capacity) if counts.numel() else 1
    return max(1, min(need, max_rounds))


# ------------------------------------------------------------------------------------------------
# Expert FFN
# ------------------------------------------------------------------------------------------------
def mlp(x, gate_w, up_w, down_w):
    """One SwiGLU MLP with bias-free linears: down(silu(gate(x)) * up(x)); every Linear / silu / mul
    rounds to the tensor dtype, as torch modules do."""
    return F.linear(F.silu(F.linear(x, gate_w)) * F.linear(x, up_w), down_w)


def expert_ffn(x_sorted, counts, gate_w, up_w, down_w, row_weight=None):
    """Rows grouped by expert: expert e owns the next counts[e] rows.  gate_w/up_w [E,I,H], down_w [E,H,I]."""
    outs, start = [], 0
    for e, n in enumerate(counts.tolist()):
        outs.append(mlp(x_sorted[start : start + n], gate_w[e], up_w[e], down_w[e]))
        start += n
    y = torch.cat(outs, dim=0) if outs else x_sorted.new_empty((0, x_sorted.shape[1]))
    if row_weight is not None:
        y = y * row_weight[:, None]
    return y


def expert_ffn_backward(x_sorted, counts, gate_w, up_w, down_w, dy):
    """(dx, d_gate, d_up, d_down) by autograd over ``expert_ffn`` -- the reference's CPU backward."""
    with torch.enable_grad():
        leaves = [t.detach().clone().requires_grad_(True) for t in (x_sorted, gate_w, up_w, down_w)]
        y = expert_ffn(leaves[0], counts, leaves[1], leaves[2], leaves[3])
        return torch.autograd.grad(y, leaves, dy)


def expert_ffn_backward_explicit(x_sorted, counts, gate_w, up_w, down_w, dy):
    """(dx, d_gate, d_up, d_down) by the reference's explicit dgrad / wgrad formulas (megakernel.py:332-357, what its
    ``_FusedMoE.backward`` runs on a GPU), spelled with library matmuls and rounding where those kernels round:
    ``[g|u]`` and ``da = dy @ down_w`` to the tensor dtype, the SwiGLU backward in fp32 arithmetic rounded once
    (:187-197), ``dx = [dg|du] @ [gate_w; up_w]`` as ONE contraction over 2I rounded once, the weight gradients as
    contractions over the expert's rows.  Mathematically the same as ``expert_ffn_backward``; in bf16 the autograd
    form rounds ``da*u``, ``dg``, ``du`` and the two halves of ``dx`` separately."""
    dxs, dgs, dus, dds, start = [], [], [], [], 0
    for e, n in enumerate(counts.tolist()):
        x, d = x_sorted[start : start + n], dy[start : start + n]
        inter13 = torch.cat([F.linear(x, gate_w[e]), F.linear(x, up_w[e])], dim=1)
        a = F.silu(inter13[:, : gate_w.shape[1]]) * inter13[:, gate_w.shape[1] :]
        da = d @ down_w[e]
        d13 = silu_and_mul_bwd(inter13, da)
        dxs.append(d13 @ torch.cat([gate_w[e], up_w[e]], dim=0))
        dds.append(d.t() @ a)
        dw13 = d13.t() @ x
        dgs.append(dw13[: gate_w.shape[1]])
        dus.append(dw13[gate_w.shape[1] :])
        start += n
    dx = torch.cat(dxs, dim=0) if dxs else torch.zeros_like(x_sorted)
    return dx, torch.stack(dgs), torch.stack(dus), torch.stack(dds)


class _ExplicitFfn(torch.autograd.Function):
    """``expert_ffn`` whose backward is ``expert_ffn_backward_explicit`` (the reference's ``_FusedMoE``,
    megakernel.py:376-400, without a row weight)."""

    @staticmethod
    def forward(ctx, x_sorted, counts, gate_w, up_w, down_w):
        ctx.save_for_backward(x_sorted, gate_w, up_w, down_w)
        ctx.counts = counts
        return expert_ffn(x_sorted, counts, gate_w, up_w, down_w)

    @staticmethod
    def backward(ctx, dy):
        x_sorted, gate_w, up_w, down_w = ctx.saved_tensors
        dx, dg, du, dd = expert_ffn_backward_explicit(x_sorted, ctx.counts, gate_w, up_w, down_w, dy)
        return dx, None, dg, du, dd


def silu_and_mul_bwd(inter13, da):
    """inter13 = [g | u] ([N,2I]); da [N,I] -> [dg | du] in fp32 arithmetic, cast back."""
    inter = da.shape[1]
    wide = torch.float64 if inter13.dtype == torch.float64 else torch.float32   # fp32 arithmetic, as the reference
    g, u, d = inter13[:, :inter].to(wide), inter13[:, inter:].to(wide), da.to(wide)
    s = torch.sigmoid(g)
    dg = d * u * s * (1 + g * (1 - s))
    du = d * g * s
    return torch.cat([dg, du], dim=1).to(inter13.dtype)


def combine_topk(y, weights, num_tokens, top_k):
    """out[t] = sum_j (y[t*k+j] * w[t*k+j]); the product is rounded to the dtype before the sum."""
    return (y * weights.unsqueeze(-1)).view(num_tokens, top_k, -1).sum(dim=1)


# ------------------------------------------------------------------------------------------------
# FP8 E4M3 (OCP "FN" variant: no inf, 0x7F/0xFF = NaN, max 448, min subnormal 2^-9)
# ------------------------------------------------------------------------------------------------
def e4m3_decode_table():
    """Closed-form value of every code: sign * 2^(e-7) * (1 + m/8) (e>0), sign * 2^-6 * m/8 (e=0)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e, m = (code >> 3) & 0xF, code & 0x7
        if e == 0xF and m == 0x7:
            out[code] = np.nan
        elif e == 0:
            out[code] = sign * math.ldexp(m / 8.0, -6)
        else:
            out[code] = sign * math.ldexp(1.0 + m / 8.0, e - 7)
    return out


def e4m3_encode_rne(x):
    """Round-to-nearest-even fp32 -> E4M3FN code (numpy, bit level).  |x| > 464 (the midpoint past
    448; 464 itself ties to the even 448) and NaN map to the NaN code, like torch's cast; callers
    clamp to +-448 first."""
    bits = np.ascontiguousarray(np.asarray(x, dtype=np.float32)).view(np.uint32).astype(np.int64)
    sign = ((bits >> 24) & 0x80).astype(np.int64)
    mag = bits & 0x7FFFFFFF
    out = np.zeros(mag.shape, dtype=np.int64)

    nan_or_big = mag >= 0x43F00000  # 480.0 and above (incl. inf/NaN) -> NaN code
    # normal range of e4m3: |x| >= 2^-6  (fp32 exponent field >= 121)
    normal = (mag >= (121 << 23)) & ~nan_or_big
    # RNE on the 20 dropped mantissa bits
    lsb = (mag >> 20) & 1
    rounded = mag + 0x7FFFF + lsb
    code_n = ((rounded >> 20) - ((127 - 7) << 3)) & 0xFF
    # 464 < |x| < 480 rounds up past 448 -> code 0x7F which already is the NaN code
    out = np.where(normal, code_n, out)

    # subnormal range: value = m * 2^-9, m = RNE(|x| * 2^9) in 0..8 (8 -> smallest normal, code 0x08)
    sub = mag < (121 << 23)
    xf = np.abs(np.asarray(x, dtype=np.float32).astype(np.float64)) * 512.0
    m = np.rint(xf).astype(np.int64)  # rint = ties-to-even
    out = np.where(sub, m, out)
    out = np.where(nan_or_big, 0x7F, out)
    return (out | sign).astype(np.uint8)


def quant_fp8(x, encoder="torch"):
    """Per-row scaled E4M3: amax and scale are computed IN x's DTYPE (bf16 rounding when x is bf16),
    the quotient in fp32.  Returns (codes uint8 [N,H], scale fp32 [N])."""
    amax = x.abs().amax(dim=-1, keepdim=True)
    amax = torch.maximum(amax, torch.tensor(1e-4, dtype=x.dtype))  # the floor is cast to x.dtype
    amax = torch.where(torch.isnan(x).any(dim=-1, keepdim=True), torch.full_like(amax, float("nan")), amax)
    scale = amax / E4M3_MAX
    ratio = (x.float() / scale.float()).clamp(-E4M3_MAX, E4M3_MAX)
    if encoder == "torch":
        codes = ratio.to(torch.float8_e4m3fn).view(torch.uint8)
    else:
        codes = torch.from_numpy(e4m3_encode_rne(ratio.numpy()))
    return codes, scale.squeeze(-1).float()


def dequant_fp8(codes, scale, dtype):
    """codes -> dtype (exact), scale -> dtype (rounds when dtype is bf16), product rounded to dtype."""
    vals = torch.from_numpy(e4m3_decode_table())[codes.long()]
    return vals.to(dtype) * scale.unsqueeze(-1).to(dtype)


# ------------------------------------------------------------------------------------------------
# Whole layer
# ------------------------------------------------------------------------------------------------
class LayerWeights:
    """Plain container: router [E,H] (+ optional bias [E]), experts gate/up [E,I,H], down [E,H,I],
    optional shared MLP (gate [Is,H], up [Is,H], down [H,Is]), expert_bias [E] for loss-free balancing,
    optional LatentMoE projections ``latent = (down [L,H], up [H,L])`` -- the experts then work in width L
    (gate/up [E,I,L], down [E,L,I]) while the router and the shared expert keep the full width H."""

    def __init__(self, router_w, gate_w, up_w, down_w, router_b=None, shared=None, expert_bias=None, latent=None):
        self.router_w, self.router_b = router_w, router_b
        self.gate_w, self.up_w, self.down_w = gate_w, up_w, down_w
        self.shared = shared
        self.expert_bias = expert_bias
        self.latent = latent

    def tensors(self):
        ts = [self.router_w, self.gate_w, self.up_w, self.down_w]
        if self.router_b is not None:
            ts.append(self.router_b)
        if self.shared is not None:
            ts.extend(self.shared)
        if self.latent is not None:
            ts.extend(self.latent)
        return ts


def run_local_experts(routed, expert_idx, w, ffn_backward="autograd"):
    order, inv, counts = permute_plan_fast(expert_idx, w.gate_w.shape[0])
    if ffn_backward == "explicit":
        y_sorted = _ExplicitFfn.apply(routed[order], counts, w.gate_w, w.up_w, w.down_w)
    else:
        y_sorted = expert_ffn(routed[order], counts, w.gate_w, w.up_w, w.down_w)
    return y_sorted[inv], (order, inv, counts)


def moe_forward(
    tokens,
    w,
    top_k,
    norm_topk_prob=True,
    use_loss_free=False,
    capacity_factor=0.0,
    capacity_dropless=True,
    max_rounds=8,
    fp8_dispatch=False,
    aux_coef=0.0,
    bias_rate=0.0,
    training=False,
    routing=None,
    logits=None,
    dispatch_dtype=None,
    ffn_backward="autograd",
):
    """Naive (or capacity-capped) EP=1 MoE layer on [T,H] tokens.  Returns (out [T,H], info dict).

    ``routing=(topk_idx, topk_w)`` bypasses the router (the reference's tests call the private
    ``_moe_naive`` / ``_moe_capped`` that way); ``logits`` substitutes externally computed router
    logits so a GPU run's own logits can be scored with this selection rule.
    With ``fp8_dispatch`` each routed row goes through quant -> dequant just before the expert FFN
    (what the reference's FP8 all-to-all does to the rows it ships), gradient straight through;
    ``dispatch_dtype`` (test aid) quantises the rows as that dtype would -- amax and scale rounded to it -- when the
    rest of the layer is evaluated in a wider one (an fp32-arithmetic reference for a bf16 layer).
    ``ffn_backward``: "autograd" differentiates the expert FFN op by op (the reference on a CPU, megakernel.py:321-329),
    "explicit" uses its dgrad / wgrad formulas (the reference on a GPU, :332-357); uncapped path only.
    """
    T, H = tokens.shape
    E = w.gate_w.shape[0]
    info = {}
    if routing is None:
        if logits is None:
            logits = F.linear(tokens, w.router_w, w.router_b)
        bias = w.expert_bias if use_loss_free else None
        topk_idx, topk_w, probs = softmax_topk_route(logits, top_k, bias, norm_topk_prob, tokens.dtype)
        info.update(logits=logits, probs=probs)
        if training and (aux_coef > 0 or bias_rate > 0):
            aux, new_bias, counts_f = balance(probs, topk_idx, E, top_k, aux_coef, bias_rate, w.expert_bias)
            info.update(aux=aux, new_bias=new_bias)
    else:
        topk_idx, topk_w = routing
    info.update(topk_idx=topk_idx, topk_w=topk_w)

    shared_out = mlp(tokens, *w.shared) if w.shared is not None else None
    # LatentMoE: the routed path runs on the down-projected tokens (a bias-free Linear, rounded to the tensor dtype)
    routed_in = F.linear(tokens, w.latent[0]) if w.latent is not None else tokens
    D = routed_in.shape[1]
    routed, expert_idx, weights, token_idx = expand_routed(routed_in, topk_idx, topk_w)
    if fp8_dispatch:
        wire = dispatch_dtype or routed.dtype
        codes, scale = quant_fp8(routed.detach().to(wire))
        deq = dequant_fp8(codes, scale, wire).to(routed.dtype)
        routed = routed + (deq - routed).detach()  # value of deq, gradient of identity
        info.update(fp8_codes=codes, fp8_scale=scale)

    if capacity_factor > 0:
        C = compute_capacity(T, top_k, E, capacity_factor)
        within, counts = slot_assignment(expert_idx, E)
        rounds = capacity_rounds(counts, C, capacity_dropless, max_rounds)
        out = torch.zeros(T, D, dtype=tokens.dtype)
        keep_any = torch.zeros_like(within, dtype=torch.bool)
        for r in range(rounds):
            slot = within - r * C
            keep = (slot >= 0) & (slot < C)
            if not bool(keep.any()):
                continue
            keep_any |= keep
            target = expert_idx[keep] * C + slot[keep]
            buf = torch.zeros(E * C, D, dtype=tokens.dtype).index_add(0, target, routed[keep])
            ybuf = expert_ffn(buf, torch.full((E,), C, dtype=torch.int64), w.gate_w, w.up_w, w.down_w)
            contrib = ybuf[target] * weights[keep].unsqueeze(-1).to(ybuf.dtype)
            out = out + torch.zeros(T, D, dtype=tokens.dtype).index_add(0, token_idx[keep], contrib)
        info.update(capacity=C, within=within, counts=counts, keep=keep_any, rounds=rounds)
    else:
        y, (order, inv, counts) = run_local_experts(routed, expert_idx, w, ffn_backward)
        info.update(order=order, inv_order=inv, counts=counts, y_routed=y)
        out = combine_topk(y, weights, T, top_k)

    if w.latent is not None:  # back up to the full width before the shared expert is added
        out = F.linear(out, w.latent[1])
    if shared_out is not None:
        out = out + shared_out
    return out, info


def moe_brute_force(tokens, w, top_k, norm_topk_prob=True):
    """Independent per-token restatement (one token, one expert at a time) used to pin moe_forward;
    mirrors the structure of the brute-force check in the reference's own test
    (tests/test_expert_parallel.py:32-48)."""
    logits = F.linear(tokens, w.router_w, w.router_b)
    out = torch.zeros_like(tokens)
    for t in range(tokens.shape[0]):
        p = torch.softmax(logits[t].float(), dim=-1)
        picks = sorted(range(p.numel()), key=lambda e: (-float(p[e]), e))[:top_k]
        pw = torch.stack([p[e] for e in picks])
        if norm_topk_prob and top_k > 1:
            pw = pw / pw.sum()
        pw = pw.to(tokens.dtype)
        for j, e in enumerate(picks):
            out[t] += pw[j] * mlp(tokens[t : t + 1], w.gate_w[e], w.up_w[e], w.down_w[e]).squeeze(0)
    if w.shared is not None:
        out = out + mlp(tokens, *w.shared)
    return out
