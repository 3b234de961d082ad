"""torch.autograd wrappers over the C-ABI kernels: router, permute plan, gather, combine.

Host-side plumbing only (tensor allocation, stream, argument marshalling); all arithmetic is in
``libpicomoe.so``.  Every function requires CUDA tensors.
"""

from dataclasses import dataclass
from typing import Optional

import torch

from picotron_amd import _lib


def _empty(shape, dtype, device):
    return torch.empty(shape, dtype=dtype, device=device)


# ------------------------------------------------------------------------------------------------
# Router
# ------------------------------------------------------------------------------------------------
class _Route(torch.autograd.Function):
    """softmax -> top-k -> gate weights (+ aux loss and loss-free bias step when ``balance``)."""

    @staticmethod
    def forward(ctx, logits, bias_f32, top_k, norm_topk, balance, aux_coef, bias_rate):
        _lib.require_cuda(logits)
        lib = _lib.load()
        logits = logits.contiguous()
        T, E = logits.shape
        dev = logits.device
        idx = _empty((T, top_k), torch.int64, dev)
        w = _empty((T, top_k), logits.dtype, dev)
        probs = _empty((T, E), torch.float32, dev)
        counts = partial = None
        n_part = 0
        # one zero fill serves the pick counters (added to with integer atomics) and the aux-loss scalar
        zeros = torch.zeros(E + 1 if balance else 1, dtype=torch.int32, device=dev)
        if balance:
            counts = zeros[:E]
            if aux_coef > 0:
                n_part = lib.picomoe_route_partials(T, E)
                partial = _empty((n_part, E), torch.float32, dev)
        _lib.check(
            lib.picomoe_route_fwd(
                _lib.ptr(logits), _lib.dtype_code(logits.dtype), T, E, top_k, _lib.ptr(bias_f32), int(bool(norm_topk)),
                _lib.ptr(idx), _lib.ptr(w), _lib.ptr(probs), _lib.ptr(counts), _lib.ptr(partial), _lib.stream_ptr(),
            ),
            "picomoe_route_fwd",
        )
        aux = zeros[-1:].view(torch.float32).reshape(())
        if balance and T > 0:
            _lib.check(
                lib.picomoe_balance(
                    _lib.ptr(counts), _lib.ptr(partial), n_part, T, E, top_k, float(aux_coef), float(bias_rate),
                    _lib.ptr(aux) if aux_coef > 0 else None, _lib.ptr(bias_f32) if bias_rate > 0 else None, _lib.stream_ptr(),
                ),
                "picomoe_balance",
            )
        ctx.save_for_backward(probs, idx, counts)
        ctx.cfg = (top_k, bool(norm_topk), float(aux_coef) if balance else 0.0, logits.dtype)
        ctx.mark_non_differentiable(idx)
        ctx.set_materialize_grads(False)   # no zero tensors for the outputs nobody differentiated (the indices, an unused aux)
        return idx, w, aux

    @staticmethod
    def backward(ctx, _d_idx, d_w, d_aux):
        probs, idx, counts = ctx.saved_tensors
        top_k, norm, aux_coef, dtype = ctx.cfg
        T, E = probs.shape
        lib = _lib.load()
        d_logits = _empty((T, E), dtype, probs.device)
        d_w = d_w.contiguous() if d_w is not None else None
        use_aux = aux_coef > 0 and d_aux is not None and counts is not None
        d_aux = d_aux.contiguous().float() if use_aux else None
        _lib.check(
            lib.picomoe_route_bwd(
                _lib.ptr(probs), _lib.ptr(idx), _lib.ptr(d_w), _lib.dtype_code(dtype), T, E, top_k, int(norm),
                _lib.ptr(d_aux), _lib.ptr(counts) if use_aux else None, aux_coef, _lib.ptr(d_logits), _lib.stream_ptr(),
            ),
            "picomoe_route_bwd",
        )
        return d_logits, None, None, None, None, None, None


GATE_DGRAD_MAX_EXPERTS = 16


def gate_dgrad_supported(tokens, weight):
    """Whether picomoe_gate_bwd takes this gate: up to 16 experts, fp32 or bf16 in one dtype, rows of whole 16-byte chunks."""
    return (tokens.is_cuda and tokens.dim() == 2 and weight.dim() == 2 and tokens.dtype == weight.dtype
            and tokens.dtype in (torch.float32, torch.bfloat16) and weight.shape[0] <= GATE_DGRAD_MAX_EXPERTS
            and (tokens.shape[1] * tokens.element_size()) % 16 == 0 and tokens.shape[1] <= 1 << 22
            and not torch.is_autocast_enabled())


def gate_bwd(d_logits, weight, addend, tokens, want_weight_grad):
    """(d_tokens, d_weight or None) of ``linear(tokens, weight)`` with ``addend`` (the tokens' gradient from their other
    readers, or None) summed in.  d_weight is None when it was not asked for or the kernel has no
    fused form for this many experts (the caller then runs the GEMM)."""
    lib = _lib.load()
    T, H = tokens.shape
    E = weight.shape[0]
    dt = _lib.dtype_code(tokens.dtype)
    d_logits, weight, tokens = d_logits.contiguous(), weight.contiguous(), tokens.contiguous()
    addend = addend.to(tokens.dtype).contiguous() if addend is not None else None
    d_tokens = _empty((T, H), tokens.dtype, tokens.device)
    ws_bytes = lib.picomoe_gate_bwd_workspace_bytes(dt, T, E, H) if want_weight_grad else 0
    if ws_bytes < 0:
        raise _lib.PicomoeError(f"picomoe_gate_bwd_workspace_bytes refused {T} tokens x {E} experts x {H}")
    d_weight = ws = None
    if ws_bytes > 0:
        d_weight = _empty((E, H), tokens.dtype, tokens.device)
        ws = _empty((ws_bytes,), torch.uint8, tokens.device)
    _lib.check(
        lib.picomoe_gate_bwd(_lib.ptr(d_logits), _lib.ptr(weight), _lib.ptr(addend), _lib.ptr(tokens) if d_weight is not None else None,
                             dt, T, E, H, _lib.ptr(d_tokens), _lib.ptr(d_weight), _lib.ptr(ws), ws_bytes, _lib.stream_ptr()),
        "picomoe_gate_bwd",
    )
    return d_tokens, d_weight


class _GateTap(torch.autograd.Function):
    """(logits, tokens) = (tokens @ weight.T, tokens): the router's gate Linear with the tokens handed through.

    Everything else that reads the tokens (dispatch, shared expert) reads the second output, so autograd delivers the sum
    of their gradients here together with d_logits, and one kernel writes d_tokens = that sum + d_logits @ weight (for up
    to 8 experts a second one sums d_weight = d_logits.T @ tokens from one read of the tokens) -- where an ``nn.Linear`` node beside the others costs a GEMM that
    writes [T, H], an add that reads two and writes one, and a GEMM with an E-row output that reads the tokens at a
    fraction of the memory rate.  The logits stay a library GEMM, as in the reference (expert_parallel.py:65, :174).
    """

    @staticmethod
    def forward(ctx, tokens, weight):
        ctx.save_for_backward(tokens, weight)
        ctx.set_materialize_grads(False)
        return torch.nn.functional.linear(tokens, weight), tokens

    @staticmethod
    def backward(ctx, d_logits, d_tap):
        tokens, weight = ctx.saved_tensors
        if d_logits is None:
            return (d_tap if ctx.needs_input_grad[0] else None), None
        d_tokens = d_weight = None
        if ctx.needs_input_grad[0]:
            d_tokens, d_weight = gate_bwd(d_logits, weight, d_tap, tokens, ctx.needs_input_grad[1])
        if ctx.needs_input_grad[1] and d_weight is None:
            d_weight = d_logits.t() @ tokens
        return d_tokens, d_weight


def gate_tap(tokens, weight):
    """Router logits and the tokens to hand to every other reader of them (see _GateTap); needs gate_dgrad_supported."""
    return _GateTap.apply(tokens, weight)


def route(logits, bias_f32, top_k, norm_topk, balance=False, aux_coef=0.0, bias_rate=0.0):
    """Returns (topk_idx int64 [T,k], topk_w [T,k] in logits.dtype, aux fp32 scalar)."""
    return _Route.apply(logits, bias_f32, top_k, norm_topk, balance, aux_coef, bias_rate)


# ------------------------------------------------------------------------------------------------
# Permutation plan
# ------------------------------------------------------------------------------------------------
@dataclass
class Plan:
    """Result of the stable counting sort of routed rows by expert (see include/picomoe.h)."""

    order: torch.Tensor        # int32 [R]  row at each sorted position (-1 past the kept rows)
    inv_order: torch.Tensor    # int32 [R]  sorted position of each row (-1 = dropped)
    counts: torch.Tensor       # int64 [E]  rows per expert before any capacity limit
    kept_counts: torch.Tensor  # int64 [E]  rows per expert in this plan's layout
    within: Optional[torch.Tensor] = None  # int32 [R] rank of a row inside its expert
    capacity: int = 0


def permute_plan(expert_idx, num_experts, capacity=0, round_index=0, want_within=False, static_scratch=False):
    """``static_scratch``: run the plan on the library's fixed 1 MiB scratch array (``picomoe_permute_plan_static``: no
    workspace tensor) instead of a workspace allocated here; inputs too large for it are refused."""
    _lib.require_cuda(expert_idx)
    lib = _lib.load()
    expert_idx = expert_idx.contiguous().to(torch.int64)
    R = expert_idx.numel()
    dev = expert_idx.device
    order = _empty((R,), torch.int32, dev)
    inv = _empty((R,), torch.int32, dev)
    counts = _empty((num_experts,), torch.int64, dev)
    kept = _empty((num_experts,), torch.int64, dev)
    within = _empty((R,), torch.int32, dev) if want_within else None
    ws_bytes = lib.picomoe_permute_workspace_bytes(R, num_experts)
    if ws_bytes < 0:
        raise _lib.PicomoeError(f"permute plan: unsupported size (rows={R}, experts={num_experts})")
    if static_scratch:
        with torch.cuda.device(dev):  # the library looks its scratch array up on the current device
            _lib.check(
                lib.picomoe_permute_plan_static(
                    _lib.ptr(expert_idx), R, num_experts, int(capacity), int(round_index), _lib.ptr(order), _lib.ptr(inv),
                    _lib.ptr(counts), _lib.ptr(kept), _lib.ptr(within), _lib.stream_ptr(),
                ),
                "picomoe_permute_plan_static",
            )
        return Plan(order, inv, counts, kept, within, int(capacity))
    ws = _empty((max(ws_bytes, 4),), torch.uint8, dev)
    _lib.check(
        lib.picomoe_permute_plan(
            _lib.ptr(expert_idx), R, num_experts, int(capacity), int(round_index), _lib.ptr(order), _lib.ptr(inv),
            _lib.ptr(counts), _lib.ptr(kept), _lib.ptr(within), _lib.ptr(ws), _lib.stream_ptr(),
        ),
        "picomoe_permute_plan",
    )
    return Plan(order, inv, counts, kept, within, int(capacity))


# ------------------------------------------------------------------------------------------------
# Row movers
# ------------------------------------------------------------------------------------------------
def gather_rows(src, row_map, div, n_out):
    lib = _lib.load()
    src = src.contiguous()
    out = _empty((n_out, src.shape[1]), src.dtype, src.device)
    _lib.check(
        lib.picomoe_gather_rows(_lib.ptr(src), _lib.ptr(row_map), int(div), n_out, src.shape[1], _lib.dtype_code(src.dtype),
                                _lib.ptr(out), _lib.stream_ptr()),
        "picomoe_gather_rows",
    )
    return out


def _weights_like(weights, y):
    """Gate weights in the dtype of the rows they scale: the combine kernels read both as one element type (a bf16
    weight buffer read as fp32 would be read past its end).  The reference casts the same way
    (expert_parallel.py:184, capacity_moe.py:158)."""
    if weights is None:
        return None
    if not weights.is_floating_point():
        raise _lib.PicomoeError(f"combine: gate weights must be floating point, got {weights.dtype}")
    return weights.to(y.dtype).contiguous()


def combine_rows(y, inv_order, weights, n_tokens, top_k):
    lib = _lib.load()
    y = y.contiguous()
    weights = _weights_like(weights, y)
    if weights is not None and weights.numel() != n_tokens * top_k:
        raise _lib.PicomoeError(f"combine: {weights.numel()} gate weights for {n_tokens} tokens x top-{top_k}")
    out = _empty((n_tokens, y.shape[1]), y.dtype, y.device)
    _lib.check(
        lib.picomoe_combine_fwd(_lib.ptr(y), _lib.ptr(inv_order), _lib.ptr(weights), n_tokens, top_k, y.shape[1],
                                _lib.dtype_code(y.dtype), _lib.ptr(out), _lib.stream_ptr()),
        "picomoe_combine_fwd",
    )
    return out


class _ExpandPermute(torch.autograd.Function):
    """out[pos] = src[order[pos] // div]  (token-major expansion and the sort by expert in one gather).
    Backward: d_src[t] = sum_j d_out[inv_order[t*div + j]] -- a gather-sum, no atomics."""

    @staticmethod
    def forward(ctx, src, order, inv_order, div, n_out):
        _lib.require_cuda(src)
        ctx.save_for_backward(inv_order)
        ctx.meta = (src.shape[0], div)
        return gather_rows(src, order, div, n_out)

    @staticmethod
    def backward(ctx, d_out):
        (inv_order,) = ctx.saved_tensors
        n_src, div = ctx.meta
        return combine_rows(d_out, inv_order, None, n_src, div), None, None, None, None


def expand_permute(src, order, inv_order, div, n_out):
    return _ExpandPermute.apply(src, order, inv_order, div, n_out)


class _DispatchFp8(torch.autograd.Function):
    """x_sorted[inv_order[t*k + j]] = dequantise(quantise(tokens[t])) in one pass over the tokens (FP8 E4M3, one scale per
    token), optionally with the codes and scales in the same sorted order.  Backward: straight through the quantiser,
    then the gather-sum of the expand + permute: d_tokens[t] = sum_j d_x_sorted[inv_order[t*k + j]]."""

    @staticmethod
    def forward(ctx, tokens, inv_order, top_k, n_out, with_codes):
        _lib.require_cuda(tokens, inv_order)
        lib = _lib.load()
        tokens = tokens.contiguous()
        T, H = tokens.shape
        # every position is written when nothing is dropped; under a capacity window the unkept tail must not hold garbage
        x_sorted = _empty((n_out, H), tokens.dtype, tokens.device)
        q_sorted = _empty((n_out, H), torch.uint8, tokens.device) if with_codes else None
        scale_sorted = _empty((n_out,), torch.float32, tokens.device) if with_codes else None
        _lib.check(
            lib.picomoe_dispatch_fp8(_lib.ptr(tokens), _lib.dtype_code(tokens.dtype), T, H, _lib.ptr(inv_order), int(top_k), n_out,
                                     _lib.ptr(x_sorted), _lib.ptr(q_sorted), _lib.ptr(scale_sorted), None, None, _lib.stream_ptr()),
            "picomoe_dispatch_fp8",
        )
        ctx.save_for_backward(inv_order)
        ctx.meta = (T, int(top_k))
        if with_codes:
            ctx.mark_non_differentiable(q_sorted, scale_sorted)
            return x_sorted, q_sorted, scale_sorted
        return x_sorted, None, None

    @staticmethod
    def backward(ctx, d_x_sorted, _d_q, _d_scale):
        (inv_order,) = ctx.saved_tensors
        n_tokens, top_k = ctx.meta
        return combine_rows(d_x_sorted, inv_order, None, n_tokens, top_k), None, None, None, None


def dispatch_fp8(tokens, inv_order, top_k, n_out, with_codes=False):
    """(x_sorted, q_sorted or None, scale_sorted or None): the FP8 dispatch of one rank fused with expand + permute."""
    return _DispatchFp8.apply(tokens, inv_order, top_k, n_out, with_codes)


class _UnpermuteCombine(torch.autograd.Function):
    """out[t] = sum_j w[t,j] * y[inv_order[t*k+j]] over kept rows (w None: k = 1 plain un-permute)."""

    @staticmethod
    def forward(ctx, y, weights, inv_order, order, n_tokens, top_k, zero_fill):
        _lib.require_cuda(y)
        w_dtype = weights.dtype if weights is not None else None
        y = y.contiguous()
        weights = _weights_like(weights, y)  # the kernels read weights and rows as one element type
        ctx.save_for_backward(y, weights, inv_order, order)
        ctx.meta = (n_tokens, top_k, zero_fill, w_dtype)
        return combine_rows(y, inv_order, weights, n_tokens, top_k)

    @staticmethod
    def backward(ctx, d_out):
        y, weights, inv_order, order = ctx.saved_tensors
        n_tokens, top_k, zero_fill, w_dtype = ctx.meta
        d_out = d_out.to(y.dtype).contiguous()
        if weights is None:
            return gather_rows(d_out, order, 1, y.shape[0]), None, None, None, None, None, None
        lib = _lib.load()
        d_y = (torch.zeros if zero_fill else torch.empty)(y.shape, dtype=y.dtype, device=y.device)
        d_w = _empty(weights.shape, weights.dtype, weights.device)
        _lib.check(
            lib.picomoe_combine_bwd(_lib.ptr(d_out), _lib.ptr(y), _lib.ptr(inv_order), _lib.ptr(weights), n_tokens, top_k,
                                    y.shape[1], _lib.dtype_code(y.dtype), _lib.ptr(d_y), _lib.ptr(d_w), _lib.stream_ptr()),
            "picomoe_combine_bwd",
        )
        return d_y, d_w.to(w_dtype), None, None, None, None, None


def unpermute_combine(y, weights, inv_order, order, n_tokens, top_k, zero_fill=False):
    return _UnpermuteCombine.apply(y, weights, inv_order, order, n_tokens, top_k, zero_fill)
