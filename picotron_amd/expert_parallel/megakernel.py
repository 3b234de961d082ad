"""Expert FFN (grouped SwiGLU GEMMs) on hand-written gfx950 kernels.

Same public surface as picotron/expert_parallel/megakernel.py: ``fused_moe`` (:403),
``fused_moe_forward`` (:294), ``fused_moe_dgrad`` (:332), ``fused_moe_wgrad`` (:350),
``fused_moe_backward`` (:360), ``torch_fused_ffn`` (:308), ``torch_moe_backward`` (:321),
``cuda_available`` (:408).  ``x_sorted [N,H]`` holds rows grouped by expert, ``counts [E]`` is a device
tensor read by the kernels (no host copy, no block schedule built on the host), ``gate_w/up_w [E,I,H]``,
``down_w [E,H,I]``.

Differences in mechanism, not in results: gate and up are consumed in place (no ``cat`` into w13), SwiGLU
is the epilogue of the gate/up GEMM, silu-mul-backward is the epilogue of the ``dy @ down_w`` GEMM, and the
autograd path keeps ``[g|u]`` from the forward instead of recomputing it.
"""

import collections
import warnings

import torch
import torch.nn.functional as F

from picotron_amd import _lib


def cuda_available():
    """Whether the HIP kernels can run: a GPU is visible and libpicomoe.so loads."""
    if not torch.cuda.is_available():
        return False
    _lib.load()
    return True


def _counts64(counts, device):
    if not torch.is_tensor(counts):
        counts = torch.tensor(list(counts), dtype=torch.int64, device=device)
    return counts.to(device=device, dtype=torch.int64).contiguous()


_FAMILY_NAMES = {0: "generic", 1: "bf16_mfma", 2: "f32_mfma"}
_warned_generic = set()


def kernel_family(dtype, hidden, inter):
    """Which kernels the expert FFN runs for this dtype and these widths: "bf16_mfma" (bf16, multiples of 64, >= 128),
    "f32_mfma" (fp32, multiples of 4, >= 32) or "generic" (scalar-FMA tiles: any shape, far slower)."""
    return _FAMILY_NAMES[_lib.load().picomoe_ffn_kernel_family(_lib.dtype_code(dtype), int(hidden), int(inter))]


def _check_weights(x, gate_w, up_w, down_w):
    E, I, H = gate_w.shape
    if up_w.shape != (E, I, H) or down_w.shape != (E, H, I) or x.shape[1] != H:
        raise _lib.PicomoeError(f"fused_moe: shapes x{tuple(x.shape)} gate{tuple(gate_w.shape)} up{tuple(up_w.shape)} down{tuple(down_w.shape)}")
    if not (x.dtype == gate_w.dtype == up_w.dtype == down_w.dtype):
        raise _lib.PicomoeError("fused_moe: x and the weights must share one dtype")
    key = (x.dtype, H, I)
    if key not in _warned_generic and kernel_family(*key) == "generic":
        _warned_generic.add(key)   # once per shape: the results are the same, only the speed is not
        warnings.warn(
            f"picotron_amd: expert FFN with hidden {H}, FFN {I}, {x.dtype} runs the generic scalar-FMA kernels, not the "
            "matrix pipes (bf16 needs both widths to be multiples of 64 and >= 128, fp32 multiples of 4 and >= 32)",
            RuntimeWarning, stacklevel=3)
    return E, I, H


def _gate_up(x, counts, gate_w, up_w, keep_inter13):
    lib = _lib.load()
    E, I, H = gate_w.shape
    N = x.shape[0]
    act = torch.empty((N, I), dtype=x.dtype, device=x.device)
    inter13 = torch.empty((N, 2 * I), dtype=x.dtype, device=x.device) if keep_inter13 else None
    ws = _ffn_workspace(x.device) if x.dtype == torch.bfloat16 else None
    _lib.check(
        lib.picomoe_ffn_gate_up(_lib.ptr(x), _lib.ptr(counts), E, N, H, I, _lib.ptr(gate_w), _lib.ptr(up_w),
                                _lib.dtype_code(x.dtype), _lib.ptr(act), _lib.ptr(inter13), _lib.ptr(ws),
                                ws.numel() if ws is not None else 0, _lib.stream_ptr()),
        "picomoe_ffn_gate_up",
    )
    return act, inter13


def fp8_gemm_supported(hidden, inter):
    """Shapes the FP8 MFMA gate/up kernel tiles (everything else runs the bf16 kernels on the dequantised rows)."""
    return hidden % 256 == 0 and inter % 128 == 0


def quantize_expert_weights(w):
    """w [E, I, H] bf16/fp32 -> (E4M3 codes uint8 [E, I, H], fp32 scale [E * I]): every output row gets the scale
    amax / 448 of the FP8 dispatch quantiser (``_per_token_quant_fp8``), with the same kernel."""
    lib = _lib.load()
    _lib.require_cuda(w)
    w = w.contiguous()
    E, I, H = w.shape
    q = torch.empty((E, I, H), dtype=torch.uint8, device=w.device)
    scale = torch.empty((E * I,), dtype=torch.float32, device=w.device)
    _lib.check(
        lib.picomoe_fp8_quant(_lib.ptr(w), _lib.dtype_code(w.dtype), E * I, H, _lib.ptr(q), _lib.ptr(scale), _lib.stream_ptr()),
        "picomoe_fp8_quant",
    )
    return q, scale


def _gate_up_fp8(xq, x_scale, counts, gate_q, gate_scale, up_q, up_scale, keep_inter13, dtype=torch.bfloat16):
    """gate/up GEMM + SwiGLU on FP8 MFMA: xq [N,H] E4M3 codes + x_scale [N]; weights as ``quantize_expert_weights``."""
    lib = _lib.load()
    E, I, H = gate_q.shape
    N = xq.shape[0]
    act = torch.empty((N, I), dtype=dtype, device=xq.device)
    inter13 = torch.empty((N, 2 * I), dtype=dtype, device=xq.device) if keep_inter13 else None
    _lib.check(
        lib.picomoe_ffn_gate_up_fp8(_lib.ptr(xq), _lib.ptr(x_scale), _lib.ptr(counts), E, N, H, I, _lib.ptr(gate_q),
                                    _lib.ptr(up_q), _lib.ptr(gate_scale), _lib.ptr(up_scale), _lib.ptr(act),
                                    _lib.ptr(inter13), _lib.stream_ptr()),
        "picomoe_ffn_gate_up_fp8",
    )
    return act, inter13


def _quantize_rows(x):
    """x [N, D] bf16 -> (E4M3 codes uint8 [N, D], fp32 scale [N]) with the FP8 dispatch quantiser."""
    lib = _lib.load()
    N, D = x.shape
    q = torch.empty((N, D), dtype=torch.uint8, device=x.device)
    scale = torch.empty((N,), dtype=torch.float32, device=x.device)
    _lib.check(
        lib.picomoe_fp8_quant(_lib.ptr(x), _lib.dtype_code(x.dtype), N, D, _lib.ptr(q), _lib.ptr(scale), _lib.stream_ptr()),
        "picomoe_fp8_quant",
    )
    return q, scale


def _down_fp8(act, counts, down_q, down_scale, row_weight):
    """down GEMM on FP8 MFMA: the SwiGLU output ``act`` [N, I] bf16 is quantised per row here (one more pass over it),
    ``down_q [E, H, I]`` / ``down_scale [E * H]`` as ``quantize_expert_weights(down_w)``."""
    lib = _lib.load()
    E, H, I = down_q.shape
    N = act.shape[0]
    aq, a_scale = _quantize_rows(act)
    y = torch.empty((N, H), dtype=act.dtype, device=act.device)
    _lib.check(
        lib.picomoe_ffn_down_fp8(_lib.ptr(aq), _lib.ptr(a_scale), _lib.ptr(counts), E, N, H, I, _lib.ptr(down_q),
                                 _lib.ptr(down_scale), _lib.ptr(row_weight), _lib.ptr(y), _lib.stream_ptr()),
        "picomoe_ffn_down_fp8",
    )
    return y


_workspaces = collections.OrderedDict()
_MAX_WORKSPACES = 4


def _ffn_workspace(device):
    """Scratch for the split last round of the row-grouped kernels (picomoe_ffn_workspace_bytes, 64 MB): one buffer
    per device and stream, allocated on first use -- kernels of one stream run one after the other, so they can share it.
    At most ``_MAX_WORKSPACES`` buffers are kept; when a further stream asks for one, the least recently used goes back
    to the caching allocator, which hands it out again only on the stream it was allocated and used on, i.e. in order
    behind the kernels that still read it."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None:
        while len(_workspaces) >= _MAX_WORKSPACES:
            _workspaces.popitem(last=False)
        ws = torch.empty(_lib.load().picomoe_ffn_workspace_bytes(), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    else:
        _workspaces.move_to_end(key)
    return ws


def release_workspaces():
    """Drops every cached split-round workspace (64 MB per device and stream that has run an expert FFN)."""
    _workspaces.clear()


def _down(act, counts, down_w, row_weight):
    lib = _lib.load()
    E, H, I = down_w.shape
    N = act.shape[0]
    y = torch.empty((N, H), dtype=act.dtype, device=act.device)
    ws = _ffn_workspace(act.device) if act.dtype == torch.bfloat16 else None
    _lib.check(
        lib.picomoe_ffn_down(_lib.ptr(act), _lib.ptr(counts), E, N, H, I, _lib.ptr(down_w), _lib.ptr(row_weight),
                             _lib.dtype_code(act.dtype), _lib.ptr(y), _lib.ptr(ws), ws.numel() if ws is not None else 0,
                             _lib.stream_ptr()),
        "picomoe_ffn_down",
    )
    return y


def _dgrad_act(dy, counts, down_w, inter13, want_act):
    lib = _lib.load()
    E, H, I = down_w.shape
    N = dy.shape[0]
    d13 = torch.empty((N, 2 * I), dtype=dy.dtype, device=dy.device)
    act = torch.empty((N, I), dtype=dy.dtype, device=dy.device) if want_act else None
    ws = _ffn_workspace(dy.device) if dy.dtype == torch.bfloat16 else None
    _lib.check(
        lib.picomoe_ffn_dgrad_act(_lib.ptr(dy), _lib.ptr(counts), E, N, H, I, _lib.ptr(down_w), _lib.ptr(inter13),
                                  _lib.dtype_code(dy.dtype), _lib.ptr(d13), _lib.ptr(act), _lib.ptr(ws),
                                  ws.numel() if ws is not None else 0, _lib.stream_ptr()),
        "picomoe_ffn_dgrad_act",
    )
    return d13, act


def _dgrad_x(d13, counts, gate_w, up_w):
    lib = _lib.load()
    E, I, H = gate_w.shape
    N = d13.shape[0]
    dx = torch.empty((N, H), dtype=d13.dtype, device=d13.device)
    ws = _ffn_workspace(d13.device) if d13.dtype == torch.bfloat16 else None
    _lib.check(
        lib.picomoe_ffn_dgrad_x(_lib.ptr(d13), _lib.ptr(counts), E, N, H, I, _lib.ptr(gate_w), _lib.ptr(up_w),
                                _lib.dtype_code(d13.dtype), _lib.ptr(dx), _lib.ptr(ws), ws.numel() if ws is not None else 0,
                                _lib.stream_ptr()),
        "picomoe_ffn_dgrad_x",
    )
    return dx


def _wgrad(lhs, ld_lhs, rhs, ld_rhs, counts, E, N, P, Q, dtype, device, lhs_offset=0, which=None):
    """out [E, P, Q] = per expert lhs_e^T @ rhs_e.  ``which`` ("down", "gate", "up", "gate_up") names the weight gradient for
    timing hooks; it does not change the call."""
    lib = _lib.load()
    out = torch.empty((E, P, Q), dtype=dtype, device=device)
    lhs_ptr = _lib.ctypes.c_void_p(lhs.data_ptr() + lhs_offset * lhs.element_size())
    _lib.check(
        lib.picomoe_ffn_wgrad(lhs_ptr, ld_lhs, _lib.ptr(rhs), ld_rhs, _lib.ptr(counts), E, N, P, Q, _lib.dtype_code(dtype),
                              _lib.ptr(out), _lib.stream_ptr()),
        "picomoe_ffn_wgrad",
    )
    return out


def _prep(x_sorted, counts, *weights):
    _lib.require_cuda(x_sorted, *weights)
    return x_sorted.contiguous(), _counts64(counts, x_sorted.device), [w.contiguous() for w in weights]


def fused_moe_forward(x_sorted, counts, gate_w, up_w, down_w, row_weight=None):
    """x_sorted [N,H] (rows grouped by expert); gate_w/up_w [E,I,H]; down_w [E,H,I]; counts [E]."""
    x, counts, (gw, uw, dw) = _prep(x_sorted, counts, gate_w, up_w, down_w)
    _check_weights(x, gw, uw, dw)
    if x.shape[0] == 0:
        return torch.empty((0, x.shape[1]), device=x.device, dtype=x.dtype)
    act, _ = _gate_up(x, counts, gw, uw, keep_inter13=False)
    rw = row_weight.to(x.dtype).contiguous() if row_weight is not None else None
    return _down(act, counts, dw, rw)


def fused_moe_dgrad(x_sorted, counts, gate_w, up_w, down_w, dy):
    """Explicit input-grad.  Returns (dx, a, d_inter13); ``a`` / ``d_inter13`` feed ``fused_moe_wgrad``.
    Stateless like the reference: the forward intermediates are rebuilt here."""
    x, counts, (gw, uw, dw) = _prep(x_sorted, counts, gate_w, up_w, down_w)
    dy = dy.contiguous()
    act, inter13 = _gate_up(x, counts, gw, uw, keep_inter13=True)
    d13, _ = _dgrad_act(dy, counts, dw, inter13, want_act=False)
    dx = _dgrad_x(d13, counts, gw, uw)
    return dx, act, d13


def fused_moe_wgrad(x_sorted, counts, a, d_inter13, dy):
    """Explicit weight-grads from the forward intermediates.  Returns (d_gate, d_up, d_down)."""
    _lib.require_cuda(x_sorted, a, d_inter13, dy)
    x, a, d13, dy = x_sorted.contiguous(), a.contiguous(), d_inter13.contiguous(), dy.contiguous()
    counts = _counts64(counts, x.device)
    E, N, H, I = counts.numel(), x.shape[0], x.shape[1], a.shape[1]
    d_down = _wgrad(dy, H, a, I, counts, E, N, H, I, x.dtype, x.device, which="down")
    d_gate = _wgrad(d13, 2 * I, x, H, counts, E, N, I, H, x.dtype, x.device, which="gate")
    d_up = _wgrad(d13, 2 * I, x, H, counts, E, N, I, H, x.dtype, x.device, lhs_offset=I, which="up")
    return d_gate, d_up, d_down


def fused_moe_backward(x_sorted, counts, gate_w, up_w, down_w, dy):
    """(dx, d_gate, d_up, d_down) with explicit dgrad + wgrad kernels."""
    if x_sorted.shape[0] == 0:
        return (torch.zeros_like(x_sorted), torch.zeros_like(gate_w), torch.zeros_like(up_w), torch.zeros_like(down_w))
    dx, a, d13 = fused_moe_dgrad(x_sorted, counts, gate_w, up_w, down_w, dy)
    d_gate, d_up, d_down = fused_moe_wgrad(x_sorted, counts, a, d13, dy)
    return dx, d_gate, d_up, d_down


class _FusedMoE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x_sorted, gate_w, up_w, down_w, counts, row_weight, fp8=None):
        x, counts, (gw, uw, dw) = _prep(x_sorted, counts, gate_w, up_w, down_w)
        _check_weights(x, gw, uw, dw)
        ctx.counts = counts
        ctx.has_rw = row_weight is not None
        if x.shape[0] == 0:
            ctx.empty = True
            ctx.save_for_backward(x, gw, uw, dw)
            return torch.empty((0, x.shape[1]), device=x.device, dtype=x.dtype)
        ctx.empty = False
        needs_grad = any(ctx.needs_input_grad[:4]) or (ctx.has_rw and ctx.needs_input_grad[5])
        down_fp8 = None
        if fp8 is not None:
            # forward gate/up on FP8 MFMA from the dispatch's codes; the backward below is the bf16 one on x_sorted
            xq, x_scale, gate_q, gate_scale, up_q, up_scale = fp8[:6]
            down_fp8 = fp8[6:8] if len(fp8) >= 8 else None
            act, inter13 = _gate_up_fp8(xq.contiguous(), x_scale.contiguous(), counts, gate_q, gate_scale, up_q, up_scale,
                                        keep_inter13=needs_grad, dtype=x.dtype)
        else:
            act, inter13 = _gate_up(x, counts, gw, uw, keep_inter13=needs_grad)
        rw = row_weight.to(x.dtype).contiguous() if ctx.has_rw else None
        y = _down_fp8(act, counts, down_fp8[0], down_fp8[1], rw) if down_fp8 is not None else _down(act, counts, dw, rw)
        if needs_grad:
            ctx.save_for_backward(x, gw, uw, dw, act, inter13, rw)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        if ctx.empty:
            x, gw, uw, dw = ctx.saved_tensors
            return torch.zeros_like(x), torch.zeros_like(gw), torch.zeros_like(uw), torch.zeros_like(dw), None, None, None
        x, gw, uw, dw, act, inter13, rw = ctx.saved_tensors
        counts = ctx.counts
        dy = grad_y.contiguous()
        d_rw = None
        if rw is not None:
            # y = y0 * rw: d_rw = <dy, y0>, d_y0 = dy * rw  (y0 rebuilt by one more down GEMM)
            y0 = _down(act, counts, dw, None)
            d_rw = (dy.float() * y0.float()).sum(dim=1).to(rw.dtype)
            dy = dy * rw[:, None]
        # only the GEMMs whose results autograd asked for (frozen experts, or an input that needs no gradient, skip theirs)
        want_dx, want_gate, want_up, want_down = ctx.needs_input_grad[:4]
        E, N, H, I = counts.numel(), x.shape[0], x.shape[1], act.shape[1]
        dx = d_gate = d_up = d_down = None
        if want_dx or want_gate or want_up:
            d13, _ = _dgrad_act(dy, counts, dw, inter13, want_act=False)
            if want_dx:
                dx = _dgrad_x(d13, counts, gw, uw)
        if want_down:
            d_down = _wgrad(dy, H, act, I, counts, E, N, H, I, x.dtype, x.device, which="down")
        if want_gate and want_up:
            # one launch for both: [dg | du] is the left operand as it lies (2I columns), the result [E, 2I, H] holds
            # d gate_w[e] and d up_w[e] one after the other, and each expert's slice of either is contiguous
            d_gu = _wgrad(d13, 2 * I, x, H, counts, E, N, 2 * I, H, x.dtype, x.device, which="gate_up")
            d_gate, d_up = d_gu[:, :I], d_gu[:, I:]
        elif want_gate:
            d_gate = _wgrad(d13, 2 * I, x, H, counts, E, N, I, H, x.dtype, x.device, which="gate")
        elif want_up:
            d_up = _wgrad(d13, 2 * I, x, H, counts, E, N, I, H, x.dtype, x.device, lhs_offset=I, which="up")
        return dx, d_gate, d_up, d_down, None, d_rw, None


def fused_moe(x_sorted, counts, gate_w, up_w, down_w, row_weight=None, fp8=None):
    """Differentiable fused MoE expert FFN.  counts [E] = per-expert row counts.

    ``fp8`` (optional, not in the reference): ``(xq [N,H] E4M3 codes, x_scale [N], gate_q, gate_scale, up_q,
    up_scale[, down_q, down_scale])`` -- the rows of ``x_sorted`` as the FP8 dispatch ships them and the weights from
    ``quantize_expert_weights``; the forward gate/up GEMM then runs on FP8 MFMA and, when the down weights are given
    too, so does the forward down GEMM (on the SwiGLU output quantised per row); the backward stays bf16."""
    return _FusedMoE.apply(x_sorted, gate_w, up_w, down_w, counts, row_weight, fp8)


def torch_fused_ffn(x_sorted, counts, gate_w, up_w, down_w, row_weight):
    """Per-expert loop over library matmuls, kept because the reference exposes it by name
    (megakernel.py:308-318).  Nothing in this package dispatches to it."""
    outs, offset = [], 0
    for e, n in enumerate(counts.tolist()):
        x = x_sorted[offset : offset + n]
        outs.append((F.silu(x @ gate_w[e].T) * (x @ up_w[e].T)) @ down_w[e].T)
        offset += n
    y = torch.cat(outs, dim=0) if outs else x_sorted.new_empty((0, x_sorted.shape[1]))
    return y * row_weight[:, None] if row_weight is not None else y


def torch_moe_backward(x_sorted, counts, gate_w, up_w, down_w, dy):
    """Autograd over ``torch_fused_ffn`` (megakernel.py:321-329); exposed by name only, never dispatched to."""
    with torch.enable_grad():
        leaves = [t.detach().requires_grad_(True) for t in (x_sorted, gate_w, up_w, down_w)]
        y = torch_fused_ffn(leaves[0], counts, leaves[1], leaves[2], leaves[3], None)
        return torch.autograd.grad(y, leaves, dy)
