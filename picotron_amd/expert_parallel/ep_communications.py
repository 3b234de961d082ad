"""FP8 E4M3 dispatch quantise / dequantise on the GPU.

Mirrors the per-token FP8 cast of the reference (picotron/expert_parallel/ep_communications.py:59-68
``_per_token_quant_fp8`` and the dequantise expression at :100).  The reference's all-to-all wrappers
in the same file only run with more than one expert-parallel rank and have no counterpart here.
"""

import torch

from picotron_amd import _lib

_FP8_E4M3_MAX = 448.0


def _per_token_quant_fp8(x):
    """Cast rows of ``x`` [N,H] to float8_e4m3fn with a per-row scale.  Returns (fp8 [N,H], scale fp32 [N])."""
    _lib.require_cuda(x)
    x = x.contiguous()
    n, h = x.shape
    q = torch.empty((n, h), dtype=torch.uint8, device=x.device)
    scale = torch.empty((n,), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    _lib.check(
        lib.picomoe_fp8_quant(_lib.ptr(x), _lib.dtype_code(x.dtype), n, h, _lib.ptr(q), _lib.ptr(scale), _lib.stream_ptr()),
        "picomoe_fp8_quant",
    )
    return q.view(torch.float8_e4m3fn), scale


def _dequant_fp8(q, scale, dtype):
    """``q.to(dtype) * scale[:, None].to(dtype)`` in one pass."""
    _lib.require_cuda(q, scale)
    q = q.contiguous()
    n, h = q.shape
    out = torch.empty((n, h), dtype=dtype, device=q.device)
    lib = _lib.load()
    _lib.check(
        lib.picomoe_fp8_dequant(
            _lib.ptr(q.view(torch.uint8)), _lib.ptr(scale.contiguous()), n, h, _lib.ptr(out), _lib.dtype_code(dtype), _lib.stream_ptr()
        ),
        "picomoe_fp8_dequant",
    )
    return out


class _Fp8RoundTrip(torch.autograd.Function):
    """quantise -> dequantise with a straight-through gradient (what the reference's FP8 dispatch
    does to the rows it ships, ep_communications.py:82-113, minus the exchange)."""

    @staticmethod
    def forward(ctx, x):
        q, scale = _per_token_quant_fp8(x)
        ctx.mark_non_differentiable(q, scale)
        return _dequant_fp8(q, scale, x.dtype), q, scale

    @staticmethod
    def backward(ctx, grad_out, _grad_q, _grad_scale):
        return grad_out


def fp8_round_trip(x, with_codes=False):
    """dequantise(quantise(x)) with a straight-through gradient; ``with_codes`` also returns the E4M3 codes and the
    per-row scales the dequantised rows were built from (for the FP8 GEMM)."""
    out, q, scale = _Fp8RoundTrip.apply(x)
    return (out, q, scale) if with_codes else out
