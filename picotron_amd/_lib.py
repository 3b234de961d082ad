"""ctypes binding of ``libpicomoe.so`` (the C-ABI library of gfx950 kernels).

There is no fallback: if the library has not been built, or a call returns a non-zero code, this
module raises.  Build with ``make -C picotron_amd/csrc`` (or ``__graft_entry__.build()``).
"""

import ctypes
import os

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libpicomoe.so")
HEADER_PATH = os.path.join(os.path.dirname(_PKG_DIR), "include", "picomoe.h")
ABI_VERSION = 6

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_p, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float

# name -> argtypes (every entry point returns int unless listed in _RESTYPES)
_SIGNATURES = {
    "picomoe_abi_version": [],
    "picomoe_error_string": [_i32],
    "picomoe_fp8_quant": [_p, _i32, _i64, _i64, _p, _p, _p],
    "picomoe_fp8_dequant": [_p, _p, _i64, _i64, _p, _i32, _p],
    "picomoe_dispatch_fp8": [_p, _i32, _i64, _i64, _p, _i32, _i64, _p, _p, _p, _p, _p, _p],
    "picomoe_route_partials": [_i64, _i32],
    "picomoe_route_fwd": [_p, _i32, _i64, _i32, _i32, _p, _i32, _p, _p, _p, _p, _p, _p],
    "picomoe_route_bwd": [_p, _p, _p, _i32, _i64, _i32, _i32, _i32, _p, _p, _f32, _p, _p],
    "picomoe_balance": [_p, _p, _i32, _i64, _i32, _i32, _f32, _f32, _p, _p, _p],
    "picomoe_gate_bwd_workspace_bytes": [_i32, _i64, _i32, _i64],
    "picomoe_gate_bwd": [_p, _p, _p, _p, _i32, _i64, _i32, _i64, _p, _p, _p, _i64, _p],
    "picomoe_permute_workspace_bytes": [_i64, _i32],
    "picomoe_permute_plan": [_p, _i64, _i32, _i64, _i64, _p, _p, _p, _p, _p, _p, _p],
    "picomoe_permute_plan_static_max_bytes": [],
    "picomoe_permute_plan_static_init": [],
    "picomoe_permute_plan_static": [_p, _i64, _i32, _i64, _i64, _p, _p, _p, _p, _p, _p],
    "picomoe_gather_rows": [_p, _p, _i32, _i64, _i64, _i32, _p, _p],
    "picomoe_combine_fwd": [_p, _p, _p, _i64, _i32, _i64, _i32, _p, _p],
    "picomoe_combine_bwd": [_p, _p, _p, _p, _i64, _i32, _i64, _i32, _p, _p, _p],
    "picomoe_ffn_gate_up": [_p, _p, _i32, _i64, _i64, _i64, _p, _p, _i32, _p, _p, _p, _i64, _p],
    "picomoe_ffn_gate_up_fp8": [_p, _p, _p, _i32, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p, _p],
    "picomoe_ffn_down_fp8": [_p, _p, _p, _i32, _i64, _i64, _i64, _p, _p, _p, _p, _p],
    "picomoe_ffn_down": [_p, _p, _i32, _i64, _i64, _i64, _p, _p, _i32, _p, _p, _i64, _p],
    "picomoe_ffn_dgrad_act": [_p, _p, _i32, _i64, _i64, _i64, _p, _p, _i32, _p, _p, _p, _i64, _p],
    "picomoe_ffn_dgrad_x": [_p, _p, _i32, _i64, _i64, _i64, _p, _p, _i32, _p, _p, _i64, _p],
    "picomoe_ffn_workspace_bytes": [],
    "picomoe_ffn_kernel_family": [_i32, _i64, _i64],
    "picomoe_ffn_wgrad": [_p, _i64, _p, _i64, _p, _i32, _i64, _i64, _i64, _i32, _p, _p],
    "picomoe_diag_mfma_loop_flop": [_i32, _i64, _i32],
    "picomoe_diag_mfma_loop": [_p, _i64, _i32, _i64, _i64, _i64, _i32, _p, _p],
}
_RESTYPES = {"picomoe_error_string": ctypes.c_char_p, "picomoe_permute_workspace_bytes": ctypes.c_int64,
             "picomoe_permute_plan_static_max_bytes": ctypes.c_int64,
             "picomoe_ffn_workspace_bytes": ctypes.c_int64, "picomoe_gate_bwd_workspace_bytes": ctypes.c_int64, "picomoe_diag_mfma_loop_flop": ctypes.c_int64}

_lib = None


class PicomoeError(RuntimeError):
    pass


def load():
    """Load the library once; raise if it is missing or its ABI version differs."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise PicomoeError(
            f"{LIB_PATH} not found: the HIP kernels are not built (run `make -C picotron_amd/csrc`). "
            "picotron_amd has no CPU or eager fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, ctypes.c_int)
    got = lib.picomoe_abi_version()
    if got != ABI_VERSION:
        raise PicomoeError(f"libpicomoe ABI {got} != expected {ABI_VERSION}; rebuild the library")
    _lib = lib
    return lib


def exported_symbols():
    return sorted(_SIGNATURES)


def check(code, what):
    if code != 0:
        msg = load().picomoe_error_string(code)
        raise PicomoeError(f"{what} failed with code {code}: {msg.decode() if msg else '?'}")


def dtype_code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise PicomoeError(f"picotron_amd kernels support float32 and bfloat16, got {dtype}") from None


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise PicomoeError(
                "picotron_amd runs on the GPU only (HIP kernels, no CPU fallback); got a tensor on " + str(t.device)
            )


def stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)
