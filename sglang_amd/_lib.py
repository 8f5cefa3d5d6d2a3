"""ctypes binding of libfp8k.so (the C ABI declared in include/fp8k.h and include/fp8k_tune.h).

There is one code path: if the shared library is missing or fails to load, importing this
module raises; nothing falls back to torch or CPU code.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libfp8k.so")

ABI_VERSION = 3

F32, F16, BF16 = 0, 1, 2
SCALE_F32, SCALE_UE8M0_PACKED, SCALE_UE8M0_F32 = 0, 1, 2

_DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_f32 = ctypes.c_float
_c_ptr = ctypes.c_void_p

# name -> (restype, argtypes)
SIGNATURES = {
    "fp8k_last_error": (ctypes.c_char_p, []),
    "fp8k_abi_version": (_c_int, []),
    "fp8k_group_quant": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_f32, _c_f32, _c_f32, _c_int, _c_i64, _c_i64, _c_int, _c_ptr],
    ),
    "fp8k_silu_mul_group_quant": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_f32, _c_f32, _c_f32, _c_int, _c_i64, _c_i64, _c_int, _c_ptr],
    ),
    "fp8k_group_quant_masked": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_f32, _c_f32, _c_f32, _c_int, _c_i64, _c_i64, _c_i64,
         _c_int, _c_int, _c_ptr, _c_ptr],
    ),
    "fp8k_token_quant": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_ptr]),
    "fp8k_tensor_quant": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_ptr]),
    "fp8k_tensor_quant_mla": (_c_int, [_c_ptr, _c_ptr, _c_ptr] + [_c_i64] * 5 + [_c_f32, _c_int, _c_ptr]),
    "fp8k_bmm_fp8": (_c_int, [_c_ptr] * 5 + [_c_i64] * 10 + [_c_int, _c_ptr]),
    "fp8k_moe_prepare_input": (_c_int, [_c_ptr] + [_c_i64] * 5 + [_c_ptr] * 7),
    "fp8k_shuffle_rows": (_c_int, [_c_ptr] * 3 + [_c_i64] * 3 + [_c_ptr]),
    "fp8k_apply_shuffle_mul_sum": (_c_int, [_c_ptr] * 4 + [_c_i64] * 4 + [_c_int, _c_ptr]),
    "fp8k_moe_blocks_from_offsets": (_c_int, [_c_ptr] * 2 + [_c_i64] * 3 + [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr]),
    "fp8k_moe_slot_blocks_from_offsets": (_c_int, [_c_ptr] * 2 + [_c_i64, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr]),
    "fp8k_moe_block_gemm_silu_quant": (_c_int, [_c_ptr] * 9 + [_c_i64] * 15 + [_c_f32, _c_int, _c_int, _c_ptr]),
    "fp8k_block_gemm": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr] + [_c_i64] * 10 + [_c_int, _c_ptr, _c_i64, _c_ptr],
    ),
    "fp8k_block_gemm_ue8m0": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr] + [_c_i64] * 10 + [_c_int, _c_ptr, _c_i64, _c_ptr],
    ),
    "fp8k_block_gemm_workspace_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "fp8k_block_gemm_noalloc": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr] + [_c_i64] * 10 + [_c_int, _c_ptr]),
    "fp8k_scaled_mm": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr] + [_c_i64] * 6 + [_c_int, _c_int, _c_ptr, _c_i64, _c_ptr],
    ),
    "fp8k_scaled_mm_workspace_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "fp8k_tune_force_gemm_plan": (None, [_c_int, _c_int]),
    "fp8k_tune_stream_read": (_c_int, [_c_ptr, _c_i64, _c_ptr]),
    "fp8k_tune_stream_read_tiles": (_c_int, [_c_ptr, _c_i64, _c_i64, _c_ptr]),
    "fp8k_tune_stream_read_write": (_c_int, [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_i64, _c_i64, _c_ptr]),
    "fp8k_tune_mfma_peak": (_c_int, [_c_ptr, _c_i64, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr]),
    "fp8k_tune_mfma_loop": (_c_int, [_c_ptr, _c_i64, _c_i64, _c_int, _c_ptr, _c_i64, _c_ptr, _c_ptr]),
    "fp8k_moe_align_block_size": (
        _c_int,
        [_c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_ptr],
    ),
    "fp8k_moe_block_gemm": (_c_int, [_c_ptr] * 9 + [_c_i64] * 16 + [_c_int, _c_int, _c_ptr]),
    "fp8k_moe_block_gemm_ue8m0": (_c_int, [_c_ptr] * 9 + [_c_i64] * 16 + [_c_int, _c_int, _c_ptr]),
    "fp8k_moe_balance_blocks": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "fp8k_moe_sort_scales": (_c_int, [_c_ptr] * 4 + [_c_i64] * 6 + [_c_ptr]),
    "fp8k_silu_and_mul": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr]),
    "fp8k_gelu_and_mul": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr]),
    "fp8k_activation": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr]),
    "fp8k_moe_sum_reduce": (_c_int, [_c_ptr, _c_ptr] + [_c_i64] * 6 + [_c_f32, _c_int, _c_ptr]),
    "fp8k_moe_sum": (_c_int, [_c_ptr, _c_ptr] + [_c_i64] * 6 + [_c_int, _c_ptr]),
    "fp8k_moe_fused_gate": (
        _c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr] + [_c_i64] * 6 + [ctypes.c_double, _c_int, _c_int, _c_ptr],
    ),
}


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "sglang_amd: %s is missing. Build it with `python sglang_amd/csrc/build.py` "
            "(hipcc, gfx950). There is no fallback path." % LIB_PATH
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.restype = res
        fn.argtypes = args
    got = lib.fp8k_abi_version()
    if got != ABI_VERSION:
        raise ImportError("sglang_amd: libfp8k.so has ABI version %d, the Python side expects %d" % (got, ABI_VERSION))
    return lib


lib = _load()


def check(status: int) -> None:
    """Raise RuntimeError with the library's message for a non-zero status (TORCH_CHECK analogue)."""
    if status != 0:
        raise RuntimeError(lib.fp8k_last_error().decode("utf-8", "replace") or "fp8k error %d" % status)


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise RuntimeError("fp8k: unsupported dtype %s (float32, float16, bfloat16 only)" % dt) from None


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("fp8k: tensors must live on the GPU (got a %s tensor)" % t.device.type)
