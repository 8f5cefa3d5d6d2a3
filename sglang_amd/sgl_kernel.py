"""The ops SGLang reaches through ``sgl_kernel`` on this path, backed by libfp8k.so.

Signatures, argument meaning and error behaviour follow sgl-kernel/python/sgl_kernel/gemm.py,
moe.py and elementwise.py of the reference; the native side is the C ABI in include/fp8k.h.
Quant ops write into caller-allocated outputs; GEMM ops return a fresh tensor.  Every launch goes
on the current torch stream of the tensor's device and never synchronises.
"""
from __future__ import annotations

import weakref
from typing import Optional


import torch

from . import _lib
from ._lib import check, dtype_code, lib, require_cuda, stream_ptr

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX = 448.0
FP8_MIN = -448.0

_workspaces: dict = {}   # (device index, stream handle) -> the buffer handed out on that stream
_retired: list = []      # every buffer ever handed out and since outgrown: kept alive for the life of the process


def _workspace(device: torch.device, nbytes: int) -> Optional[torch.Tensor]:
    """Scratch of the GEMM entry points (float partials of K-cut launches, the column-major scale copy), one buffer per
    (device, stream) so that GEMMs on two streams never share one.

    A buffer that has been handed out is never released: a HIP graph captured earlier still holds its address, and its
    replays write partials there.  When a later call needs more, a larger buffer takes its place for new launches and
    the old one is parked in `_retired`.  Growth is geometric (at least double, at least 32 MiB), so a process parks
    a handful of buffers at most.  Allocation under stream capture goes through torch's allocator like the GEMM's
    output tensor does, into the capturing graph's pool; `reserve_workspace` sizes the buffer ahead of a capture."""
    if nbytes <= 0:
        return None
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        size = max(nbytes, 32 << 20, 2 * buf.numel() if buf is not None else 0)
        if buf is not None:
            _retired.append(buf)
        buf = torch.empty(size, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def reserve_workspace(device: torch.device, nbytes: int) -> None:
    """Make the current stream's GEMM scratch on `device` at least `nbytes` large (see fp8k_*_workspace_bytes in
    include/fp8k.h for what a shape needs); call it before capturing a graph to keep the allocation out of the
    capture."""
    _workspace(torch.device(device), int(nbytes))


# --------------------------------------------------------------------------------------------
# quantisation
# --------------------------------------------------------------------------------------------


def sgl_per_token_group_quant_8bit(
    input: torch.Tensor,
    output_q: torch.Tensor,
    output_s: torch.Tensor,
    group_size: int,
    eps: float,
    fp8_min: float,
    fp8_max: float,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:100-136 (op schema common_extension.cc:128-152).

    output_s selects the scale layout by its strides and dtype: float32 [M, K/g] in any of row-major,
    column-major, column-major padded; int32 [M, ceil(K/g/4)] (column-major, M padded to 4) when
    scale_ue8m0.  `enable_v2` is accepted for signature compatibility: there is one kernel.
    fuse_silu_and_mul (the v2 op, gemm.py:118-133): input is [M, 2K] (gate columns, then up), output_q [M, K];
    what is quantised is silu_and_mul's 16-bit result, bit for bit.
    """
    require_cuda(input, output_q, output_s, masked_m)
    if masked_m is not None:
        return _group_quant_masked(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0,
                                   fuse_silu_and_mul, masked_m)
    if not input.is_contiguous():
        raise RuntimeError("input must be contiguous")
    if not output_q.is_contiguous():
        raise RuntimeError("output_q must be contiguous")
    if output_q.dtype != FP8_DTYPE:
        raise RuntimeError("output_q must be float8_e4m3fn (int8 destination is not built on this path)")
    if input.numel() % group_size != 0:
        raise RuntimeError("input.numel() %% group_size != 0 (%d, %d)" % (input.numel(), group_size))
    if output_s.dim() != 2:
        raise RuntimeError("output_s.dim() must be 2")
    if fuse_silu_and_mul and input.shape[-1] % 2 != 0:
        raise RuntimeError("fuse_silu_and_mul needs an even last dimension")
    K = input.shape[-1] // 2 if fuse_silu_and_mul else input.shape[-1]
    if K % group_size != 0:
        raise RuntimeError("the last dimension of `x` cannot be divisible by `group_size`")
    M = input.numel() // input.shape[-1] if K else 0
    G = K // group_size
    if output_q.numel() != M * K:
        raise RuntimeError("output_q has the wrong number of elements")
    if scale_ue8m0:
        if output_s.dtype != torch.int32:
            raise RuntimeError("scale_ue8m0 needs an int32 packed output_s")
        if output_s.shape[0] != M or output_s.shape[1] != (G + 3) // 4:
            raise RuntimeError("packed output_s must be [M, ceil(K/group/4)]")
        kind = _lib.SCALE_UE8M0_PACKED
    else:
        if output_s.dtype != torch.float32:
            raise RuntimeError("output_s must be float32")
        if output_s.shape[0] != M or output_s.shape[1] != G:
            raise RuntimeError("output_s must be [M, K/group_size]")
        kind = _lib.SCALE_F32
    fn = lib.fp8k_silu_mul_group_quant if fuse_silu_and_mul else lib.fp8k_group_quant
    check(
        fn(
            input.data_ptr(), output_q.data_ptr(), output_s.data_ptr(), M, K, group_size, float(eps), float(fp8_min),
            float(fp8_max), dtype_code(input.dtype), output_s.stride(0), output_s.stride(1), kind,
            stream_ptr(input.device),
        )
    )


def _group_quant_masked(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, fuse_silu_and_mul,
                        masked_m) -> None:
    """Masked expert layout of the v2 op (gemm.py:118-133): input [E, m_max, K] (or 2K with fuse_silu_and_mul),
    output_q [E, m_max, K], output_s [E, m_max, K/g] float32 in any strides or int32 [E, m_max, ceil(K/g/4)] packed
    (scale_ue8m0 with a float32 output_s stores the powers of two as floats); masked_m int32 [E] - rows at or past
    masked_m[e] are neither read nor written."""
    if input.dim() != 3 or output_q.dim() != 3 or output_s.dim() != 3:
        raise RuntimeError("masked_m needs 3-D input, output_q and output_s ([num_experts, max_tokens, hidden])")
    if not (input.is_contiguous() and output_q.is_contiguous()):
        raise RuntimeError("input and output_q must be contiguous")
    if output_q.dtype != FP8_DTYPE:
        raise RuntimeError("output_q must be float8_e4m3fn (int8 destination is not built on this path)")
    E, m_max, width = input.shape
    if fuse_silu_and_mul and width % 2 != 0:
        raise RuntimeError("fuse_silu_and_mul needs an even last dimension")
    K = width // 2 if fuse_silu_and_mul else width
    if K % group_size != 0:
        raise RuntimeError("the last dimension of `x` cannot be divisible by `group_size`")
    G = K // group_size
    if tuple(output_q.shape) != (E, m_max, K):
        raise RuntimeError("output_q must be [num_experts, max_tokens, hidden]")
    if masked_m.dtype != torch.int32 or masked_m.numel() != E or not masked_m.is_contiguous():
        raise RuntimeError("masked_m must be contiguous int32 [num_experts]")
    if scale_ue8m0 and output_s.dtype == torch.float32:
        # the rounded-up power of two as a float at the place of a float scale (ep_moe/kernels.py:348-350)
        if tuple(output_s.shape) != (E, m_max, G):
            raise RuntimeError("output_s must be float32 [num_experts, max_tokens, K/group_size]")
        kind = _lib.SCALE_UE8M0_F32
    elif scale_ue8m0:
        if output_s.dtype != torch.int32 or tuple(output_s.shape) != (E, m_max, (G + 3) // 4):
            raise RuntimeError("packed output_s must be int32 [num_experts, max_tokens, ceil(K/group/4)]")
        kind = _lib.SCALE_UE8M0_PACKED
    else:
        if output_s.dtype != torch.float32 or tuple(output_s.shape) != (E, m_max, G):
            raise RuntimeError("output_s must be float32 [num_experts, max_tokens, K/group_size]")
        kind = _lib.SCALE_F32
    check(
        lib.fp8k_group_quant_masked(
            input.data_ptr(), output_q.data_ptr(), output_s.data_ptr(), E, m_max, K, group_size, float(eps),
            float(fp8_min), float(fp8_max), dtype_code(input.dtype), output_s.stride(0), output_s.stride(1),
            output_s.stride(2), kind, 1 if fuse_silu_and_mul else 0, masked_m.data_ptr(), stream_ptr(input.device),
        )
    )


# legacy alias, as in the reference (gemm.py:139-141)
sgl_per_token_group_quant_fp8 = sgl_per_token_group_quant_8bit


def sgl_per_token_quant_fp8(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:155-160; csrc/gemm/per_token_quant_fp8.cu:166-236."""
    require_cuda(input, output_q, output_s)
    if not (input.is_contiguous() and output_q.is_contiguous() and output_s.is_contiguous()):
        raise RuntimeError("input, output_q and output_s must be contiguous")
    if input.dim() != 2:
        raise RuntimeError("input must be 2-D [num_tokens, hidden_dim]")
    if output_q.dtype != FP8_DTYPE or output_s.dtype != torch.float32:
        raise RuntimeError("output_q must be float8_e4m3fn and output_s float32")
    M, K = input.shape
    if K % 8 != 0:
        raise RuntimeError("Hidden dimension must be divisible by 8, but got %d" % K)
    if output_s.numel() != M or output_q.shape != input.shape:
        raise RuntimeError("output shapes do not match the input")
    check(lib.fp8k_token_quant(input.data_ptr(), output_q.data_ptr(), output_s.data_ptr(), M, K, dtype_code(input.dtype),
                               stream_ptr(input.device)))


def sgl_per_tensor_quant_fp8(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor, is_static: bool) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:144-152; csrc/gemm/per_tensor_quant_fp8.cu:96-118.
    Dynamic mode accumulates with an atomic max, so output_s must be zero on entry (as the caller does)."""
    require_cuda(input, output_q, output_s)
    if not (input.is_contiguous() and output_q.is_contiguous() and output_s.is_contiguous()):
        raise RuntimeError("input, output_q and output_s must be contiguous")
    if output_q.dtype != FP8_DTYPE or output_s.dtype != torch.float32 or output_s.numel() != 1:
        raise RuntimeError("output_q must be float8_e4m3fn and output_s a float32 scalar")
    check(lib.fp8k_tensor_quant(input.data_ptr(), output_q.data_ptr(), output_s.data_ptr(), input.numel(),
                                dtype_code(input.dtype), 1 if is_static else 0, stream_ptr(input.device)))


# --------------------------------------------------------------------------------------------
# GEMMs
# --------------------------------------------------------------------------------------------


def _out_code(out_dtype: torch.dtype) -> int:
    if out_dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("out_dtype must be Half or BFloat16")
    return dtype_code(out_dtype)


def _check_ab(mat_a: torch.Tensor, mat_b: torch.Tensor) -> None:
    require_cuda(mat_a, mat_b)
    if mat_a.dim() != 2:
        raise RuntimeError("mat_a must be a 2D tensor")
    if mat_b.dim() != 2:
        raise RuntimeError("mat_b must be a 2D tensor")
    if mat_a.shape[1] > 1 and mat_a.stride(1) != 1:
        raise RuntimeError("mat_a must be a row major tensor")
    if mat_b.shape[0] > 1 and mat_b.stride(0) != 1:
        raise RuntimeError("mat_b must be a column major tensor")
    if mat_a.shape[1] != mat_b.shape[0]:
        raise RuntimeError("mat_a and mat_b shapes cannot be multiplied")
    if mat_a.shape[1] % 16 != 0:
        raise RuntimeError("mat_a must be multiple of 16 bytes for memory alignment")
    if mat_a.dtype != FP8_DTYPE:
        raise RuntimeError("mat_a must be Float8_e4m3fn")
    if mat_b.dtype != FP8_DTYPE:
        raise RuntimeError("mat_b must be Float8_e4m3fn")


def fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype):
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:25-32; checks fp8_blockwise_gemm_kernel.cu:368-406.

    mat_a e4m3fn [M,K] row-major; mat_b e4m3fn [K,N] column-major (a [N,K] weight transposed);
    scales_a float32 [M, K/128] (M-major or contiguous vector); scales_b float32 [K/128, N/128]
    (K-major or contiguous vector).  Both scale tensors are addressed by stride, so other
    memory orders work too.  Returns [M,N] of out_dtype.
    """
    _check_ab(mat_a, mat_b)
    require_cuda(scales_a, scales_b)
    out_code = _out_code(out_dtype)
    M, K = mat_a.shape
    N = mat_b.shape[1]
    if K % 128 != 0 or N % 128 != 0:
        raise RuntimeError("fp8_blockwise_scaled_mm needs N and K to be multiples of 128")
    if scales_a.dim() != 2 or scales_a.shape[0] != M or scales_a.shape[1] != K // 128:
        raise RuntimeError("size of scales_a is not matched")
    if scales_b.dim() != 2 or scales_b.shape[0] != K // 128 or scales_b.shape[1] != N // 128:
        raise RuntimeError("size of scales_b is not matched")
    if scales_a.dtype != torch.float32:
        raise RuntimeError("scales_a must be Float32")
    if scales_b.dtype != torch.float32:
        raise RuntimeError("scales_b must be Float32")
    if (N * 2) % 16 != 0:
        raise RuntimeError("out must be multiple of 16 bytes for memory alignment")
    out = torch.empty((M, N), dtype=out_dtype, device=mat_a.device)
    if M == 0:
        return out
    ws_bytes = lib.fp8k_block_gemm_workspace_bytes(M, N, K)
    ws = _workspace(mat_a.device, ws_bytes)
    check(
        lib.fp8k_block_gemm(
            mat_a.data_ptr(), mat_b.data_ptr(), scales_a.data_ptr(), scales_b.data_ptr(), out.data_ptr(), M, N, K,
            mat_a.stride(0) if M > 1 else K, mat_b.stride(1) if N > 1 else K,
            scales_a.stride(0), scales_a.stride(1), scales_b.stride(1), scales_b.stride(0), out.stride(0), out_code,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, stream_ptr(mat_a.device),
        )
    )
    return out


def fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:35-43; checks fp8_gemm_kernel.cu:1450-1487.

    C = (mat_a @ mat_b) * scales_a[m] * scales_b[n] (+ bias[n]).  bias may be out_dtype (the
    device op's rule) or float32 (the CPU twin's rule, csrc/cpu/gemm_fp8.cpp:523); it is added in
    float32 before the output cast.
    """
    _check_ab(mat_a, mat_b)
    require_cuda(scales_a, scales_b, bias)
    out_code = _out_code(out_dtype)
    M, K = mat_a.shape
    N = mat_b.shape[1]
    if scales_a.numel() != M:
        raise RuntimeError("size of scales_a is not matched")
    if scales_b.numel() != N:
        raise RuntimeError("size of scales_b is not matched")
    if not scales_a.is_contiguous():
        raise RuntimeError("scales_a must be contiguous")
    if not scales_b.is_contiguous():
        raise RuntimeError("scales_b msut be contiguous")
    if scales_a.dtype != torch.float32:
        raise RuntimeError("scales_a must be Float32")
    if scales_b.dtype != torch.float32:
        raise RuntimeError("scales_b must be Float32")
    bias_code = _lib.F32
    if bias is not None:
        if bias.numel() != N:
            raise RuntimeError("size of bias is not matched")
        if not bias.is_contiguous():
            raise RuntimeError("bias must be contiguous")
        if bias.dtype != out_dtype and bias.dtype != torch.float32:
            raise RuntimeError("bias dtype must match output dtype")
        bias_code = dtype_code(bias.dtype)
    if (N * 2) % 16 != 0:
        raise RuntimeError("out must be multiple of 16 bytes for memory alignment")
    out = torch.empty((M, N), dtype=out_dtype, device=mat_a.device)
    if M == 0:
        return out
    ws_bytes = lib.fp8k_scaled_mm_workspace_bytes(M, N, K)
    ws = _workspace(mat_a.device, ws_bytes)
    check(
        lib.fp8k_scaled_mm(
            mat_a.data_ptr(), mat_b.data_ptr(), scales_a.data_ptr(), scales_b.data_ptr(),
            bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K,
            mat_a.stride(0) if M > 1 else K, mat_b.stride(1) if N > 1 else K, out.stride(0), out_code, bias_code,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, stream_ptr(mat_a.device),
        )
    )
    return out


def tensor_quant_mla(x: torch.Tensor, x_q: torch.Tensor, x_s: torch.Tensor, eps: float) -> None:
    """Per-tensor quant of a strided [H, S, D] tensor into the contiguous x_q; x_s (one float32, zero on entry) receives
    max(absmax, eps) / 448.  Native side of fp8_kernel.per_tensor_quant_mla_fp8 (include/fp8k.h: fp8k_tensor_quant_mla)."""
    require_cuda(x, x_q, x_s)
    if x.dim() != 3 or x.stride(2) != 1:
        raise RuntimeError("per_tensor_quant_mla_fp8: x must be 3-D with a contiguous last dimension")
    if x_q.dtype != FP8_DTYPE or not x_q.is_contiguous() or x_q.shape != x.shape:
        raise RuntimeError("per_tensor_quant_mla_fp8: x_q must be contiguous float8_e4m3fn of x's shape")
    if x_s.dtype != torch.float32 or x_s.numel() != 1:
        raise RuntimeError("per_tensor_quant_mla_fp8: x_s must be one float32")
    H, S, D = x.shape
    check(lib.fp8k_tensor_quant_mla(x.data_ptr(), x_q.data_ptr(), x_s.data_ptr(), H, S, D, x.stride(0), x.stride(1), float(eps),
                                    dtype_code(x.dtype), stream_ptr(x.device)))


def bmm_fp8(A: torch.Tensor, B: torch.Tensor, A_scale: torch.Tensor, B_scale: torch.Tensor, dtype: torch.dtype,
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:66-82 (a cuBLASLt batched GEMM there).  A e4m3fn [b, m, k] with k
    contiguous, B e4m3fn [b, k, n] column-major per entry (k contiguous: a [b, n, k] weight transposed), one float32
    scale per operand; returns / fills out [b, m, n] = (A @ B) * A_scale * B_scale in `dtype`.  No host synchronisation:
    the scalar scales are broadcast to vectors on the device."""
    require_cuda(A, B, A_scale, B_scale, out)
    if A.dim() != 3 or B.dim() != 3 or A.shape[0] != B.shape[0] or A.shape[2] != B.shape[1]:
        raise RuntimeError("bmm_fp8: A [b, m, k] and B [b, k, n] expected")
    if A.dtype != FP8_DTYPE or B.dtype != FP8_DTYPE:
        raise RuntimeError("bmm_fp8: A and B must be float8_e4m3fn (e5m2 is not built on this path)")
    b, m, k = A.shape
    n = B.shape[2]
    if (k > 1 and A.stride(2) != 1) or (k > 1 and B.stride(1) != 1):
        raise RuntimeError("bmm_fp8: A must be row-major and B column-major in their last two dimensions")
    if A_scale.numel() != 1 or B_scale.numel() != 1:
        raise RuntimeError("bmm_fp8: one scale per operand expected")
    out_code = _out_code(dtype)
    if out is None:
        out = torch.empty((b, m, n), device=A.device, dtype=dtype)
    elif out.shape != (b, m, n) or out.dtype != dtype or (n > 1 and out.stride(2) != 1):
        raise RuntimeError("bmm_fp8: out must be [b, m, n] of the result dtype with a contiguous last dimension")
    if b == 0 or m == 0 or n == 0:
        return out
    if k % 128 != 0 or n % 8 != 0:
        # the kernel walks K in blocks of 128 and writes 8 columns at a time: zero padding changes no sum
        kp, np_ = (k + 127) // 128 * 128, (n + 7) // 8 * 8
        Ap = A.new_zeros((b, m, kp), dtype=torch.uint8)
        Ap[:, :, :k] = A.view(torch.uint8)
        Bp = B.new_zeros((b, np_, kp), dtype=torch.uint8)
        Bp[:, :n, :k] = B.view(torch.uint8).transpose(1, 2)
        res = bmm_fp8(Ap.view(FP8_DTYPE), Bp.view(FP8_DTYPE).transpose(1, 2), A_scale, B_scale, dtype)
        out.copy_(res[:, :, :n])
        return out
    sa = A_scale.reshape(1).to(torch.float32).expand(m).contiguous()
    sb = B_scale.reshape(1).to(torch.float32).expand(n).contiguous()
    check(lib.fp8k_bmm_fp8(A.data_ptr(), B.data_ptr(), sa.data_ptr(), sb.data_ptr(), out.data_ptr(), b, m, n, k,
                           A.stride(0) if b > 1 else m * k, A.stride(1) if m > 1 else k, B.stride(0) if b > 1 else n * k,
                           B.stride(2) if n > 1 else k, out.stride(0) if b > 1 else m * n, out.stride(1) if m > 1 else n,
                           out_code, stream_ptr(A.device)))
    return out


def _block_gemm_nk(A, B, As, Bs, out_dtype):
    """Block GEMM on the Triton-side layout: B [N,K] row-major, Bs [ceil(N/128), ceil(K/128)].

    Used by w8a8_block_fp8_matmul; unlike fp8_blockwise_scaled_mm it admits N, K that are not
    multiples of 128 (python/sglang/srt/layers/quantization/fp8_kernel.py:1072-1149 uses cdiv + masks).
    """
    require_cuda(A, B, As, Bs)
    if A.dtype != FP8_DTYPE or B.dtype != FP8_DTYPE:
        raise RuntimeError("A and B must be Float8_e4m3fn")
    out_code = _out_code(out_dtype)
    M, K = A.shape
    N = B.shape[0]
    if K % 16 != 0:
        raise RuntimeError("mat_a must be multiple of 16 bytes for memory alignment")
    if (N * 2) % 16 != 0:
        raise RuntimeError("out must be multiple of 16 bytes for memory alignment")
    out = torch.empty((M, N), dtype=out_dtype, device=A.device)
    if M == 0:
        return out
    ws_bytes = lib.fp8k_block_gemm_workspace_bytes(M, N, K)
    ws = _workspace(A.device, ws_bytes)
    check(
        lib.fp8k_block_gemm(
            A.data_ptr(), B.data_ptr(), As.data_ptr(), Bs.data_ptr(), out.data_ptr(), M, N, K,
            A.stride(0) if M > 1 else K, B.stride(0) if N > 1 else K, As.stride(0), As.stride(1), Bs.stride(0),
            Bs.stride(1), out.stride(0), out_code, ws.data_ptr() if ws is not None else None,
            ws.numel() if ws is not None else 0, stream_ptr(A.device),
        )
    )
    return out


def unpack_ue8m0_scales(packed: torch.Tensor, num_groups: int) -> torch.Tensor:
    """int32 words of four UE8M0 exponent bytes [..., M, ceil(G/4)] -> float32 powers of two [..., M, G]
    (byte g % 4 of word g // 4 is the exponent of group g; decode is byte << 23, fp8_utils.py:549-550 of the reference)."""
    shifts = torch.arange(0, 32, 8, device=packed.device, dtype=torch.int32)
    exps = (packed.unsqueeze(-1) >> shifts) & 0xFF
    return (exps.reshape(*packed.shape[:-1], -1)[..., :num_groups] << 23).contiguous().view(torch.float32)


def unpack_ue8m0_weight_scales(packed: torch.Tensor, K: int) -> torch.Tensor:
    """Packed UE8M0 weight scales in the layout the reference hands to DeepGEMM - int32 [..., N, ceil(K/128/4)], one
    row per weight row, the 128 rows of a block carrying the same words (fp8_kernel.py:1036-1043, inverse transform
    fp8_utils.py:529-564) - to float32 powers of two [..., ceil(N/128), K/128], one row per 128-row block."""
    kb = (K + 127) // 128
    return unpack_ue8m0_scales(packed[..., ::128, :], kb)


# Tensors declared to hold powers of two, by the memory they describe: (device, address of the first element, shape,
# strides) -> weak reference to the tensor object that was marked.  A Python attribute on the tensor object alone would
# be lost by every `.data`, `nn.Parameter(t)` or view that describes the same memory with a new object; an entry lives
# only as long as the marked object does (so the memory cannot have been handed to another tensor meanwhile).
_UE8M0_MARKED: dict = {}


def _memory_key(t: torch.Tensor):
    return (str(t.device), t.data_ptr(), tuple(t.shape), tuple(t.stride()))


def is_ue8m0(scales: torch.Tensor) -> bool:
    """True for a float32 scale tensor whose memory has been declared to hold powers of two only (mark_ue8m0): the
    marked tensor itself, its `.data`, a Parameter wrapped around it, or any other tensor object of the same device,
    address, shape and strides, for as long as the marked object is alive."""
    if scales.dtype != torch.float32:
        return False
    if getattr(scales, "_fp8k_ue8m0", False):  # the marked object itself (also what a graph tracer can see)
        return True
    # no addresses while tracing or under fake tensors: unmarked objects take the float-scale kernels
    if torch.compiler.is_compiling() or isinstance(scales, torch._subclasses.fake_tensor.FakeTensor):
        return False
    ref = _UE8M0_MARKED.get(_memory_key(scales))
    return ref is not None and ref() is not None


def mark_ue8m0(scales: torch.Tensor, check: bool = True) -> torch.Tensor:
    """Declare a float32 weight-scale tensor to hold positive powers of two only, which lets the block GEMM hand the
    exponents to the matrix core instead of multiplying.  With `check` (the default; one device synchronisation, meant
    for weight-loading time) every mantissa is verified to be zero first.  The declaration is about the contents: mark
    again after overwriting them.  Returns the same tensor."""
    if scales.dtype != torch.float32:
        raise RuntimeError("mark_ue8m0: float32 scales expected")
    if check:
        bits = scales.contiguous().view(torch.int32)
        if bool(((bits & 0x7FFFFF) != 0).any()) or bool((bits <= 0).any()):
            raise RuntimeError("mark_ue8m0: the scales are not all positive powers of two")
    key = _memory_key(scales)

    def _forget(ref, key=key):
        if _UE8M0_MARKED.get(key) is ref:
            del _UE8M0_MARKED[key]

    _UE8M0_MARKED[key] = weakref.ref(scales, _forget)
    scales._fp8k_ue8m0 = True
    return scales


def _block_gemm_nk_ue8m0(A, B, As_packed, Bs, out_dtype):
    """Block GEMM with packed UE8M0 activation scales (as the group quant writes them with scale_ue8m0=True) and float32
    weight scales that are powers of two: the matrix core applies both scales itself (include/fp8k.h:
    fp8k_block_gemm_ue8m0).  A weight scale with a non-zero mantissa would lose it here, so callers route to this
    function only for scales known to be powers of two (see fp8_kernel.w8a8_block_fp8_matmul); up to 128 rows, where the
    kernels have no such mode, the exponents are expanded and the float-scale kernels run - the same numbers."""
    require_cuda(A, B, As_packed, Bs)
    if A.dtype != FP8_DTYPE or B.dtype != FP8_DTYPE:
        raise RuntimeError("A and B must be Float8_e4m3fn")
    if As_packed.dtype != torch.int32 or Bs.dtype != torch.float32:
        raise RuntimeError("packed activation scales must be int32, weight scales float32")
    out_code = _out_code(out_dtype)
    M, K = A.shape
    N = B.shape[0]
    G = (K + 127) // 128
    if As_packed.shape[0] != M or As_packed.shape[1] != (G + 3) // 4:
        raise RuntimeError("packed activation scales must be [M, ceil(K/128/4)]")
    if M <= 128 or K % 128 != 0 or N % 4 != 0:
        return _block_gemm_nk(A, B, unpack_ue8m0_scales(As_packed, G), Bs, out_dtype)
    if (N * 2) % 16 != 0:
        raise RuntimeError("out must be multiple of 16 bytes for memory alignment")
    out = torch.empty((M, N), dtype=out_dtype, device=A.device)
    ws_bytes = lib.fp8k_block_gemm_workspace_bytes(M, N, K)
    ws = _workspace(A.device, ws_bytes)
    check(
        lib.fp8k_block_gemm_ue8m0(
            A.data_ptr(), B.data_ptr(), As_packed.data_ptr(), Bs.data_ptr(), out.data_ptr(), M, N, K, A.stride(0),
            B.stride(0) if N > 1 else K, As_packed.stride(0), As_packed.stride(1), Bs.stride(0), Bs.stride(1),
            out.stride(0), out_code, ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            stream_ptr(A.device),
        )
    )
    return out


# --------------------------------------------------------------------------------------------
# fused-MoE helpers
# --------------------------------------------------------------------------------------------


def moe_align_block_size(
    topk_ids: torch.Tensor,
    num_experts: int,
    block_size: int,
    sorted_token_ids: torch.Tensor,
    experts_ids: torch.Tensor,
    num_tokens_post_pad: torch.Tensor,
    cumsum_buffer: Optional[torch.Tensor],
    pad_sorted_token_ids: bool = False,
) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/moe.py:6-25; csrc/moe/moe_align_kernel.cu:302-366.

    `num_experts` is the number of buckets: the Python caller passes E+1 so that id -1 (an expert
    on another rank) lands in bucket 0 and expert e in bucket e+1.  All outputs are caller-allocated.
    """
    require_cuda(topk_ids, sorted_token_ids, experts_ids, num_tokens_post_pad, cumsum_buffer)
    if topk_ids.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("topk_ids must be int32 or int64")
    if not topk_ids.is_contiguous():
        raise RuntimeError("topk_ids must be contiguous")
    for t, name in ((sorted_token_ids, "sorted_token_ids"), (experts_ids, "experts_ids"),
                    (num_tokens_post_pad, "num_tokens_post_pad")):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("%s must be a contiguous int32 tensor" % name)
    if cumsum_buffer is not None:
        if cumsum_buffer.dtype != torch.int32 or cumsum_buffer.numel() < num_experts + 1:
            raise RuntimeError("cumsum_buffer must be int32 with at least num_experts + 1 entries")
    check(
        lib.fp8k_moe_align_block_size(
            topk_ids.data_ptr(), 1 if topk_ids.dtype == torch.int64 else 0, topk_ids.numel(), num_experts, block_size,
            sorted_token_ids.data_ptr(), sorted_token_ids.numel(), experts_ids.data_ptr(), experts_ids.numel(),
            num_tokens_post_pad.data_ptr(), cumsum_buffer.data_ptr() if cumsum_buffer is not None else None,
            1 if pad_sorted_token_ids else 0, stream_ptr(topk_ids.device),
        )
    )


def _act_and_mul(name: str, fn, input: torch.Tensor, out: Optional[torch.Tensor]) -> torch.Tensor:
    if input.shape[-1] * input.dtype.itemsize % 16 != 0:
        raise ValueError("The pointers must be multiple of 16 bytes.")
    if out is not None:
        assert input.ndim == out.ndim, f"{input.ndim} != {out.ndim}"
        assert input.shape[:-1] == out.shape[:-1], f"{input.shape[:-1]} != {out.shape[:-1]}"
        assert input.shape[-1] == 2 * out.shape[-1], f"{input.shape[-1]} != {2 * out.shape[-1]}"
    else:
        out = torch.empty(input.shape[:-1] + (input.shape[-1] // 2,), device=input.device, dtype=input.dtype)
    require_cuda(input, out)
    if out.dtype != input.dtype:
        raise RuntimeError("%s: out must have the dtype of input" % name)
    if not (input.is_contiguous() and out.is_contiguous()):
        raise RuntimeError("%s: input and out must be contiguous" % name)
    d = out.shape[-1]
    rows = out.numel() // d if d else 0
    check(fn(input.data_ptr(), out.data_ptr(), rows, d, 2 * d, d, dtype_code(input.dtype), stream_ptr(input.device)))
    return out


def silu_and_mul(input: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Reference: sgl-kernel/python/sgl_kernel/elementwise.py:172-184."""
    return _act_and_mul("silu_and_mul", lib.fp8k_silu_and_mul, input, out)


def gelu_and_mul(input: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Reference: sgl-kernel/python/sgl_kernel/elementwise.py:202-214 (the erf form of gelu)."""
    return _act_and_mul("gelu_and_mul", lib.fp8k_gelu_and_mul, input, out)


ACTIVATION_KINDS = {"silu": 0, "gelu": 1, "relu2": 2}


def activation(input: torch.Tensor, kind: str, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(input) elementwise: the activation of experts without a gate projection - F.silu, F.gelu (erf form) and
    torch.square(F.relu(.)) in the reference (python/sglang/srt/layers/moe/fused_moe_triton/fused_moe.py:566-572)."""
    if kind not in ACTIVATION_KINDS:
        raise ValueError(f"Unsupported activation: {kind=}")
    if input.shape[-1] * input.dtype.itemsize % 16 != 0:
        raise ValueError("The pointers must be multiple of 16 bytes.")
    if out is None:
        out = torch.empty_like(input)
    require_cuda(input, out)
    if out.shape != input.shape or out.dtype != input.dtype:
        raise RuntimeError("activation: out must have the shape and dtype of input")
    if not (input.is_contiguous() and out.is_contiguous()):
        raise RuntimeError("activation: input and out must be contiguous")
    d = input.shape[-1]
    rows = input.numel() // d if d else 0
    check(lib.fp8k_activation(input.data_ptr(), out.data_ptr(), rows, d, d, d, ACTIVATION_KINDS[kind], dtype_code(input.dtype),
                              stream_ptr(input.device)))
    return out


def moe_sum_reduce(input_tensor: torch.Tensor, output_tensor: torch.Tensor, routed_scaling_factor: float = 0) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/moe.py:83-92; csrc/moe/moe_sum_reduce.cu:227-.
    input [tokens, topk, hidden] (hidden contiguous), output [tokens, hidden]."""
    T, topk, H = _sum_args("moe_sum_reduce", input_tensor, output_tensor)
    check(lib.fp8k_moe_sum_reduce(input_tensor.data_ptr(), output_tensor.data_ptr(), T, topk, H, input_tensor.stride(0),
                                  input_tensor.stride(1), output_tensor.stride(0), float(routed_scaling_factor),
                                  dtype_code(input_tensor.dtype), stream_ptr(input_tensor.device)))


def _sum_args(op: str, input_tensor: torch.Tensor, output_tensor: torch.Tensor):
    require_cuda(input_tensor, output_tensor)
    if input_tensor.dim() != 3 or output_tensor.dim() != 2:
        raise RuntimeError("%s: input must be [tokens, topk, hidden] and output [tokens, hidden]" % op)
    T, topk, H = input_tensor.shape
    if output_tensor.shape[0] != T or output_tensor.shape[1] != H:
        raise RuntimeError("%s: output shape does not match the input" % op)
    if input_tensor.dtype != output_tensor.dtype:
        raise RuntimeError("%s: input and output dtypes differ" % op)
    if (H > 1 and input_tensor.stride(2) != 1) or (H > 1 and output_tensor.stride(1) != 1):
        raise RuntimeError("%s: the hidden dimension must be contiguous" % op)
    return T, topk, H


def moe_sum(input_tensor: torch.Tensor, output_tensor: torch.Tensor) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/moe.py:95-102; csrc/moe/moe_sum.cu:11-69.  input [tokens, topk, hidden],
    output [tokens, hidden].  As in the reference, 2, 3 and 4 experts per token are summed in the element type, one
    rounding per addition; any other count is the float-accumulated sum of moe_sum_reduce with factor 1."""
    T, topk, H = _sum_args("moe_sum", input_tensor, output_tensor)
    if topk == 0:
        raise RuntimeError("moe_sum: input must be [tokens, topk, hidden] with topk >= 1")
    check(lib.fp8k_moe_sum(input_tensor.data_ptr(), output_tensor.data_ptr(), T, topk, H, input_tensor.stride(0),
                           input_tensor.stride(1), output_tensor.stride(0), dtype_code(input_tensor.dtype),
                           stream_ptr(input_tensor.device)))


def moe_sort_scales(A_scale, sorted_token_ids, num_tokens_post_padded, top_k: int, num_valid_tokens: int) -> torch.Tensor:
    """Activation scales gathered into the order of sorted_token_ids (see include/fp8k.h: fp8k_moe_sort_scales):
    returns a [len(sorted_token_ids), K/128] view with strides (1, len): row i holds the scales of slot
    sorted_token_ids[i].  Pass it to moe_block_gemm with scales_sorted=True."""
    require_cuda(A_scale, sorted_token_ids, num_tokens_post_padded)
    if A_scale.dtype != torch.float32 or A_scale.dim() != 2:
        raise RuntimeError("moe_sort_scales: A_scale must be Float32 [rows, K/128]")
    cap, kb = sorted_token_ids.numel(), A_scale.shape[1]
    out = torch.empty((kb, cap), dtype=torch.float32, device=A_scale.device)
    check(
        lib.fp8k_moe_sort_scales(
            A_scale.data_ptr(), out.data_ptr(), sorted_token_ids.data_ptr(), num_tokens_post_padded.data_ptr(), cap, kb,
            top_k, num_valid_tokens, A_scale.stride(0), A_scale.stride(1), stream_ptr(A_scale.device),
        )
    )
    return out.t()


def moe_balance_blocks(sorted_token_ids, expert_ids, num_tokens_post_padded, block_m: int, num_valid_tokens: int,
                       num_experts: int) -> torch.Tensor:
    """The table of moe_align_block_size with every expert's slots dealt out evenly over the blocks the expert already has
    (include/fp8k.h: fp8k_moe_balance_blocks); returns the new sorted_token_ids, expert_ids and num_tokens_post_padded
    stay valid.  For the grouped GEMM with several blocks per expert: blocks of one expert then take the same time and
    share their weight tiles in L2."""
    require_cuda(sorted_token_ids, expert_ids, num_tokens_post_padded)
    for t, name in ((sorted_token_ids, "sorted_token_ids"), (expert_ids, "expert_ids"), (num_tokens_post_padded, "num_tokens_post_padded")):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("moe_balance_blocks: %s must be contiguous int32" % name)
    cap = sorted_token_ids.numel()
    if expert_ids.numel() * block_m < cap - cap % block_m:
        raise RuntimeError("moe_balance_blocks: expert_ids is shorter than the block table")
    out = torch.empty_like(sorted_token_ids)
    check(lib.fp8k_moe_balance_blocks(sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(), cap,
                                      block_m, num_valid_tokens, num_experts, out.data_ptr(), stream_ptr(out.device)))
    return out


def moe_block_gemm(A, B, C, A_scale, B_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded,
                   mul_routed_weight: bool, top_k: int, block_m: int, num_valid_tokens: int,
                   scales_sorted: bool = False, pow2_scales: bool = False, balanced: bool = False) -> None:
    """Grouped block-FP8 GEMM behind invoke_fused_moe_kernel (see include/fp8k.h: fp8k_moe_block_gemm).
    A e4m3fn [rows, K]; B e4m3fn [E, N, K]; A_scale float32 [rows, K/128] (scales_sorted: one row per entry of
    sorted_token_ids, from moe_sort_scales); B_scale float32 [E, N/128, K/128];
    C [num_valid_tokens, N] (any leading shape, flattened) bf16/fp16, written in place.
    pow2_scales: the caller vouches that every scale is a power of two (UE8M0); 256-slot blocks with sorted scales
    then let the matrix cores apply the scales (fp8k_moe_block_gemm_ue8m0).
    balanced: sorted_token_ids went through moe_balance_blocks (a hint for the 256-slot kernel's schedule)."""
    require_cuda(A, B, C, A_scale, B_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded)
    if A.dtype != FP8_DTYPE or B.dtype != FP8_DTYPE:
        raise RuntimeError("moe_block_gemm: A and B must be Float8_e4m3fn")
    if A_scale.dtype != torch.float32 or B_scale.dtype != torch.float32:
        raise RuntimeError("moe_block_gemm: scales must be Float32")
    if B.dim() != 3 or B_scale.dim() != 3 or A.dim() != 2 or A_scale.dim() != 2:
        raise RuntimeError("moe_block_gemm: A [rows,K], B [E,N,K], A_scale [rows,K/128], B_scale [E,N/128,K/128]")
    E, N, K = B.shape
    if A.shape[1] != K or (K > 1 and (A.stride(1) != 1 or B.stride(2) != 1)):
        raise RuntimeError("moe_block_gemm: K must be the contiguous dimension of A and B")
    if A_scale.shape[0] != (sorted_token_ids.numel() if scales_sorted else A.shape[0]) or A_scale.shape[1] != (K + 127) // 128:
        raise RuntimeError("moe_block_gemm: A_scale shape does not match A")
    if B_scale.shape[0] != E or B_scale.shape[1] != (N + 127) // 128 or B_scale.shape[2] != (K + 127) // 128:
        raise RuntimeError("moe_block_gemm: B_scale shape does not match B")
    C2 = C.view(-1, C.shape[-1])
    if C2.shape[1] != N or C2.shape[0] < num_valid_tokens or C2.stride(1) != 1:
        raise RuntimeError("moe_block_gemm: C must be [num_valid_tokens, N] with N contiguous")
    if A.shape[0] * top_k < num_valid_tokens:
        raise RuntimeError("moe_block_gemm: A has too few rows for num_valid_tokens / top_k")
    if mul_routed_weight:
        if topk_weights.dtype != torch.float32 or not topk_weights.is_contiguous() or topk_weights.numel() < num_valid_tokens:
            raise RuntimeError("moe_block_gemm: topk_weights must be contiguous Float32 with one entry per slot")
    for t in (sorted_token_ids, expert_ids, num_tokens_post_padded):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("moe_block_gemm: index tensors must be contiguous int32")
    if expert_ids.numel() * block_m < sorted_token_ids.numel() - (sorted_token_ids.numel() % block_m):
        raise RuntimeError("moe_block_gemm: expert_ids is shorter than sorted_token_ids / block_m")
    check(
        (lib.fp8k_moe_block_gemm_ue8m0 if pow2_scales else lib.fp8k_moe_block_gemm)(
            A.data_ptr(), B.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(), C2.data_ptr(),
            sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(),
            topk_weights.data_ptr() if mul_routed_weight else None, sorted_token_ids.numel(), block_m,
            num_valid_tokens, top_k, E, N, K, A.stride(0), A_scale.stride(0), A_scale.stride(1), B.stride(0),
            B.stride(1), B_scale.stride(0), B_scale.stride(1), B_scale.stride(2), C2.stride(0), _out_code(C.dtype),
            (1 if scales_sorted else 0) | (2 if balanced else 0), stream_ptr(A.device),
        )
    )


def prepare_moe_input(topk_ids, expert_offsets, problem_sizes1, problem_sizes2, input_permutation, output_permutation,
                      num_experts, n, k, blockscale_offsets: Optional[torch.Tensor] = None) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/moe.py:217-240 (csrc/moe/prepare_moe_input.cu).  Sorts the (token, k)
    slots of topk_ids int32 [m, topk] by expert into contiguous row ranges: expert_offsets int32 [E + 1],
    problem_sizes1 / 2 int32 [E, 3] = (rows, 2n, k) / (rows, k, n), input_permutation [m * topk] (row -> token),
    output_permutation [m * topk] (slot -> row).  The order of the rows inside an expert is not defined."""
    require_cuda(topk_ids, expert_offsets, problem_sizes1, problem_sizes2, input_permutation, output_permutation,
                 blockscale_offsets)
    if topk_ids.dtype != torch.int32 or topk_ids.dim() != 2 or not topk_ids.is_contiguous():
        raise RuntimeError("prepare_moe_input: topk_ids must be contiguous int32 [m, topk]")
    numel = topk_ids.numel()
    for name, t, need in (("expert_offsets", expert_offsets, num_experts + 1), ("problem_sizes1", problem_sizes1, 3 * num_experts),
                          ("problem_sizes2", problem_sizes2, 3 * num_experts), ("input_permutation", input_permutation, numel),
                          ("output_permutation", output_permutation, numel), ("blockscale_offsets", blockscale_offsets, num_experts + 1)):
        if t is None:
            continue
        if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < need:
            raise RuntimeError("prepare_moe_input: %s must be contiguous int32 with at least %d entries" % (name, need))
    check(lib.fp8k_moe_prepare_input(topk_ids.data_ptr(), numel, max(topk_ids.shape[1], 1), num_experts, n, k,
                                     expert_offsets.data_ptr(), None if blockscale_offsets is None else blockscale_offsets.data_ptr(),
                                     problem_sizes1.data_ptr(), problem_sizes2.data_ptr(), input_permutation.data_ptr(),
                                     output_permutation.data_ptr(), stream_ptr(topk_ids.device)))


def shuffle_rows_out(input_tensor: torch.Tensor, dst2src_map: torch.Tensor, output_tensor: torch.Tensor) -> None:
    """output[d] = input[dst2src_map[d]] for 2-D contiguous tensors of one dtype (the op behind shuffle_rows)."""
    require_cuda(input_tensor, dst2src_map, output_tensor)
    if input_tensor.dtype != output_tensor.dtype:
        raise RuntimeError("shuffle_rows: input and output tensors must have the same data type")
    if input_tensor.dim() != 2 or output_tensor.dim() != 2 or input_tensor.shape[1] != output_tensor.shape[1]:
        raise RuntimeError("shuffle_rows: 2-D tensors with the same row length expected")
    if not (input_tensor.is_contiguous() and output_tensor.is_contiguous()):
        raise RuntimeError("shuffle_rows: input and output must be contiguous")
    if dst2src_map.dtype != torch.int32 or not dst2src_map.is_contiguous() or dst2src_map.numel() < output_tensor.shape[0]:
        raise RuntimeError("shuffle_rows: dst2src_map must be contiguous int32 with one entry per output row")
    check(lib.fp8k_shuffle_rows(input_tensor.data_ptr(), dst2src_map.data_ptr(), output_tensor.data_ptr(), input_tensor.shape[0],
                                output_tensor.shape[0], input_tensor.shape[1] * input_tensor.element_size(),
                                stream_ptr(input_tensor.device)))


def shuffle_rows(input_tensor: torch.Tensor, dst2src_map: torch.Tensor, output_tensor_shape) -> torch.Tensor:
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:302-309."""
    output_tensor = torch.empty(output_tensor_shape, device=input_tensor.device, dtype=input_tensor.dtype)
    shuffle_rows_out(input_tensor, dst2src_map, output_tensor)
    return output_tensor


def apply_shuffle_mul_sum(input: torch.Tensor, output: torch.Tensor, permutation: torch.Tensor,
                          factors: Optional[torch.Tensor]) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/moe.py:243-251:
    output = (input[permutation].view(m, topk, k) * factors.view(m, topk, 1)).sum(dim=1), summed in float32."""
    require_cuda(input, output, permutation, factors)
    if input.dim() != 2 or output.dim() != 2 or (permutation is not None and permutation.dim() != 1):
        raise RuntimeError("apply_shuffle_mul_sum: input [m * topk, k], output [m, k], permutation [m * topk]")
    if input.dtype != output.dtype or not (input.is_contiguous() and output.is_contiguous()) or input.shape[1] != output.shape[1]:
        raise RuntimeError("apply_shuffle_mul_sum: input and output must be contiguous, of one dtype and row length")
    m = output.shape[0]
    if permutation is None:  # rows already in slot order: output[t] sums input[t * topk .. t * topk + topk - 1]
        topk = input.shape[0] // m if m else 0
        if input.shape[0] != m * topk:
            raise RuntimeError("apply_shuffle_mul_sum: without a permutation input must hold m * topk rows")
    else:
        topk = permutation.numel() // m if m else 0
        if permutation.numel() != m * topk or permutation.dtype != torch.int32 or not permutation.is_contiguous():
            raise RuntimeError("apply_shuffle_mul_sum: permutation size must match m * topk (contiguous int32)")
    if factors is not None:
        if factors.dtype != output.dtype:
            raise RuntimeError("apply_shuffle_mul_sum: factors must match output dtype")
        if factors.numel() != m * topk or not factors.is_contiguous():
            raise RuntimeError("apply_shuffle_mul_sum: factors must have shape [m * topk]")
    check(lib.fp8k_apply_shuffle_mul_sum(input.data_ptr(), output.data_ptr(), None if permutation is None else permutation.data_ptr(),
                                         None if factors is None else factors.data_ptr(), m, topk, output.shape[1], input.shape[0],
                                         dtype_code(output.dtype), stream_ptr(output.device)))


def _expert_major_block_m(rows: int, num_experts: int) -> int:
    """Slots per block of the grouped GEMM op from the mean rows per expert (the op hands the kernel per-row scales,
    for which the 64- and 128-row streaming forms were measured ahead of the 256-row one up to about 96 rows)."""
    per_expert = (rows + num_experts - 1) // max(num_experts, 1)
    for limit, bm in ((4, 16), (22, 32), (48, 64), (96, 128)):
        if per_expert <= limit:
            return bm
    return 256


def fp8_blockwise_scaled_grouped_mm(output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a, scales_b,
                                    stride_a, stride_b, stride_c, layout_sfa, layout_sfb, problem_sizes, expert_offsets,
                                    workspace) -> None:
    """Reference: sgl-kernel/python/sgl_kernel/moe.py:175-214 (csrc/moe/fp8_blockwise_moe_kernel.cu).  For every expert e:
    output[rows_e] = a[rows_e] @ b[e] with 1x128 scales on a and 128x128 scales on b, rows_e = expert_offsets[e] ..
    + problem_sizes[e, 0].  a e4m3fn [rows, K]; b e4m3fn [E, K, N] column-major per expert (a [E, N, K] weight
    transposed); scales_a float32 [rows, K/128]; scales_b float32 [E, K/128, N/128] with any strides (the reference
    passes the [E, N/128, K/128] checkpoint tensor transposed), or, when N/128 != K/128 makes the shape unambiguous, the
    un-transposed [E, N/128, K/128] tensor; output bf16 / fp16 [rows, N].  The pointer arrays, stride
    vectors, scale-layout buffers and the workspace serve the reference's CUTLASS launcher and are ignored here:
    the grouped kernel takes a block table built on the device from expert_offsets and problem_sizes."""
    require_cuda(output, a, b, scales_a, scales_b, problem_sizes, expert_offsets)
    if a.dim() != 2 or b.dim() != 3 or output.dim() != 2:
        raise RuntimeError("fp8_blockwise_scaled_grouped_mm: a [rows, K], b [E, K, N], output [rows, N]")
    E, K, N = b.shape
    if b.stride(1) != 1 and K > 1:
        raise RuntimeError("fp8_blockwise_scaled_grouped_mm: b must be column-major per expert (K contiguous)")
    kb, nb = (K + 127) // 128, (N + 127) // 128
    if scales_b.dim() != 3 or scales_b.shape[0] != E:
        raise RuntimeError("fp8_blockwise_scaled_grouped_mm: scales_b must be [E, K/128, N/128]")
    # the op's own layout is [E, K/128, N/128] whatever the strides (a square tensor is always read that way); a tensor
    # whose shape can only be the un-transposed [E, N/128, K/128] checkpoint tensor is taken as that
    if tuple(scales_b.shape[1:]) == (kb, nb):
        bs = scales_b.transpose(1, 2)
    elif tuple(scales_b.shape[1:]) == (nb, kb):
        bs = scales_b
    else:
        raise RuntimeError("fp8_blockwise_scaled_grouped_mm: scales_b must be the [E, N/128, K/128] tensor or its transpose")
    if problem_sizes.dtype != torch.int32 or problem_sizes.shape != (E, 3) or not problem_sizes.is_contiguous():
        raise RuntimeError("fp8_blockwise_scaled_grouped_mm: problem_sizes must be contiguous int32 [E, 3]")
    if expert_offsets.dtype != torch.int32 or expert_offsets.numel() < E or not expert_offsets.is_contiguous():
        raise RuntimeError("fp8_blockwise_scaled_grouped_mm: expert_offsets must be contiguous int32 with E entries")
    rows = a.shape[0]
    if rows == 0:
        return
    block_m = _expert_major_block_m(rows, E)
    cap = (rows + min(rows, E) * (block_m - 1)) // block_m * block_m
    table = torch.empty((cap + cap // block_m + 1,), device=a.device, dtype=torch.int32)
    sorted_ids, expert_ids, post_pad = table[:cap], table[cap:cap + cap // block_m], table[cap + cap // block_m:]
    check(lib.fp8k_moe_blocks_from_offsets(expert_offsets.data_ptr(), problem_sizes.data_ptr(), E, rows, block_m,
                                           sorted_ids.data_ptr(), cap, expert_ids.data_ptr(), cap // block_m, post_pad.data_ptr(),
                                           stream_ptr(a.device)))
    moe_block_gemm(a, b.transpose(1, 2), output, scales_a, bs, None, sorted_ids, expert_ids, post_pad, False, 1, block_m, rows)


def moe_slot_blocks(topk_ids: torch.Tensor, expert_offsets: torch.Tensor, problem_sizes: torch.Tensor,
                    output_permutation: torch.Tensor, block_m: int):
    """Block table of the grouped GEMM for the expert-major layout, holding token SLOTS (include/fp8k.h:
    fp8k_moe_slot_blocks_from_offsets): from what prepare_moe_input wrote (expert_offsets, problem_sizes,
    output_permutation = slot -> row) returns (sorted_token_ids, expert_ids, num_tokens_post_padded) in the form
    moe_align_block_size produces, so moe_block_gemm gathers token slot // topk from the un-shuffled activations."""
    require_cuda(topk_ids, expert_offsets, problem_sizes, output_permutation)
    E = problem_sizes.shape[0]
    slots = topk_ids.numel()
    for t, name, need in ((topk_ids, "topk_ids", slots), (expert_offsets, "expert_offsets", E),
                          (problem_sizes, "problem_sizes", 3 * E), (output_permutation, "output_permutation", slots)):
        if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < need:
            raise RuntimeError("moe_slot_blocks: %s must be contiguous int32 with at least %d entries" % (name, need))
    cap = max((slots + min(slots, E) * (block_m - 1)) // block_m * block_m, block_m)
    table = torch.empty((cap + cap // block_m + 1,), device=topk_ids.device, dtype=torch.int32)
    sorted_ids, expert_ids, post_pad = table[:cap], table[cap:cap + cap // block_m], table[cap + cap // block_m:]
    check(lib.fp8k_moe_slot_blocks_from_offsets(expert_offsets.data_ptr(), problem_sizes.data_ptr(), E, topk_ids.data_ptr(),
                                                output_permutation.data_ptr(), slots, block_m, sorted_ids.data_ptr(), cap,
                                                expert_ids.data_ptr(), cap // block_m, post_pad.data_ptr(),
                                                stream_ptr(topk_ids.device)))
    return sorted_ids, expert_ids, post_pad


def moe_block_gemm_silu_quant(A, B, A_scale_sorted, B_scale, out_q, out_s, sorted_token_ids, expert_ids,
                              num_tokens_post_padded, top_k: int, num_valid_tokens: int, act_dtype: torch.dtype,
                              eps: float = 1e-10, balanced: bool = False) -> None:
    """Grouped GEMM 1 of the fused MoE layer (256-slot blocks) with silu_and_mul and the group requantisation inside its
    write-out (include/fp8k.h: fp8k_moe_block_gemm_silu_quant).  A e4m3fn [rows, K]; B e4m3fn [E, 2 I, K] (gate rows,
    then up rows); A_scale_sorted float32 [len(sorted_token_ids), K/128] as moe_sort_scales returns it; B_scale float32
    [E, 2 I/128, K/128]; out_q e4m3fn [num_valid_tokens, I]; out_s float32 [len(sorted_token_ids), I/128] in the same
    sorted layout (column-major: one row of the underlying [I/128, len] buffer per column block)."""
    require_cuda(A, B, A_scale_sorted, B_scale, out_q, out_s, sorted_token_ids, expert_ids, num_tokens_post_padded)
    if A.dtype != FP8_DTYPE or B.dtype != FP8_DTYPE or out_q.dtype != FP8_DTYPE:
        raise RuntimeError("moe_block_gemm_silu_quant: A, B and out_q must be Float8_e4m3fn")
    if A_scale_sorted.dtype != torch.float32 or B_scale.dtype != torch.float32 or out_s.dtype != torch.float32:
        raise RuntimeError("moe_block_gemm_silu_quant: scales must be Float32")
    if B.dim() != 3 or A.dim() != 2 or out_q.dim() != 2:
        raise RuntimeError("moe_block_gemm_silu_quant: A [rows,K], B [E,2I,K], out_q [slots,I]")
    E, N, K = B.shape
    I = N // 2
    cap = sorted_token_ids.numel()
    kb = (K + 127) // 128
    if N % 256 != 0 or A.shape[1] != K or A.stride(1) != 1 or B.stride(2) != 1:
        raise RuntimeError("moe_block_gemm_silu_quant: N must be 2 I with I a multiple of 128, K contiguous")
    if tuple(A_scale_sorted.shape) != (cap, kb) or A_scale_sorted.stride(0) != 1:
        raise RuntimeError("moe_block_gemm_silu_quant: A_scale_sorted must be the [len(sorted_token_ids), K/128] view of moe_sort_scales")
    if tuple(out_s.shape) != (cap, I // 128) or out_s.stride(0) != 1 or (I // 128 > 1 and out_s.stride(1) < cap):
        raise RuntimeError("moe_block_gemm_silu_quant: out_s must be a [len(sorted_token_ids), I/128] view with the slots contiguous")
    if tuple(out_q.shape) != (num_valid_tokens, I) or out_q.stride(1) != 1:
        raise RuntimeError("moe_block_gemm_silu_quant: out_q must be [num_valid_tokens, I] with I contiguous")
    if tuple(B_scale.shape) != (E, N // 128, kb):
        raise RuntimeError("moe_block_gemm_silu_quant: B_scale shape does not match B")
    if A.shape[0] * top_k < num_valid_tokens:
        raise RuntimeError("moe_block_gemm_silu_quant: A has too few rows for num_valid_tokens / top_k")
    for t in (sorted_token_ids, expert_ids, num_tokens_post_padded):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("moe_block_gemm_silu_quant: index tensors must be contiguous int32")
    if expert_ids.numel() * 256 < cap - (cap % 256):
        raise RuntimeError("moe_block_gemm_silu_quant: expert_ids is shorter than sorted_token_ids / 256")
    check(lib.fp8k_moe_block_gemm_silu_quant(
        A.data_ptr(), B.data_ptr(), A_scale_sorted.data_ptr(), B_scale.data_ptr(), out_q.data_ptr(), out_s.data_ptr(),
        sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(), cap, num_valid_tokens, top_k, E,
        N, K, A.stride(0), A_scale_sorted.stride(1) if kb > 1 else cap, B.stride(0), B.stride(1), B_scale.stride(0),
        B_scale.stride(1), B_scale.stride(2), out_q.stride(0), out_s.stride(1) if I // 128 > 1 else cap, float(eps),
        dtype_code(act_dtype), 1 if balanced else 0, stream_ptr(A.device)))


def moe_fused_gate(
    input_tensor: torch.Tensor,
    bias: torch.Tensor,
    num_expert_group: int,
    topk_group: int,
    topk: int,
    num_fused_shared_experts: int = 0,
    routed_scaling_factor: float = 0,
    apply_routed_scaling_factor_on_output: bool = False,
):
    """Reference: sgl-kernel/python/sgl_kernel/moe.py:105-137 (csrc/moe/moe_fused_gate.cu).  Hierarchical top-k:
    groups are ranked by the sum of their two best biased sigmoid scores, the best `topk_group` groups stay, the
    `topk` best experts among them are taken; returns (weights float32 [rows, topk], ids int32 [rows, topk]).
    `topk` includes `num_fused_shared_experts` trailing shared-expert entries."""
    require_cuda(input_tensor, bias)
    if input_tensor.dtype != bias.dtype:
        raise RuntimeError("input and bias should have the same dtype")
    if input_tensor.dim() != 2 or bias.dim() != 1 or bias.shape[0] != input_tensor.shape[1]:
        raise RuntimeError("moe_fused_gate: input [num_rows, num_experts], bias [num_experts]")
    if not (input_tensor.is_contiguous() and bias.is_contiguous()):
        raise RuntimeError("moe_fused_gate: input and bias must be contiguous")
    rows, experts = input_tensor.shape
    output = torch.empty((rows, topk), device=input_tensor.device, dtype=torch.float32)
    indices = torch.empty((rows, topk), device=input_tensor.device, dtype=torch.int32)
    check(
        lib.fp8k_moe_fused_gate(
            input_tensor.data_ptr(), bias.data_ptr(), output.data_ptr(), indices.data_ptr(), rows, experts,
            int(num_expert_group), int(topk_group), int(topk), int(num_fused_shared_experts),
            float(routed_scaling_factor), 1 if apply_routed_scaling_factor_on_output else 0,
            dtype_code(input_tensor.dtype), stream_ptr(input_tensor.device),
        )
    )
    return output, indices
