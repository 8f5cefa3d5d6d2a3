"""Entry points of ``sglang.srt.layers.quantization.fp8_kernel`` on this path.

gfx950 is OCP FP8: fp8_dtype is float8_e4m3fn and fp8_max is 448 (the reference's fnuz branch,
fp8_kernel.py:81-95, applies to gfx94x only and is not reproduced).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import custom_ops as _ops
from . import sgl_kernel as _k

fp8_dtype = torch.float8_e4m3fn
fp8_max = 448.0
fp8_min = -448.0


def ceil_align(x: int, y: int) -> int:
    return (x + y - 1) // y * y


def create_per_token_group_quant_fp8_output_scale(
    x_shape, device, group_size: int, column_major_scales: bool, scale_tma_aligned: bool, scale_ue8m0: bool
) -> torch.Tensor:
    """Reference: fp8_kernel.py:437-478 - the four scale layouts, returned as strided views."""
    if scale_ue8m0:
        assert column_major_scales and scale_tma_aligned
        *x_batch, x_q_mn, x_q_k = x_shape
        x_s_mn, x_s_k = x_q_mn, x_q_k // 128
        aligned_mn = ceil_align(x_s_mn, 4)
        aligned_k = ceil_align(x_s_k, 4)
        return torch.empty((*x_batch, aligned_k // 4, aligned_mn), device=device, dtype=torch.int).transpose(-1, -2)[
            ..., :x_s_mn, :
        ]
    if column_major_scales:
        if scale_tma_aligned:
            aligned_size = (x_shape[-2] + 3) // 4 * 4
            return torch.empty(
                tuple(x_shape[:-2]) + (x_shape[-1] // group_size, aligned_size), device=device, dtype=torch.float32
            ).transpose(-1, -2)[: x_shape[-2], :]
        return torch.empty(
            (x_shape[-1] // group_size,) + tuple(x_shape[:-1]), device=device, dtype=torch.float32
        ).permute(-1, -2)
    return torch.empty(tuple(x_shape[:-1]) + (x_shape[-1] // group_size,), device=device, dtype=torch.float32)


def sglang_per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_kernel.py:481-531."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    out_shape = (*x.shape[:-1], x.shape[-1] // (2 if fuse_silu_and_mul else 1))
    x_q = torch.empty(out_shape, device=x.device, dtype=fp8_dtype)
    x_s = create_per_token_group_quant_fp8_output_scale(
        x_shape=out_shape,
        device=x.device,
        group_size=group_size,
        column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0,
    )
    if masked_m is not None:
        # masked expert layout [num_experts, max_tokens, hidden]: scales keep their three strides
        if x.dim() != 3:
            raise RuntimeError("masked_m needs a 3-D input [num_experts, max_tokens, hidden]")
        if x.numel() > 0:
            _ops.sgl_per_token_group_quant_8bit(
                x, x_q, x_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, fuse_silu_and_mul, masked_m, enable_v2=enable_v2
            )
        return x_q, x_s
    if x.shape[0] > 0:
        s2 = x_s if x_s.dim() == 2 else x_s.reshape(-1, x_s.shape[-1]) if not (column_major_scales or scale_ue8m0) else x_s
        if s2.dim() != 2:
            raise RuntimeError("column-major scale layouts need a 2-D input")
        _ops.sgl_per_token_group_quant_8bit(
            x, x_q, s2, group_size, eps, fp8_min, fp8_max, scale_ue8m0, fuse_silu_and_mul, masked_m, enable_v2=enable_v2
        )
    return x_q, x_s


def per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: torch.dtype = fp8_dtype,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_kernel.py:219-327 (the Triton entry point); same kernel as the sgl-kernel one here."""
    if dtype != fp8_dtype:
        raise RuntimeError("per_token_group_quant_fp8: only float8_e4m3fn is built on gfx950")
    return sglang_per_token_group_quant_fp8(
        x, group_size, eps, column_major_scales=column_major_scales, scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0,
    )


def sglang_per_token_quant_fp8(x: torch.Tensor, dtype: torch.dtype = fp8_dtype):
    """Reference: fp8_kernel.py:577-593 - dynamic per-token quant, scales [M,1] float32."""
    assert x.is_contiguous(), "`x` is not contiguous"
    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    x_s = torch.empty(x.shape[0], 1, device=x.device, dtype=torch.float32)
    _ops.sgl_per_token_quant_fp8(x, x_q, x_s)
    return x_q, x_s


def scaled_fp8_quant(
    input: torch.Tensor,
    scale: Optional[torch.Tensor] = None,
    num_token_padding: Optional[int] = None,
    use_per_token_if_dynamic: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_kernel.py:1431-1468 (sgl-kernel branch): static per-tensor when `scale` is given,
    else dynamic per-token or per-tensor."""
    assert input.ndim == 2, f"Expected 2D input tensor, got {input.ndim}D"
    shape = input.shape
    if num_token_padding:
        shape = (max(num_token_padding, input.shape[0]), shape[1])
    output = torch.empty(shape, device=input.device, dtype=fp8_dtype)
    if scale is None:
        if use_per_token_if_dynamic:
            scale = torch.empty((shape[0], 1), device=input.device, dtype=torch.float32)
            _ops.sgl_per_token_quant_fp8(input, output[: input.shape[0]], scale[: input.shape[0]])
        else:
            scale = torch.zeros(1, device=input.device, dtype=torch.float32)
            _ops.sgl_per_tensor_quant_fp8(input, output[: input.shape[0]], scale, is_static=False)
    else:
        assert scale.numel() == 1, f"Expected scalar scale, got numel={scale.numel()}"
        _ops.sgl_per_tensor_quant_fp8(input, output[: input.shape[0]], scale, is_static=True)
    return output, scale


def static_quant_fp8(x: torch.Tensor, x_s: torch.Tensor, repeat_scale: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_kernel.py:639-692 (a Triton kernel there): q = cast(clamp(x * (1 / x_s), -448, 448)) with the
    given per-tensor scale - the arithmetic of the static branch of sgl_per_tensor_quant_fp8, which runs it here.
    repeat_scale: the scale is returned once per row ([rows, 1]) instead of as given."""
    assert x.is_contiguous(), "`x` is not contiguous"
    assert x_s.numel() == 1, "only supports per-tensor scale"
    x_q = torch.empty_like(x, device=x.device, dtype=fp8_dtype)
    scale = x_s.reshape(1).to(torch.float32)
    if x.numel() > 0:
        _ops.sgl_per_tensor_quant_fp8(x.view(-1, x.shape[-1]), x_q.view(-1, x.shape[-1]), scale, is_static=True)
    if repeat_scale:
        return x_q, scale.expand(x.numel() // max(x.shape[-1], 1)).reshape(-1, 1).contiguous()
    return x_q, x_s


def sglang_per_token_group_quant_8bit(
    x: torch.Tensor,
    group_size: int,
    dst_dtype: torch.dtype,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_kernel.py:535-574.  The int8 destination of the reference is another quantisation path and is not
    built here."""
    if dst_dtype != fp8_dtype:
        raise RuntimeError("sglang_per_token_group_quant_8bit: only float8_e4m3fn is built on gfx950")
    return sglang_per_token_group_quant_fp8(
        x, group_size, eps, column_major_scales=column_major_scales, scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0, fuse_silu_and_mul=fuse_silu_and_mul, masked_m=masked_m, enable_v2=enable_v2,
    )


def per_token_group_quant_8bit(
    x: torch.Tensor,
    group_size: int,
    dst_dtype: torch.dtype,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_kernel.py:404-434 (the Triton entry point, with its fused silu_and_mul branch :330-401); the same
    kernel as the sgl-kernel entry point here."""
    return sglang_per_token_group_quant_8bit(x, group_size, dst_dtype, eps, column_major_scales, scale_tma_aligned,
                                             scale_ue8m0, fuse_silu_and_mul, masked_m)


def per_tensor_quant_mla_fp8(x: torch.Tensor, x_s_out: torch.Tensor, eps: float = 1e-12) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_kernel.py:1221-1266 - tensor-wise quantisation specialised for the MLA absorbed products: x is a
    (possibly transposed) [num_head, num_seq, head_size] view, the result is contiguous.  x_s_out: one float32 that
    must be zero on entry (the maximum is accumulated atomically) and receives max(absmax, eps) / 448."""
    assert x.dim() == 3, "`x` is not a 3d-tensor"
    assert x_s_out.shape == (1,) and x_s_out.dtype == torch.float32 and x_s_out.device == x.device
    x_q = x.new_empty(x.size(), dtype=fp8_dtype)
    if x.numel() > 0:
        _ops.tensor_quant_mla(x, x_q, x_s_out, eps)
    return x_q, x_s_out


def per_token_group_quant_mla_deep_gemm_masked_fp8(
    x: torch.Tensor, group_size: int = 128, eps: float = 1e-12, dtype: torch.dtype = fp8_dtype
):
    """Reference: fp8_kernel.py:1319-1362 - per-token-group quantisation of a [b, m, k] tensor into the masked layout
    of the grouped GEMM: x_q [b, ceil256(m), k], scales [b, ceil256(m), k/g] stored as [b, k/g, ceil256(m)] (m
    contiguous), masked_m [b] = m.  Returns (x_q, scales, masked_m, m, aligned_m); rows at or past m are not written.
    x is first laid out as [b, aligned_m, k] (one copy, which also takes care of transposed inputs); the quantisation
    is the masked form of the group quant kernel.  An all-zero group gets the scale of the eps clamp in the input
    type (bf16(eps) / 448 for a bf16 input, where the reference's Triton kernel has eps / 448); its bytes are zero."""
    assert x.dim() == 3, "`x` is not a 3d-tensor"
    if dtype != fp8_dtype:
        raise RuntimeError("per_token_group_quant_mla_deep_gemm_masked_fp8: only float8_e4m3fn is built on gfx950")
    b, m, k = x.shape
    aligned_m = (m + 255) // 256 * 256  # 256 is the largest row block of the grouped GEMM
    num_tiles_k = k // group_size
    assert num_tiles_k * group_size == k, f"k % {group_size} must be zero"
    x_q = x.new_empty((b, aligned_m, k), dtype=dtype)
    x_s = x.new_empty((b, num_tiles_k, aligned_m), dtype=torch.float32)
    masked_m = torch.full((b,), m, dtype=torch.int32, device=x.device)
    if b * m > 0:
        if m == aligned_m and x.is_contiguous():
            xp = x
        else:
            xp = x.new_empty((b, aligned_m, k))
            xp[:, :m].copy_(x)
        _ops.sgl_per_token_group_quant_8bit(xp, x_q, x_s.transpose(1, 2), group_size, eps, fp8_min, fp8_max, False, False, masked_m)
    return x_q, x_s.transpose(1, 2), masked_m, m, aligned_m


def w8a8_block_fp8_matmul(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.float16,
) -> torch.Tensor:
    """Reference: fp8_kernel.py:1153-1168, checks :1003-1048.

    A e4m3fn [..., K]; B e4m3fn [N, K] contiguous; As float32 [..., ceil(K/bk)]; Bs float32
    [ceil(N/bn), ceil(K/bk)]; block_size must be [128, 128] on this path.

    UE8M0 scales (reference: the int32 forms admitted at fp8_kernel.py:1018-1043 and consumed by the DeepGEMM path,
    fp8_utils.py:229-268): As may be the packed tensor that the group quant returns with scale_ue8m0=True (int32
    [M, ceil(K/128/4)]), Bs the packed weight scales (int32 [N, ceil(K/128/4)], the rows of a block alike).  When
    both operands' scales are known to be powers of two - Bs packed, or float32 and declared with
    sgl_kernel.mark_ue8m0 (requant_weight_ue8m0 / quant_weight_ue8m0 return it so) - the matrix core applies the
    exponents itself.  Packed activation scales next to ordinary float32 weight scales are expanded to floats and
    take the float-scale kernels: a float scale is never read as a bare exponent.
    """
    assert len(block_size) == 2
    block_n, block_k = block_size
    if block_n != 128 or block_k != 128:
        raise RuntimeError("w8a8_block_fp8_matmul: only block_size [128, 128] is built on this path")
    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1] and A.is_contiguous()
    packed = As.dtype == torch.int32
    assert packed or (A.shape[-1] + block_k - 1) // block_k == As.shape[-1]
    assert B.ndim == 2 and B.is_contiguous() and Bs.ndim == 2
    N, K = B.shape
    kb = (K + block_k - 1) // block_k
    bs_pow2 = False
    if Bs.dtype == torch.int32:
        assert Bs.shape[0] == N and Bs.shape[1] == (kb + 3) // 4
        Bs = _k.unpack_ue8m0_weight_scales(Bs, K)
        bs_pow2 = True
    else:
        assert (N + block_n - 1) // block_n == Bs.shape[0]
        assert kb == Bs.shape[1]
        bs_pow2 = _k.is_ue8m0(Bs)
    M = A.numel() // A.shape[-1]
    C_shape = A.shape[:-1] + (N,)
    A2 = A.reshape(M, K)
    if packed:
        if As.dim() != 2:
            raise RuntimeError("w8a8_block_fp8_matmul: packed UE8M0 scales need a 2-D activation")
        if Bs.dtype != torch.float32:
            raise RuntimeError("w8a8_block_fp8_matmul: weight scales must be float32 or packed int32 UE8M0")
        if bs_pow2:
            return _ops.block_gemm_nk_ue8m0(A2, B, As, Bs, output_dtype).reshape(C_shape)
        return _ops.block_gemm_nk(A2, B, _k.unpack_ue8m0_scales(As, kb), Bs, output_dtype).reshape(C_shape)
    As2 = As.reshape(M, As.shape[-1])
    if As2.dtype != torch.float32 or Bs.dtype != torch.float32:
        raise RuntimeError("w8a8_block_fp8_matmul: scales must be float32 (or packed int32 UE8M0 scales)")
    out = _ops.block_gemm_nk(A2, B, As2, Bs, output_dtype)
    return out.reshape(C_shape)


# the reference dispatches between a Triton and a DeepGEMM implementation of the same op (fp8_kernel.py:1051-1169); one
# implementation here
w8a8_block_fp8_matmul_triton = w8a8_block_fp8_matmul
w8a8_block_fp8_matmul_deepgemm = w8a8_block_fp8_matmul
