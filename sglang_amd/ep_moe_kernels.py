"""Masked-layout MoE helpers of the DeepEP low-latency path on this library's kernels.

Reference: python/sglang/srt/layers/moe/ep_moe/kernels.py:364-429 (`silu_and_mul_masked_post_quant_fwd`, a Triton
kernel there).  Together with `deep_gemm_wrapper.grouped_gemm_nt_f8f8bf16_masked` these are the three compute steps
of the masked expert runner (moe_runner/deep_gemm.py): grouped GEMM, silu_and_mul + requant, grouped GEMM.
"""
import torch

from . import custom_ops as _ops
from .fp8_kernel import fp8_max, fp8_min


def silu_and_mul_masked_post_quant_fwd(
    input: torch.Tensor,
    output: torch.Tensor,
    output_scale: torch.Tensor,
    quant_group_size: int,
    masked_m: torch.Tensor,
    scale_ue8m0: bool = False,
) -> None:
    """input [expert_num, token_num_padded, 2*hidden] bf16/fp16; output [expert_num, token_num_padded, hidden]
    float8_e4m3fn; output_scale float32 [expert_num, token_num_padded, hidden // group] in any strides; masked_m
    int32 [expert_num].  Rows at or past masked_m[e] are left untouched.  The values quantised are
    T(T(silu(gate)) * up) in the input type T, the scale is max(amax, 1e-10) / 448, as in the reference kernel."""
    assert input.is_contiguous()
    assert output.dtype == torch.float8_e4m3fn
    assert output.is_contiguous()
    assert len(input.shape) == 3
    assert input.shape[0] == masked_m.shape[0]
    assert input.shape[-1] % 2 == 0
    assert (input.shape[-1] // 2) % quant_group_size == 0
    if scale_ue8m0 and quant_group_size != 128:
        raise RuntimeError("silu_and_mul_masked_post_quant_fwd: UE8M0 scales are built for groups of 128")
    # scale_ue8m0 with a float32 output_scale: the kernel stores 2^ceil(log2(amax / 448)) as a float (reference kernel
    # :348-350)
    _ops.sgl_per_token_group_quant_8bit(input, output, output_scale, quant_group_size, 1e-10, fp8_min, fp8_max, scale_ue8m0,
                                        True, masked_m.to(torch.int32))


def tma_align_input_scale(input_scale: torch.Tensor) -> torch.Tensor:
    """Float32 scales [m, k/128] copied into column-major storage with the m dimension padded to a multiple of 4
    (16 bytes), returned as a [m, k/128] view.  Reference: ep_moe/kernels.py:896-968 (a Triton copy kernel there).  The
    grouped entry points of this library read scales through their strides and do not need the copy; it is here for
    callers that make it."""
    assert input_scale.dim() == 2
    m, kb = input_scale.shape
    out = torch.empty((kb, (m + 3) // 4 * 4), dtype=input_scale.dtype, device=input_scale.device)
    out[:, :m] = input_scale.t()
    return out.t()[:m]
