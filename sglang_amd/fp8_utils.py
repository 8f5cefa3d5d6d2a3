"""Entry points of ``sglang.srt.layers.quantization.fp8_utils`` on this path: the callables
``Fp8LinearMethod.apply`` (fp8.py:471-527) and ``W8A8Fp8LinearMethod.apply`` (w8a8_fp8.py:182-194)
reach.  There is a single backend, so the dispatcher always returns the same function.
"""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from . import sgl_kernel as _ops
from .fp8_kernel import (
    fp8_dtype,
    scaled_fp8_quant,
    sglang_per_token_group_quant_fp8,
    sglang_per_token_quant_fp8,
    w8a8_block_fp8_matmul,
)


def ceil_to_ue8m0(x: torch.Tensor) -> torch.Tensor:
    """Reference: fp8_utils.py:585-586."""
    return torch.pow(2.0, torch.ceil(torch.log2(x.abs())))


def w8a8_block_fp8_linear(
    input: torch.Tensor,
    weight: torch.Tensor,
    block_size: List[int],
    weight_scale: torch.Tensor,
    input_scale: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Reference: cutlass_/triton_w8a8_block_fp8_linear, fp8_utils.py:196-226,306-326.

    input [..., K] bf16/fp16; weight e4m3fn [N,K]; weight_scale float32 [ceil(N/128), ceil(K/128)].
    Flatten -> per-token-group quant (column-major scales) -> block GEMM -> + bias -> reshape.
    """
    assert input_scale is None
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[0]]
    q_input, x_scale = sglang_per_token_group_quant_fp8(input_2d, block_size[1], column_major_scales=True)
    output = w8a8_block_fp8_matmul(q_input, weight, x_scale, weight_scale, block_size, output_dtype=input_2d.dtype)
    if bias is not None:
        output = output + bias
    return output.to(dtype=input_2d.dtype).view(*output_shape)


def dispatch_w8a8_block_fp8_linear() -> Callable:
    """Reference: fp8_utils.py:151-161 - chosen once at import there; one path here."""
    return w8a8_block_fp8_linear


def apply_fp8_linear(
    input: torch.Tensor,
    weight: torch.Tensor,
    weight_scale: torch.Tensor,
    input_scale: Optional[torch.Tensor] = None,
    input_scale_ub: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    cutlass_fp8_supported: bool = True,
    use_per_token_if_dynamic: bool = False,
    pad_output: Optional[bool] = None,
    compressed_tensor_quant: bool = False,
) -> torch.Tensor:
    """Reference: fp8_utils.py:639-823, the fp8_scaled_mm route (:683-736).

    weight e4m3fn [K,N] column-major (the layer stores weight.t()); weight_scale per tensor
    (numel 1) or per channel (numel N).  Static per-tensor activation scale when input_scale is
    given, else dynamic per-token (or per-tensor) quantisation.
    """
    input_2d = input.view(-1, input.shape[-1])
    N = weight.shape[1]
    output_shape = [*input.shape[:-1], N]
    if input_scale is not None:
        assert input_scale.numel() == 1
        qinput, x_scale = scaled_fp8_quant(input_2d, input_scale)
    elif use_per_token_if_dynamic or weight_scale.numel() == N:
        qinput, x_scale = sglang_per_token_quant_fp8(input_2d)
    else:
        qinput, x_scale = scaled_fp8_quant(input_2d)
    M = qinput.shape[0]
    if x_scale.numel() == 1:
        x_scale = x_scale.reshape(1).expand(M).contiguous()
    if weight_scale.numel() == 1:
        weight_scale = weight_scale.reshape(1).expand(N).contiguous()
    bias_arg = bias
    if bias is not None and bias.dtype not in (input.dtype, torch.float32):
        bias_arg = bias.to(input.dtype)
    output = _ops.fp8_scaled_mm(qinput, weight, x_scale.reshape(-1), weight_scale.reshape(-1).to(torch.float32),
                                out_dtype=input.dtype, bias=bias_arg)
    return output.view(*output_shape)
