"""Entry points of ``sglang.srt.layers.quantization.fp8_utils`` on this path: the callables
``Fp8LinearMethod.apply`` (fp8.py:471-527) and ``W8A8Fp8LinearMethod.apply`` (w8a8_fp8.py:182-194)
reach.  There is a single backend, so the dispatcher always returns the same function.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Tuple

import torch

from . import custom_ops as _ops
from .sgl_kernel import mark_ue8m0, unpack_ue8m0_weight_scales  # noqa: F401  (re-exported for weight loading)
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
    """Reference: cutlass_/triton_w8a8_block_fp8_linear, fp8_utils.py:196-226,306-326, and the pre-quantised input of the
    ROCm variant (:268-304; Fp8LinearMethod.apply hands over `(x_q, x_scale)` as input / input_scale, fp8.py:500-508).

    input [..., K] bf16/fp16; weight e4m3fn [N,K]; weight_scale float32 [ceil(N/128), ceil(K/128)].
    Flatten -> per-token-group quant (column-major scales) -> block GEMM -> + bias -> reshape.
    With input_scale the input is e4m3fn already (quantised upstream in groups of block_size[1], scales float32
    [tokens, K/128] in any strides); the result is bf16, as in the reference.
    """
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[0]]
    if input_scale is not None:
        if input_2d.dtype != fp8_dtype:
            raise RuntimeError("w8a8_block_fp8_linear: input_scale given, so input must be float8_e4m3fn already")
        q_input, x_scale = input_2d, input_scale.view(-1, input_scale.shape[-1])
        out_dtype = torch.bfloat16
    else:
        q_input, x_scale = sglang_per_token_group_quant_fp8(input_2d, block_size[1], column_major_scales=True)
        out_dtype = input_2d.dtype
    output = w8a8_block_fp8_matmul(q_input, weight, x_scale, weight_scale, block_size, output_dtype=out_dtype)
    if bias is not None:
        output = output + bias
    return output.to(dtype=out_dtype).view(*output_shape)


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


# --------------------------------------------------------------------------------------------
# weight-side transforms (run once, after loading; plain tensor ops on whatever device holds the weights)
# --------------------------------------------------------------------------------------------

_FP8_MAX = 448.0


def input_to_float8(x: torch.Tensor, dtype: torch.dtype = fp8_dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_utils.py:356-372 - one scale for the whole tensor: q = sat(x * 448/amax), returns
    (q, amax/448 as a float32 scalar tensor); amax is floored at 1e-12."""
    lo, hi = x.aminmax()
    amax = torch.maximum(lo.abs(), hi.abs()).float().clamp(min=1e-12)
    to_q = _FP8_MAX / amax
    q = (x.float() * to_q).clamp(min=-_FP8_MAX, max=_FP8_MAX).to(dtype).contiguous()
    return q, to_q.float().reciprocal()


def block_quant_dequant(x_q_block: torch.Tensor, x_s: torch.Tensor, block_size: List[int], dtype: torch.dtype) -> torch.Tensor:
    """Reference: fp8_utils.py:418-438 - [..., n, k] block-quantised values times their [..., ceil(n/bn), ceil(k/bk)]
    scales, in float32, cast to `dtype`."""
    bn, bk = block_size
    n, k = x_q_block.shape[-2:]
    rows = torch.arange(n, device=x_s.device) // bn
    cols = torch.arange(k, device=x_s.device) // bk
    full = x_s.index_select(-2, rows).index_select(-1, cols)
    return (x_q_block.to(torch.float32) * full).to(dtype)


def _tensor_quant(x_f32: torch.Tensor, like: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    # the GPU path quantises with the library's per-tensor op, as the reference does with scaled_fp8_quant
    if x_f32.is_cuda and x_f32.dim() == 2:
        return scaled_fp8_quant(x_f32.contiguous())
    return input_to_float8(x_f32, dtype=like.dtype)


def block_quant_to_tensor_quant(x_q_block: torch.Tensor, x_s: torch.Tensor, block_size: List[int]) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_utils.py:375-415 - [n, k] block-quantised weight -> the same weight with one scale."""
    n, k = x_q_block.shape
    assert x_s.shape[0] == (n + block_size[0] - 1) // block_size[0]
    assert x_s.shape[1] == (k + block_size[1] - 1) // block_size[1]
    return _tensor_quant(block_quant_dequant(x_q_block, x_s, block_size, torch.float32), x_q_block)


def channel_quant_to_tensor_quant(x_q_channel: torch.Tensor, x_s: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_utils.py:589-599 - per-channel scales [n, 1] -> one scale."""
    return _tensor_quant(x_q_channel.to(torch.float32) * x_s, x_q_channel)


def per_block_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_utils.py:568-582 - 128x128 block quantisation with power-of-two scales:
    scale = 2^ceil(log2(max(amax, 1e-4) / 448)), q = e4m3fn(x / scale).  x [m, n] -> (q [m, n], scale [ceil(m/128), ceil(n/128)])."""
    assert x.dim() == 2
    m, n = x.shape
    mt, nt = (m + 127) // 128, (n + 127) // 128
    padded = torch.zeros((mt * 128, nt * 128), dtype=x.dtype, device=x.device)
    padded[:m, :n] = x
    tiles = padded.view(mt, 128, nt, 128)
    amax = tiles.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    scale = ceil_to_ue8m0(amax / _FP8_MAX)
    q = (tiles * (1.0 / scale)).to(torch.float8_e4m3fn).view(mt * 128, nt * 128)[:m, :n].contiguous()
    return q, scale.view(mt, nt)


def quant_weight_ue8m0(weight_dequant: torch.Tensor, weight_block_size: List[int]) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_utils.py:479-502 - per_block_cast_to_fp8 over the last two dimensions of a bf16 weight."""
    assert list(weight_block_size) == [128, 128]
    assert weight_dequant.dtype == torch.bfloat16, f"{weight_dequant.dtype=} {weight_dequant.shape=}"
    *batch, n, k = weight_dequant.shape
    if not batch:
        q, sc = per_block_cast_to_fp8(weight_dequant)
        return q, mark_ue8m0(sc.contiguous(), check=False)  # powers of two by construction
    parts = [per_block_cast_to_fp8(w) for w in weight_dequant.reshape(-1, n, k)]
    q = torch.stack([p[0] for p in parts]).view(*batch, n, k)
    sc = torch.stack([p[1] for p in parts]).view(*batch, (n + 127) // 128, (k + 127) // 128)
    return q, mark_ue8m0(sc.contiguous(), check=False)  # powers of two by construction


def requant_weight_ue8m0(weight: torch.Tensor, weight_scale_inv: torch.Tensor, weight_block_size: List[int]) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: fp8_utils.py:453-476 - dequantise a block-FP8 weight to bf16 and quantise it again with
    power-of-two block scales.  The reference then repacks the scales into DeepGEMM's int32 layout; here they stay
    float32 [.., ceil(n/128), ceil(k/128)] powers of two, declared as such (sgl_kernel.mark_ue8m0), which is what the
    UE8M0 GEMM of this library takes."""
    assert list(weight_block_size) == [128, 128]
    deq = block_quant_dequant(weight, weight_scale_inv, weight_block_size, torch.bfloat16)
    return quant_weight_ue8m0(deq, weight_block_size)


def requant_weight_ue8m0_inplace(weight: torch.nn.Parameter, weight_scale_inv: torch.nn.Parameter,
                                 weight_block_size: List[int]) -> None:
    """Reference: fp8_utils.py:441-450 - requant_weight_ue8m0 written back into the two parameters."""
    assert isinstance(weight, torch.nn.Parameter)
    assert isinstance(weight_scale_inv, torch.nn.Parameter)
    q, s = requant_weight_ue8m0(weight.data.to(weight_scale_inv.device), weight_scale_inv.data, weight_block_size)
    weight.data = q
    weight_scale_inv.data = s
    mark_ue8m0(weight_scale_inv, check=False)  # the parameter object: it lives as long as the layer does


def transform_scale_ue8m0(sf: torch.Tensor, mn: int) -> torch.Tensor:
    """Power-of-two block scales float32 [.., ceil(mn/128), kb] -> the packed layout DeepGEMM is handed: one row per weight
    row, four exponent bytes to an int32 word (K block 4j+i in byte i of word j), [.., mn, ceil(kb/4)] with the mn
    dimension contiguous and padded to a multiple of 4.  Reference: fp8_utils.py:510-515 (which calls the DeepGEMM
    layout helper for the second half).  Accepted as weight scales by w8a8_block_fp8_matmul and the grouped entry points."""
    if sf.dtype != torch.float32:
        raise RuntimeError("transform_scale_ue8m0: float32 scales expected")
    rows = sf.index_select(-2, torch.arange(mn, device=sf.device) // 128)
    exp = (rows.contiguous().view(torch.int32) >> 23) & 0xFF
    kb = exp.shape[-1]
    if kb % 4:
        exp = torch.cat([exp, exp.new_zeros(exp.shape[:-1] + (4 - kb % 4,))], dim=-1)
    exp = exp.view(exp.shape[:-1] + (-1, 4))
    words = exp[..., 0] | (exp[..., 1] << 8) | (exp[..., 2] << 16) | (exp[..., 3] << 24)  # [.., mn, kb4]
    aligned = (mn + 3) // 4 * 4
    out = torch.zeros(words.shape[:-2] + (words.shape[-1], aligned), dtype=torch.int32, device=sf.device)
    out[..., :mn] = words.transpose(-1, -2)
    return out.transpose(-1, -2)[..., :mn, :]


def transform_scale_ue8m0_inplace(param: torch.nn.Parameter, mn: int) -> None:
    """Reference: fp8_utils.py:505-507."""
    param.data = transform_scale_ue8m0(param.data, mn=mn)


def inverse_transform_scale_ue8m0(sf_packed: torch.Tensor, mn: int) -> torch.Tensor:
    """Packed weight scales [.., mn, ceil(kb/4)] back to float32 powers of two [.., mn/128, 4 ceil(kb/4)], with the
    reference's consistency check (the 128 rows of a block must carry the same words, and packing the result again
    must give the input).  Reference: fp8_utils.py:518-565."""
    if sf_packed.dtype != torch.int32 or mn % 128 != 0 or sf_packed.shape[-2] != mn:
        raise RuntimeError("inverse_transform_scale_ue8m0: int32 [.., mn, k/4] with mn a multiple of 128 expected")
    k = sf_packed.shape[-1] * 4
    sf = unpack_ue8m0_weight_scales(sf_packed, k * 128)
    assert torch.equal(transform_scale_ue8m0(sf, mn), sf_packed), "packed scales are not uniform over their 128-row blocks"
    return sf
