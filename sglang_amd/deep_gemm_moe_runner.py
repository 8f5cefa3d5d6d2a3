"""The expert computation of the DeepGEMM MoE runner on this library's kernels: grouped GEMM w13 -> silu_and_mul +
requantisation -> grouped GEMM w2, in the two token layouts the runner is fed with.

Reference: python/sglang/srt/layers/moe/moe_runner/deep_gemm.py:103-331 (`DeepGemmRunnerCore`: `_run_contiguous_gemm`
for the DeepEP "normal" dispatch, `_run_masked_gemm` for the low-latency dispatch) and :48-58 (the float scales of the
masked input rounded up to UE8M0 exponent bytes).  The permutations in front of and behind the core
(`pre_permute_*`, `post_permute_*`) belong to the dispatchers and are not part of this path.

* contiguous: `hidden_states` e4m3fn [all_tokens, K] with the rows of every expert in one run, `m_indices[i]` = expert of
  row i (-1: padding row, left alone);
* masked: `hidden_states` e4m3fn [experts, m, K], the first `masked_m[e]` rows of expert e are real.

`scale_ue8m0` stands for the reference's process-wide `DEEPGEMM_SCALE_UE8M0` switch: the intermediate activations are
then requantised with power-of-two scales in packed int32 words, and with the weight scales packed as well (the form
the reference prepares, fp8_kernel.py:1018-1043) the grouped GEMMs let the matrix cores apply the scales.  The
activation and the requantisation are one kernel here in both layouts (same bytes and scales as silu_and_mul followed
by the group quant).
"""
from dataclasses import dataclass
from typing import Optional

import torch

from .deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_contig, grouped_gemm_nt_f8f8bf16_masked
from .fp8_kernel import sglang_per_token_group_quant_fp8

DEEPGEMM_SCALE_UE8M0 = False  # default of `scale_ue8m0` (the reference reads its switch from deep_gemm_wrapper)
_GROUP = 128


@dataclass
class DeepGemmMoeQuantInfo:
    """Reference: deep_gemm.py:93-100.  w13_weight e4m3fn [E, 2 I, K], w2_weight e4m3fn [E, K, I]; scales float32
    [E, rows/128, cols/128] or packed UE8M0 words int32 [E, rows, ceil(cols/128/4)]."""
    w13_weight: torch.Tensor
    w2_weight: torch.Tensor
    use_fp8: bool = True
    w13_scale: Optional[torch.Tensor] = None
    w2_scale: Optional[torch.Tensor] = None
    block_shape: Optional[list] = None


def cast_to_e8m0_with_rounding_up(x: torch.Tensor) -> torch.Tensor:
    """Float32 scales [.., m, kb] -> UE8M0 exponent bytes, four K blocks to an int32 word [.., m, ceil(kb/4)] (K block
    4j+i in byte i of word j), every scale rounded UP to a power of two.  Reference: deep_gemm.py:48-58 - same corner
    cases: the largest finite exponent is not pushed into the NaN/Inf one, and a denormal at or below half of the
    smallest normal keeps exponent byte 0."""
    bits = x.to(torch.float32).contiguous().view(torch.int32)
    exp = bits >> 23
    mant = bits & 0x7FFFFF
    up = (mant > 0) & (exp != 0xFE) & ~((exp == 0) & (mant <= 0x400000))
    exp = torch.where(up, exp + 1, exp) & 0xFF
    kb = exp.shape[-1]
    if kb % 4:
        exp = torch.cat([exp, exp.new_zeros(exp.shape[:-1] + (4 - kb % 4,))], dim=-1)
    exp = exp.view(exp.shape[:-1] + (-1, 4))
    return (exp[..., 0] | (exp[..., 1] << 8) | (exp[..., 2] << 16) | (exp[..., 3] << 24)).contiguous()


def _check(quant_info: DeepGemmMoeQuantInfo, k: int) -> None:
    if not quant_info.use_fp8 or quant_info.w13_scale is None or quant_info.w2_scale is None:
        raise RuntimeError("DeepGEMM MoE runner: block-FP8 weights with their scales are required")
    if quant_info.block_shape is not None and list(quant_info.block_shape) != [_GROUP, _GROUP]:
        raise RuntimeError("DeepGEMM MoE runner: block_shape must be [128, 128]")
    w13, w2 = quant_info.w13_weight, quant_info.w2_weight
    if w13.dim() != 3 or w2.dim() != 3 or w13.shape[0] != w2.shape[0] or w13.shape[2] != k or w2.shape[1] != k \
            or w13.shape[1] != 2 * w2.shape[2]:
        raise RuntimeError("DeepGEMM MoE runner: w13 [E, 2 I, K] and w2 [E, K, I] expected")


def _input_scales(scale: torch.Tensor, scale_ue8m0: bool) -> torch.Tensor:
    if scale_ue8m0 and scale.dtype != torch.int32:
        return cast_to_e8m0_with_rounding_up(scale)
    return scale


def run_contiguous_gemm(hidden_states: torch.Tensor, hidden_states_scale: torch.Tensor, m_indices: torch.Tensor,
                        quant_info: DeepGemmMoeQuantInfo, scale_ue8m0: Optional[bool] = None) -> torch.Tensor:
    """Reference: deep_gemm.py:125-206.  Returns bf16 [all_tokens, K]; rows with m_indices == -1 hold no result."""
    ue = DEEPGEMM_SCALE_UE8M0 if scale_ue8m0 is None else bool(scale_ue8m0)
    all_tokens, k = hidden_states.shape
    _check(quant_info, k)
    n = quant_info.w13_weight.shape[1]
    dev = hidden_states.device
    gateup = torch.empty((all_tokens, n), device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_contig((hidden_states, _input_scales(hidden_states_scale, ue)),
                                    (quant_info.w13_weight, quant_info.w13_scale), gateup, m_indices)
    # padding rows of `gateup` were never written: whatever they hold is quantised along and skipped by the next GEMM
    down_in, down_s = sglang_per_token_group_quant_fp8(gateup, _GROUP, column_major_scales=ue, scale_tma_aligned=ue,
                                                       scale_ue8m0=ue, fuse_silu_and_mul=True)
    del gateup
    out = torch.empty((all_tokens, k), device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_contig((down_in, down_s), (quant_info.w2_weight, quant_info.w2_scale), out, m_indices)
    return out


def run_masked_gemm(hidden_states: torch.Tensor, hidden_states_scale: torch.Tensor, masked_m: torch.Tensor,
                    expected_m: int, quant_info: DeepGemmMoeQuantInfo, scale_ue8m0: Optional[bool] = None) -> torch.Tensor:
    """Reference: deep_gemm.py:208-327.  Returns bf16 [experts, m, K]; rows at or past masked_m[e] hold no result."""
    ue = DEEPGEMM_SCALE_UE8M0 if scale_ue8m0 is None else bool(scale_ue8m0)
    groups, m, k = hidden_states.shape
    _check(quant_info, k)
    n = quant_info.w13_weight.shape[1]
    dev = hidden_states.device
    gateup = torch.empty((groups, m, n), device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_masked((hidden_states, _input_scales(hidden_states_scale, ue)),
                                    (quant_info.w13_weight, quant_info.w13_scale), gateup, masked_m, expected_m)
    down_in, down_s = sglang_per_token_group_quant_fp8(gateup, _GROUP, column_major_scales=True, scale_tma_aligned=True,
                                                       scale_ue8m0=ue, fuse_silu_and_mul=True,
                                                       masked_m=masked_m.to(torch.int32))
    del gateup
    out = torch.empty((groups, m, k), device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_masked((down_in, down_s), (quant_info.w2_weight, quant_info.w2_scale), out, masked_m, expected_m)
    return out


class DeepGemmRunnerCore:
    """Reference: deep_gemm.py:103-123.  `runner_input` carries hidden_states, hidden_states_scale, use_masked_gemm and
    either (masked_m, expected_m) or m_indices; returns the expert outputs in the layout of the input."""

    def __init__(self, activation: str = "silu", is_gated: bool = True):
        if activation != "silu" or not is_gated:
            raise RuntimeError("DeepGemmRunnerCore: only the gated silu activation is built on this path")

    def run(self, runner_input, quant_info: DeepGemmMoeQuantInfo, running_state: Optional[dict] = None) -> torch.Tensor:
        if getattr(runner_input, "use_masked_gemm", False):
            return run_masked_gemm(runner_input.hidden_states, runner_input.hidden_states_scale, runner_input.masked_m,
                                   int(runner_input.expected_m), quant_info)
        return run_contiguous_gemm(runner_input.hidden_states, runner_input.hidden_states_scale, runner_input.m_indices,
                                   quant_info)
