"""Block-FP8 fused-experts pipeline behind the reference's Python interface.

Mirrors ``sglang.srt.layers.moe.fused_moe_triton`` for the one configuration this path builds:
``use_fp8_w8a8=True`` with ``block_shape=[128, 128]`` (DeepSeek-V3 style experts).  Sequence, as in
fused_moe.py:498-639 of the reference:

    moe_align_block_size -> quant + grouped GEMM (w13) -> silu_and_mul -> quant + grouped GEMM (w2,
    times the routed weight) -> sum over top-k (times routed_scaling_factor)

silu_and_mul and the second quant are one kernel; with 256-slot blocks they run inside the write-out of the first GEMM.
activation="gelu" runs gelu_and_mul and the quant as two kernels at every block size; experts without a gate projection
(is_gated=False: silu, gelu, relu2) run the activation kernel and the quant.

Every stage is a call into libfp8k.so; intermediates are torch tensors on the current stream.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from . import custom_ops as _ops
from .fp8_kernel import sglang_per_token_group_quant_fp8

CHUNK_SIZE = 64 * 1024  # tokens per pass, as in the reference (fused_moe.py:423)


def moe_align_block_size(
    topk_ids: torch.Tensor, block_size: int, num_experts: int
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Reference: python/sglang/srt/layers/moe/fused_moe_triton/moe_align_block_size.py:17-82.

    Returns (sorted_token_ids [numel + (E+1)(B-1)], expert_ids [ceil(that/B)], num_tokens_post_padded [1]).
    Padding slots hold topk_ids.numel(); expert -1 (not on this rank) gets its own leading blocks.
    """
    max_num_tokens_padded = topk_ids.numel() + (num_experts + 1) * (block_size - 1)
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=topk_ids.device)
    max_num_m_blocks = (max_num_tokens_padded + block_size - 1) // block_size
    expert_ids = torch.empty((max_num_m_blocks,), dtype=torch.int32, device=topk_ids.device)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=topk_ids.device)
    cumsum_buffer = torch.empty((num_experts + 2,), dtype=torch.int32, device=topk_ids.device)
    _ops.moe_align_block_size(
        topk_ids, num_experts + 1, block_size, sorted_ids, expert_ids, num_tokens_post_pad, cumsum_buffer, True
    )
    return sorted_ids, expert_ids, num_tokens_post_pad


def get_default_config(M: int, E: int, topk: int) -> Dict[str, int]:
    """Rows per block of the grouped GEMM (the reference's BLOCK_SIZE_M, fused_moe_triton_config.py).

    Measured on MI355X with 256 experts, top-8 and near-balanced routing: while the layer streams every expert's
    weights for a handful of rows each, the register-streaming kernel with 16- or 32-row blocks wins (up to about 22
    rows per expert: 1.95 ms against 2.02 ms at 512 tokens); from there on the 256-row kernel, which walks its items
    with the weight stream running on across them, skips the slot groups that are padding and forms the activation and
    the requantisation in the write-out of GEMM 1 (2.06 ms against 2.13 ms with 64-row blocks at 768 tokens, 2.21
    against 2.29 with 128-row blocks at 1536, 2.48 against 2.65 at 3072).  The 64- and 128-row forms of the streaming
    kernel remain for callers that pass their own BLOCK_SIZE_M.
    """
    per_expert = (M * topk + E - 1) // max(E, 1)
    if per_expert <= 4:
        bm = 16
    elif per_expert <= 22:
        bm = 32
    else:
        bm = 256
    return {"BLOCK_SIZE_M": bm, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 128}


def blocks_want_balancing(config: Dict[str, int], slots: int, num_experts: int) -> bool:
    """Whether the layer deals every expert's slots out evenly over its blocks (moe_balance_blocks) before the grouped
    GEMMs: with 256-slot blocks and, on average, more than 192 slots per expert most experts have two and more blocks,
    whose workgroups share the expert's weight tiles in L2 only while the blocks take the same time."""
    return int(config["BLOCK_SIZE_M"]) == 256 and slots > 192 * num_experts


# block sizes from which the activation scales are first gathered into the order of sorted_token_ids
SORT_SCALES_MIN_BLOCK = 64

def gemm1_fuses_activation(config: Dict[str, Any], n_gate_up: int) -> bool:
    """Whether grouped GEMM 1 applies silu_and_mul and the requantisation in its own write-out (same bytes and scales as
    GEMM -> fused silu + quant, the [slots, 2 I] intermediate is never written): built for 256-slot blocks and an
    intermediate size that is a multiple of 128.  Measured on MI355X (E = 256, H = 7168, I = 2048): 3 % faster than the
    three-step sequence at 4096 tokens, 1 % at 8192, even at 16384; smaller blocks keep the three steps."""
    return int(config["BLOCK_SIZE_M"]) == 256 and n_gate_up % 256 == 0


def invoke_fused_moe_kernel(
    A: torch.Tensor,
    B: torch.Tensor,
    bias: Optional[torch.Tensor],
    C: torch.Tensor,
    A_scale: Optional[torch.Tensor],
    B_scale: Optional[torch.Tensor],
    B_zp: Optional[torch.Tensor],
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    sorted_token_ids: torch.Tensor,
    expert_ids: torch.Tensor,
    num_tokens_post_padded: torch.Tensor,
    mul_routed_weight: bool,
    top_k: int,
    config: Dict[str, Any],
    compute_type=None,
    use_fp8_w8a8: bool = True,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    per_channel_quant: bool = False,
    block_shape: Optional[List[int]] = None,
    no_combine: bool = False,
    a_use_tma: bool = False,
    b_use_tma: bool = False,
    c_sorted: bool = False,
    filter_expert: bool = True,
) -> None:
    """Reference: fused_moe_triton_kernels.py:586-790.  A is bf16/fp16 and is group-quantised here
    (as the reference does, :627-637) unless it already is e4m3fn with A_scale given."""
    assert topk_weights.stride(1) == 1
    assert sorted_token_ids.stride(0) == 1
    if not use_fp8_w8a8 or use_int8_w8a8 or use_int8_w8a16 or use_int4_w4a16 or per_channel_quant:
        raise RuntimeError("invoke_fused_moe_kernel: only use_fp8_w8a8 with block_shape [128, 128] is built on this path")
    if block_shape is None or list(block_shape) != [128, 128]:
        raise RuntimeError("invoke_fused_moe_kernel: block_shape must be [128, 128]")
    if bias is not None or B_zp is not None or c_sorted or a_use_tma or b_use_tma:
        raise RuntimeError("invoke_fused_moe_kernel: bias, zero points and the TMA layouts are not built on this path")
    assert B_scale is not None
    if A.dtype != torch.float8_e4m3fn:
        assert A_scale is None
        # blocks of 64 slots and more: row-major scales, which moe_sort_scales reads a row at a time
        A, A_scale = sglang_per_token_group_quant_fp8(A, block_shape[1], column_major_scales=config["BLOCK_SIZE_M"] < 64)
    assert (A.shape[-1] + 127) // 128 == A_scale.shape[-1]
    assert (B.shape[-2] + 127) // 128 == B_scale.shape[-2]
    assert (B.shape[-1] + 127) // 128 == B_scale.shape[-1]
    block_m = int(config["BLOCK_SIZE_M"])
    sort_scales = block_m >= SORT_SCALES_MIN_BLOCK
    if sort_scales:
        # the rows of a block are gathered: with the scales in the order of sorted_token_ids the lanes of a wave read
        # theirs from one cache line instead of one line per token row
        A_scale = _ops.moe_sort_scales(A_scale, sorted_token_ids, num_tokens_post_padded, top_k, topk_ids.numel())
    _ops.moe_block_gemm(
        A, B, C, A_scale, B_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded,
        mul_routed_weight, top_k, block_m, topk_ids.numel(), scales_sorted=sort_scales,
    )


def fused_experts_impl(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    b1: Optional[torch.Tensor] = None,
    b2: Optional[torch.Tensor] = None,
    inplace: bool = False,
    activation: str = "silu",
    is_gated: bool = True,
    apply_router_weight_on_input: bool = False,
    use_fp8_w8a8: bool = False,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    per_channel_quant: bool = False,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    w1_zp: Optional[torch.Tensor] = None,
    w2_zp: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
    no_combine: bool = False,
    routed_scaling_factor: Optional[float] = None,
    gemm1_alpha: Optional[float] = None,
    gemm1_limit: Optional[float] = None,
    filter_expert: bool = True,
) -> torch.Tensor:
    """Reference: fused_moe.py:369-660.  hidden_states [T,H] bf16/fp16; w1 e4m3fn [E,2I,H]; w2 e4m3fn
    [E,H,I]; w1_scale/w2_scale float32 per 128x128 block; topk_weights float32 [T,k]; topk_ids int [T,k]
    (-1 = expert on another rank, contributes zero)."""
    if not use_fp8_w8a8 or block_shape is None:
        raise RuntimeError("fused_experts_impl: only use_fp8_w8a8=True with block_shape=[128, 128] is built on this path")
    if not ((is_gated and activation in ("silu", "gelu")) or (not is_gated and activation in ("silu", "gelu", "relu2"))):
        raise ValueError(f"Unsupported activation: {activation=}, with {is_gated=}")
    if activation == "gelu":
        assert gemm1_alpha is None, "gemm1_alpha is not supported for gelu"
        assert gemm1_limit is None, "gemm1_limit is not supported for gelu"
    if gemm1_alpha is not None or gemm1_limit is not None:
        raise RuntimeError("fused_experts_impl: swiglu with alpha and limit is not built on this path")
    if b1 is not None or b2 is not None:
        raise RuntimeError("fused_experts_impl: biases are not built on this path")
    # a1_scale / a2_scale: with a block_shape the reference quantises the activations per token group whatever scale
    # it is handed (fused_moe_triton_kernels.py:619-637 overwrites A_scale), so they have no effect here either
    assert hidden_states.shape[1] == w1.shape[2], "Hidden size mismatch"
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype in [torch.float16, torch.bfloat16]

    num_tokens, _ = hidden_states.shape
    E, N, _ = w1.shape
    topk = topk_ids.shape[1]
    M = min(num_tokens, CHUNK_SIZE)
    dev, dt = hidden_states.device, hidden_states.dtype
    if topk_weights.dtype != torch.float32:
        topk_weights = topk_weights.float()
    topk_weights = topk_weights.contiguous()
    topk_ids = topk_ids.contiguous()

    cache1 = torch.empty((M * topk, N), device=dev, dtype=dt)
    cache3 = torch.empty((M, topk, w2.shape[1]), device=dev, dtype=dt)
    if no_combine:
        assert not inplace
        out_hidden_states = torch.empty((num_tokens, topk, w2.shape[1]), device=dev, dtype=dt)
    elif inplace:
        out_hidden_states = hidden_states
    else:
        out_hidden_states = torch.empty_like(hidden_states)
    if routed_scaling_factor is None:
        routed_scaling_factor = 1.0

    for chunk in range((num_tokens // CHUNK_SIZE) + 1):
        begin, end = chunk * CHUNK_SIZE, min((chunk + 1) * CHUNK_SIZE, num_tokens)
        curr = hidden_states[begin:end]
        tokens = curr.shape[0]
        if tokens == 0:
            break
        config = get_default_config(tokens, E, topk)
        curr_ids = topk_ids[begin:end]
        curr_w = topk_weights[begin:end]
        ic1 = cache1[: tokens * topk]
        ic3 = out_hidden_states[begin:end] if no_combine else cache3[:tokens]

        sorted_token_ids, expert_ids, num_tokens_post_padded = moe_align_block_size(curr_ids, config["BLOCK_SIZE_M"], E)
        balanced = blocks_want_balancing(config, tokens * topk, E)
        if balanced:
            sorted_token_ids = _ops.moe_balance_blocks(sorted_token_ids, expert_ids, num_tokens_post_padded,
                                                       config["BLOCK_SIZE_M"], tokens * topk, E)
        # apply_router_weight_on_input (fused_moe.py:533,597 of the reference): the routed weight multiplies the result of
        # GEMM 1 instead of GEMM 2; the fused write-out has no such factor, so that form keeps the three steps
        if gemm1_fuses_activation(config, N) and not apply_router_weight_on_input and activation == "silu" and is_gated:
            slots = tokens * topk
            a1_q, a1_s = sglang_per_token_group_quant_fp8(curr, block_shape[1])
            a1_s = _ops.moe_sort_scales(a1_s, sorted_token_ids, num_tokens_post_padded, topk, slots)
            a2_q = torch.empty((slots, N // 2), device=dev, dtype=torch.float8_e4m3fn)
            a2_s = torch.empty((N // 256, sorted_token_ids.numel()), device=dev, dtype=torch.float32).t()
            _ops.moe_block_gemm_silu_quant(a1_q, w1, a1_s, w1_scale, a2_q, a2_s, sorted_token_ids, expert_ids,
                                           num_tokens_post_padded, topk, slots, dt, balanced=balanced)
            _ops.moe_block_gemm(a2_q, w2, ic3, a2_s, w2_scale, curr_w, sorted_token_ids, expert_ids, num_tokens_post_padded,
                                True, 1, 256, slots, scales_sorted=True, balanced=balanced)
            if not no_combine:
                _ops.moe_sum_reduce(ic3, out_hidden_states[begin:end], routed_scaling_factor)
            continue
        invoke_fused_moe_kernel(
            curr, w1, None, ic1, None, w1_scale, None, curr_w, curr_ids, sorted_token_ids, expert_ids,
            num_tokens_post_padded, apply_router_weight_on_input, topk, config, use_fp8_w8a8=True, block_shape=block_shape,
        )
        if not is_gated:
            # fused_moe.py:566-572 of the reference: w1 is [E, N, H] without a gate half, the activation keeps the width
            ic2 = _ops.activation(ic1, activation)
            a2_q, a2_s = sglang_per_token_group_quant_fp8(ic2, block_shape[1], column_major_scales=config["BLOCK_SIZE_M"] < 64)
        elif activation == "gelu":
            # fused_moe.py:561-565 of the reference: gelu_and_mul, then the group quant at the head of GEMM 2
            ic2 = torch.empty((tokens * topk, N // 2), device=dev, dtype=dt)
            _ops.gelu_and_mul(ic1, ic2)
            a2_q, a2_s = sglang_per_token_group_quant_fp8(ic2, block_shape[1], column_major_scales=config["BLOCK_SIZE_M"] < 64)
        else:
            # silu_and_mul fused into the requantisation (same bytes as silu_and_mul + group quant, one pass less
            # over the [tokens*topk, N] intermediate)
            a2_q, a2_s = sglang_per_token_group_quant_fp8(ic1, block_shape[1], column_major_scales=config["BLOCK_SIZE_M"] < 64,
                                                          fuse_silu_and_mul=True)
        invoke_fused_moe_kernel(
            a2_q, w2, None, ic3, a2_s, w2_scale, None, curr_w, curr_ids, sorted_token_ids, expert_ids,
            num_tokens_post_padded, not apply_router_weight_on_input, 1, config, use_fp8_w8a8=True, block_shape=block_shape,
        )
        if not no_combine:
            _ops.moe_sum_reduce(ic3, out_hidden_states[begin:end], routed_scaling_factor)
    return out_hidden_states


def fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, **kwargs) -> torch.Tensor:
    """Out-of-place fused experts (the reference's outplace_fused_experts, fused_moe.py:180-245)."""
    kwargs.pop("inplace", None)
    return fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, inplace=False, **kwargs)


def biased_grouped_topk(
    hidden_states: torch.Tensor,
    gating_output: torch.Tensor,
    correction_bias: torch.Tensor,
    topk: int,
    renormalize: bool,
    num_expert_group: Optional[int] = None,
    topk_group: Optional[int] = None,
    num_fused_shared_experts: int = 0,
    routed_scaling_factor: Optional[float] = None,
    apply_routed_scaling_factor_on_output: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference: biased_grouped_topk_gpu, python/sglang/srt/layers/moe/topk.py:762-850, on the fused gate kernel.
    Its shape limits are the reference kernel's (power-of-two expert count, at most 32 experts per group, at most 64
    groups, renormalised weights); where the reference falls back to tensor ops for other shapes, this path has no
    second implementation and raises."""
    experts = gating_output.shape[1]
    fits = (
        renormalize and num_expert_group and topk_group and experts & (experts - 1) == 0
        and experts % num_expert_group == 0 and experts // num_expert_group <= 32 and num_expert_group <= 64
    )
    if not fits:
        raise RuntimeError(
            "biased_grouped_topk: built for renormalised weights, a power-of-two expert count, at most 32 experts per "
            "group and at most 64 groups (got %d experts, %s groups, renormalize=%s)" % (experts, num_expert_group, renormalize))
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    return _ops.moe_fused_gate(
        gating_output.contiguous(), correction_bias.to(gating_output.dtype).contiguous(), num_expert_group, topk_group,
        topk, num_fused_shared_experts, routed_scaling_factor if routed_scaling_factor is not None else 0.0,
        apply_routed_scaling_factor_on_output,
    )
