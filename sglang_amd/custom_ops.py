"""The ops of ``sglang_amd.sgl_kernel`` registered with the torch dispatcher under the namespace ``fp8k``.

The reference reaches its native ops as ``torch.ops.sgl_kernel.*`` (schemas: sgl-kernel/csrc/common_extension.cc:78-79,
128-152,218-244) and registers fake implementations for the ones that ``torch.compile`` meets on this path
(python/sglang/srt/layers/quantization/fp8_kernel.py:48-50,1840-1859, fp8_utils.py:58-63).  Here every op gets a
schema with its mutated arguments marked, a CUDA implementation (the ctypes wrapper in sgl_kernel.py) and a fake
implementation that only produces shapes, so a graph capture by ``torch.compile`` / FakeTensor tracing sees one opaque
node per kernel launch instead of breaking at the ctypes call.

The functions exported here have the signatures of their namesakes in sgl_kernel.py and go through the dispatcher;
the layer-level modules (fp8_kernel.py, fp8_utils.py, fused_moe.py) call these.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import sgl_kernel as _k

_lib = torch.library.Library("fp8k", "FRAGMENT")


def _register(schema: str, impl, fake) -> None:
    name = schema.split("(", 1)[0]
    _lib.define(schema)
    _lib.impl(name, impl, "CUDA")
    torch.library.register_fake("fp8k::" + name, fake, lib=_lib)


def _none(*args, **kwargs) -> None:
    return None


# ---- quantisation (outputs are caller-allocated and mutated in place)
_register(
    "sgl_per_token_group_quant_8bit(Tensor input, Tensor(a!) output_q, Tensor(b!) output_s, int group_size, float eps, "
    "float fp8_min, float fp8_max, bool scale_ue8m0=False, bool fuse_silu_and_mul=False, Tensor? masked_m=None) -> ()",
    lambda input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0=False, fuse_silu_and_mul=False,
    masked_m=None: _k.sgl_per_token_group_quant_8bit(input, output_q, output_s, group_size, eps, fp8_min, fp8_max,
                                                      scale_ue8m0, fuse_silu_and_mul, masked_m),
    _none,
)
_register("sgl_per_token_quant_fp8(Tensor input, Tensor(a!) output_q, Tensor(b!) output_s) -> ()",
          _k.sgl_per_token_quant_fp8, _none)
_register("sgl_per_tensor_quant_fp8(Tensor input, Tensor(a!) output_q, Tensor(b!) output_s, bool is_static) -> ()",
          _k.sgl_per_tensor_quant_fp8, _none)


# ---- GEMMs (return a fresh tensor)
def _mm_fake(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    return mat_a.new_empty((mat_a.shape[0], mat_b.shape[1]), dtype=out_dtype)


def _nk_fake(A, B, As, Bs, out_dtype):
    return A.new_empty((A.shape[0], B.shape[0]), dtype=out_dtype)


_register("fp8_blockwise_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype) -> Tensor",
          _k.fp8_blockwise_scaled_mm, _mm_fake)
_register("fp8_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, "
          "Tensor? bias=None) -> Tensor", _k.fp8_scaled_mm, _mm_fake)
_register("block_gemm_nk(Tensor A, Tensor B, Tensor As, Tensor Bs, ScalarType out_dtype) -> Tensor", _k._block_gemm_nk, _nk_fake)
_register("block_gemm_nk_ue8m0(Tensor A, Tensor B, Tensor As_packed, Tensor Bs, ScalarType out_dtype) -> Tensor",
          _k._block_gemm_nk_ue8m0, _nk_fake)

_register("tensor_quant_mla(Tensor x, Tensor(a!) x_q, Tensor(b!) x_s, float eps) -> ()", _k.tensor_quant_mla, _none)


def _bmm_impl(A, B, A_scale, B_scale, dtype, out) -> None:
    _k.bmm_fp8(A, B, A_scale, B_scale, dtype, out)


_register("bmm_fp8(Tensor A, Tensor B, Tensor A_scale, Tensor B_scale, ScalarType dtype, Tensor(a!) out) -> ()", _bmm_impl, _none)

# ---- expert-major MoE layout (the CUTLASS-shaped path)
_register(
    "prepare_moe_input(Tensor topk_ids, Tensor(a!) expert_offsets, Tensor(b!)? blockscale_offsets, Tensor(c!) problem_sizes1, "
    "Tensor(d!) problem_sizes2, Tensor(e!) input_permutation, Tensor(f!) output_permutation, int num_experts, int n, int k) -> ()",
    lambda topk_ids, expert_offsets, blockscale_offsets, problem_sizes1, problem_sizes2, input_permutation, output_permutation,
    num_experts, n, k: _k.prepare_moe_input(topk_ids, expert_offsets, problem_sizes1, problem_sizes2, input_permutation,
                                            output_permutation, num_experts, n, k, blockscale_offsets),
    _none,
)
_register("shuffle_rows(Tensor input, Tensor dst2src_map, Tensor(a!) output) -> ()", _k.shuffle_rows_out, _none)
_register("apply_shuffle_mul_sum(Tensor input, Tensor(a!) output, Tensor? permutation, Tensor? factors) -> ()",
          _k.apply_shuffle_mul_sum, _none)
_register(
    "fp8_blockwise_scaled_grouped_mm(Tensor(a!) output, Tensor a_ptrs, Tensor b_ptrs, Tensor out_ptrs, Tensor a_scales_ptrs, "
    "Tensor b_scales_ptrs, Tensor a, Tensor b, Tensor scales_a, Tensor scales_b, Tensor stride_a, Tensor stride_b, "
    "Tensor stride_c, Tensor layout_sfa, Tensor layout_sfb, Tensor problem_sizes, Tensor expert_offsets, Tensor workspace) -> ()",
    _k.fp8_blockwise_scaled_grouped_mm, _none,
)



def _slot_blocks_fake(topk_ids, expert_offsets, problem_sizes, output_permutation, block_m):
    slots, E = topk_ids.numel(), problem_sizes.shape[0]
    cap = max((slots + min(slots, E) * (block_m - 1)) // block_m * block_m, block_m)
    i32 = lambda n: topk_ids.new_empty((n,), dtype=torch.int32)  # noqa: E731
    return i32(cap), i32(cap // block_m), i32(1)


_register("moe_slot_blocks(Tensor topk_ids, Tensor expert_offsets, Tensor problem_sizes, Tensor output_permutation, "
          "int block_m) -> (Tensor, Tensor, Tensor)", _k.moe_slot_blocks, _slot_blocks_fake)

# ---- fused-MoE stages
_register(
    "moe_align_block_size(Tensor topk_ids, int num_experts, int block_size, Tensor(a!) sorted_token_ids, "
    "Tensor(b!) experts_ids, Tensor(c!) num_tokens_post_pad, Tensor(d!)? cumsum_buffer, bool pad_sorted_token_ids=False) -> ()",
    _k.moe_align_block_size, _none,
)
def _silu_and_mul_impl(input, out) -> None:
    _k.silu_and_mul(input, out)


_register("silu_and_mul(Tensor input, Tensor(a!) out) -> ()", _silu_and_mul_impl, _none)


def _gelu_and_mul_impl(input, out) -> None:
    _k.gelu_and_mul(input, out)


_register("gelu_and_mul(Tensor input, Tensor(a!) out) -> ()", _gelu_and_mul_impl, _none)


def _activation_impl(input, out, kind) -> None:
    _k.activation(input, kind, out)


_register("activation(Tensor input, Tensor(a!) out, str kind) -> ()", _activation_impl, _none)
_register("moe_sum_reduce(Tensor input, Tensor(a!) output, float routed_scaling_factor) -> ()", _k.moe_sum_reduce, _none)


def _sort_scales_fake(A_scale, sorted_token_ids, num_tokens_post_padded, top_k, num_valid_tokens):
    return A_scale.new_empty((A_scale.shape[1], sorted_token_ids.numel())).t()


_register("moe_sort_scales(Tensor A_scale, Tensor sorted_token_ids, Tensor num_tokens_post_padded, int top_k, "
          "int num_valid_tokens) -> Tensor", _k.moe_sort_scales, _sort_scales_fake)
_register("moe_balance_blocks(Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, int block_m, "
          "int num_valid_tokens, int num_experts) -> Tensor", _k.moe_balance_blocks,
          lambda sorted_token_ids, expert_ids, num_tokens_post_padded, block_m, num_valid_tokens, num_experts:
          torch.empty_like(sorted_token_ids))
_register(
    "moe_block_gemm(Tensor A, Tensor B, Tensor(a!) C, Tensor A_scale, Tensor B_scale, Tensor? topk_weights, "
    "Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, bool mul_routed_weight, int top_k, "
    "int block_m, int num_valid_tokens, bool scales_sorted=False, bool pow2_scales=False, bool balanced=False) -> ()",
    _k.moe_block_gemm, _none,
)


_register(
    "moe_block_gemm_silu_quant(Tensor A, Tensor B, Tensor A_scale_sorted, Tensor B_scale, Tensor(a!) out_q, Tensor(b!) out_s, "
    "Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, int top_k, int num_valid_tokens, "
    "ScalarType act_dtype, float eps=1e-10, bool balanced=False) -> ()",
    _k.moe_block_gemm_silu_quant, _none,
)


def _gate_fake(input, bias, num_expert_group, topk_group, topk, num_fused_shared_experts=0, routed_scaling_factor=0.0,
               apply_routed_scaling_factor_on_output=False):
    rows = input.shape[0]
    return input.new_empty((rows, topk), dtype=torch.float32), input.new_empty((rows, topk), dtype=torch.int32)


_register(
    "moe_fused_gate(Tensor input, Tensor bias, int num_expert_group, int topk_group, int topk, "
    "int num_fused_shared_experts=0, float routed_scaling_factor=0.0, bool apply_routed_scaling_factor_on_output=False) "
    "-> (Tensor, Tensor)", _k.moe_fused_gate, _gate_fake,
)

_ops = torch.ops.fp8k

# ---------------------------------------------------------------------------------------------------------------
# the same names as sgl_kernel.py, through the dispatcher
# ---------------------------------------------------------------------------------------------------------------


def sgl_per_token_group_quant_8bit(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0=False,
                                   fuse_silu_and_mul=False, masked_m=None, enable_v2=None) -> None:
    _ops.sgl_per_token_group_quant_8bit(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0,
                                        fuse_silu_and_mul, masked_m)


sgl_per_token_group_quant_fp8 = sgl_per_token_group_quant_8bit


def sgl_per_token_quant_fp8(input, output_q, output_s) -> None:
    _ops.sgl_per_token_quant_fp8(input, output_q, output_s)


def sgl_per_tensor_quant_fp8(input, output_q, output_s, is_static: bool) -> None:
    _ops.sgl_per_tensor_quant_fp8(input, output_q, output_s, is_static)


def fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype) -> torch.Tensor:
    return _ops.fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype)


def fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None) -> torch.Tensor:
    return _ops.fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


def block_gemm_nk(A, B, As, Bs, out_dtype) -> torch.Tensor:
    return _ops.block_gemm_nk(A, B, As, Bs, out_dtype)


def block_gemm_nk_ue8m0(A, B, As_packed, Bs, out_dtype) -> torch.Tensor:
    return _ops.block_gemm_nk_ue8m0(A, B, As_packed, Bs, out_dtype)


def tensor_quant_mla(x, x_q, x_s, eps: float) -> None:
    _ops.tensor_quant_mla(x, x_q, x_s, float(eps))


def bmm_fp8(A, B, A_scale, B_scale, dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if out is None:
        out = torch.empty((A.shape[0], A.shape[1], B.shape[2]), device=A.device, dtype=dtype)
    _ops.bmm_fp8(A, B, A_scale, B_scale, dtype, out)
    return out


def prepare_moe_input(topk_ids, expert_offsets, problem_sizes1, problem_sizes2, input_permutation, output_permutation,
                      num_experts, n, k, blockscale_offsets: Optional[torch.Tensor] = None) -> None:
    _ops.prepare_moe_input(topk_ids, expert_offsets, blockscale_offsets, problem_sizes1, problem_sizes2, input_permutation,
                           output_permutation, num_experts, n, k)


def shuffle_rows(input_tensor, dst2src_map, output_tensor_shape) -> torch.Tensor:
    output_tensor = torch.empty(output_tensor_shape, device=input_tensor.device, dtype=input_tensor.dtype)
    _ops.shuffle_rows(input_tensor, dst2src_map, output_tensor)
    return output_tensor


def apply_shuffle_mul_sum(input, output, permutation, factors) -> None:
    _ops.apply_shuffle_mul_sum(input, output, permutation, factors)


def moe_slot_blocks(topk_ids, expert_offsets, problem_sizes, output_permutation, block_m: int):
    return _ops.moe_slot_blocks(topk_ids, expert_offsets, problem_sizes, output_permutation, block_m)


def fp8_blockwise_scaled_grouped_mm(output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a, scales_b,
                                    stride_a, stride_b, stride_c, layout_sfa, layout_sfb, problem_sizes, expert_offsets,
                                    workspace) -> None:
    _ops.fp8_blockwise_scaled_grouped_mm(output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a,
                                         scales_b, stride_a, stride_b, stride_c, layout_sfa, layout_sfb, problem_sizes,
                                         expert_offsets, workspace)


def moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad,
                         cumsum_buffer, pad_sorted_token_ids=False) -> None:
    _ops.moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad,
                              cumsum_buffer, pad_sorted_token_ids)


def silu_and_mul(input: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if out is None:
        out = torch.empty(input.shape[:-1] + (input.shape[-1] // 2,), device=input.device, dtype=input.dtype)
    _ops.silu_and_mul(input, out)
    return out


def gelu_and_mul(input: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if out is None:
        out = torch.empty(input.shape[:-1] + (input.shape[-1] // 2,), device=input.device, dtype=input.dtype)
    _ops.gelu_and_mul(input, out)
    return out


def activation(input: torch.Tensor, kind: str, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if out is None:
        out = torch.empty_like(input)
    _ops.activation(input, out, kind)
    return out


def moe_sum_reduce(input_tensor, output_tensor, routed_scaling_factor: float = 0) -> None:
    _ops.moe_sum_reduce(input_tensor, output_tensor, float(routed_scaling_factor))


def moe_sort_scales(A_scale, sorted_token_ids, num_tokens_post_padded, top_k: int, num_valid_tokens: int) -> torch.Tensor:
    return _ops.moe_sort_scales(A_scale, sorted_token_ids, num_tokens_post_padded, top_k, num_valid_tokens)


def moe_balance_blocks(sorted_token_ids, expert_ids, num_tokens_post_padded, block_m: int, num_valid_tokens: int,
                       num_experts: int) -> torch.Tensor:
    return _ops.moe_balance_blocks(sorted_token_ids, expert_ids, num_tokens_post_padded, block_m, num_valid_tokens, num_experts)


def moe_block_gemm(A, B, C, A_scale, B_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded,
                   mul_routed_weight: bool, top_k: int, block_m: int, num_valid_tokens: int, scales_sorted: bool = False,
                   pow2_scales: bool = False, balanced: bool = False) -> None:
    _ops.moe_block_gemm(A, B, C, A_scale, B_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded,
                        mul_routed_weight, top_k, block_m, num_valid_tokens, scales_sorted, pow2_scales, balanced)


def moe_block_gemm_silu_quant(A, B, A_scale_sorted, B_scale, out_q, out_s, sorted_token_ids, expert_ids,
                              num_tokens_post_padded, top_k: int, num_valid_tokens: int, act_dtype, eps: float = 1e-10,
                              balanced: bool = False) -> None:
    _ops.moe_block_gemm_silu_quant(A, B, A_scale_sorted, B_scale, out_q, out_s, sorted_token_ids, expert_ids,
                                   num_tokens_post_padded, top_k, num_valid_tokens, act_dtype, float(eps), balanced)


def moe_fused_gate(input_tensor, bias, num_expert_group, topk_group, topk, num_fused_shared_experts=0,
                   routed_scaling_factor=0.0, apply_routed_scaling_factor_on_output=False) -> Tuple[torch.Tensor, torch.Tensor]:
    return _ops.moe_fused_gate(input_tensor, bias, num_expert_group, topk_group, topk, num_fused_shared_experts,
                               float(routed_scaling_factor), apply_routed_scaling_factor_on_output)
