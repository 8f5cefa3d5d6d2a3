"""The ops as the torch dispatcher sees them (sglang_amd/custom_ops.py).

Without a GPU: every op of the namespace has a schema and a fake implementation, and shapes, dtypes and strides
propagate through the layer-level functions on fake CUDA tensors (what torch.compile does while tracing), so a compiled
graph does not break at the ctypes calls.  The reference registers such fakes for its sgl_kernel ops
(python/sglang/srt/layers/quantization/fp8_kernel.py:48-50,1840-1859, fp8_utils.py:58-63).
On a GPU: the linear layer and the fused MoE layer traced by torch.compile (aot_eager backend: tracing and functionalisation,
no code generation) give the eager result bit for bit.
"""
import numpy as np
import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

OPS = ["sgl_per_token_group_quant_8bit", "sgl_per_token_quant_fp8", "sgl_per_tensor_quant_fp8", "fp8_blockwise_scaled_mm",
       "fp8_scaled_mm", "block_gemm_nk", "block_gemm_nk_ue8m0", "tensor_quant_mla", "bmm_fp8", "prepare_moe_input", "shuffle_rows", "apply_shuffle_mul_sum", "fp8_blockwise_scaled_grouped_mm", "moe_block_gemm_silu_quant", "moe_align_block_size", "silu_and_mul", "moe_sum_reduce",
       "moe_sort_scales", "moe_block_gemm", "moe_fused_gate"]


def test_every_op_is_registered_with_mutation_annotations():
    import sglang_amd.custom_ops  # noqa: F401

    for name in OPS:
        op = getattr(torch.ops.fp8k, name).default
        schema = str(op._schema)
        assert schema.startswith("fp8k::" + name)
    # caller-owned outputs are declared as mutated, so functionalisation keeps the launches in order
    for name in ("sgl_per_token_group_quant_8bit", "sgl_per_token_quant_fp8", "sgl_per_tensor_quant_fp8", "silu_and_mul",
                 "moe_sum_reduce", "moe_block_gemm", "moe_align_block_size"):
        assert "(a!)" in str(getattr(torch.ops.fp8k, name).default._schema)


def test_fake_propagation_through_the_layer_functions():
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.fp8_utils import apply_fp8_linear, w8a8_block_fp8_linear
    from sglang_amd.fused_moe import biased_grouped_topk, fused_experts_impl

    with FakeTensorMode():
        dev = "cuda"
        x = torch.empty((3, 5, 1024), dtype=torch.bfloat16, device=dev)
        w = torch.empty((768, 1024), dtype=torch.float8_e4m3fn, device=dev)
        ws = torch.empty((6, 8), dtype=torch.float32, device=dev)
        y = w8a8_block_fp8_linear(x, w, [128, 128], ws, None, torch.empty((768,), dtype=torch.bfloat16, device=dev))
        assert y.shape == (3, 5, 768) and y.dtype == torch.bfloat16 and y.device.type == "cuda"
        q, s = sglang_per_token_group_quant_fp8(x.view(15, 1024), 128, column_major_scales=True, scale_tma_aligned=True,
                                                scale_ue8m0=True)
        assert q.shape == (15, 1024) and q.dtype == torch.float8_e4m3fn
        assert s.shape == (15, 2) and s.dtype == torch.int32 and s.stride() == (1, 16)
        y2 = apply_fp8_linear(x, w.t(), torch.empty((1,), device=dev), bias=torch.empty((768,), device=dev))
        assert y2.shape == (3, 5, 768) and y2.dtype == torch.bfloat16
        # fused MoE layer: 40 tokens, 8 experts, hidden 512, intermediate 256, top-2
        h = torch.empty((40, 512), dtype=torch.bfloat16, device=dev)
        w1 = torch.empty((8, 512, 512), dtype=torch.float8_e4m3fn, device=dev)
        w2 = torch.empty((8, 512, 256), dtype=torch.float8_e4m3fn, device=dev)
        tw, ids = biased_grouped_topk(h, torch.empty((40, 8), device=dev), torch.empty((8,), device=dev), 2, True, 4, 2)
        assert tw.shape == ids.shape == (40, 2) and ids.dtype == torch.int32
        out = fused_experts_impl(h, w1, w2, tw, ids, use_fp8_w8a8=True, block_shape=[128, 128],
                                 w1_scale=torch.empty((8, 4, 4), device=dev), w2_scale=torch.empty((8, 4, 2), device=dev))
        assert out.shape == (40, 512) and out.dtype == torch.bfloat16


@pytest.mark.gpu
def test_compiled_layers_match_eager(dev):
    from oracle import fp8_oracle as O
    from sglang_amd.fp8_utils import w8a8_block_fp8_linear
    from sglang_amd.fused_moe import fused_experts_impl
    from tests.conftest import bf16_tensor, fp8_tensor

    rng = np.random.default_rng(3)
    T, E, H, I, topk = 64, 8, 512, 256, 2
    x = bf16_tensor(O.make_activation(T, H, 3), dev)
    wq, ws = O.block_quant_weight(O.make_weight(384, H, 3))
    W, Ws = fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)
    bias = bf16_tensor(O.to_bf16(rng.standard_normal(384).astype(np.float32)), dev)

    def codes(shape):
        return fp8_tensor(rng.integers(0, 0x60, shape, dtype=np.uint8) | (rng.integers(0, 2, shape, dtype=np.uint8) << 7), dev)

    w1, w2 = codes((E, 2 * I, H)), codes((E, H, I))
    w1s = torch.from_numpy((rng.uniform(0.5, 2, (E, 2 * I // 128, H // 128)) * 1e-3).astype(np.float32)).to(dev)
    w2s = torch.from_numpy((rng.uniform(0.5, 2, (E, H // 128, I // 128)) * 1e-3).astype(np.float32)).to(dev)
    ids = torch.from_numpy(np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)).to(dev)
    tw = torch.from_numpy(rng.uniform(0.1, 1, (T, topk)).astype(np.float32)).to(dev)

    def layer(x):
        h = fused_experts_impl(x, w1, w2, tw, ids, use_fp8_w8a8=True, w1_scale=w1s, w2_scale=w2s, block_shape=[128, 128],
                               routed_scaling_factor=2.5)
        return w8a8_block_fp8_linear(h, W, [128, 128], Ws, None, bias)

    eager = layer(x)
    compiled = torch.compile(layer, backend="aot_eager", fullgraph=True)
    got = compiled(x)
    torch.cuda.synchronize()
    assert torch.equal(got, eager)
    assert torch.equal(compiled(x), eager)
