"""GPU tests of the layer-level entry points (what Fp8LinearMethod.apply and W8A8Fp8LinearMethod.apply call) and of
HIP-graph capture of the path.

apply_fp8_linear (reference: python/sglang/srt/layers/quantization/fp8_utils.py:639-736) against the oracle's
quantisers + fp8_scaled_mm; w8a8_block_fp8_linear (fp8_utils.py:306-326) with bias and N-D input against the oracle's
block_fp8_linear.  Quantised bytes and scales are exact by construction of the oracle's quantisers (checked in
tests/test_quant_gpu.py); the GEMM result within max relative error 1e-2.

Graph tests replay a captured graph several times with eager work of the library between the replays and compare
every replay with the eager result bit for bit.
"""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import bf16_tensor, fp8_tensor

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _rel_err(c, ref):
    return float(np.abs(c.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


def _weight_per_tensor(N, K, seed):
    w = O.make_weight(N, K, seed)
    wq, s = O.per_tensor_quant_fp8(w)
    return w, wq, s  # s: float32 [1]


def _weight_per_channel(N, K, seed):
    w = O.make_weight(N, K, seed)
    wq, s = O.per_token_quant_fp8(w)  # one scale per output channel (row of the [N, K] weight)
    return w, wq, s.reshape(-1)


@pytest.mark.parametrize("mode", ["static", "dynamic_tensor", "dynamic_token_channel_weight", "dynamic_token_forced"])
@pytest.mark.parametrize("bias_kind", [None, "bf16", "f32", "f16"])
@pytest.mark.parametrize("shape", [(70, 1024), (3, 5, 1024)])
def test_apply_fp8_linear(dev, mode, bias_kind, shape):
    from sglang_amd.fp8_utils import apply_fp8_linear

    N, K = 768, shape[-1]
    rows = int(np.prod(shape[:-1]))
    x = O.make_activation(rows, K, seed=rows)
    rng = np.random.default_rng(rows + N)
    if mode == "dynamic_token_channel_weight":
        _, wq, w_scale = _weight_per_channel(N, K, 3)
    else:
        _, wq, w_scale = _weight_per_tensor(N, K, 3)
    sb = np.broadcast_to(w_scale, (N,)).astype(np.float32)
    if mode == "static":
        in_scale = np.float32(np.abs(x).max() / 448.0 * 1.25)
        aq, sa = O.per_tensor_quant_fp8(x, static_scale=in_scale)
        sa = np.full((rows,), sa[0], np.float32)
    elif mode == "dynamic_tensor":
        aq, sa = O.per_tensor_quant_fp8(x)
        sa = np.full((rows,), sa[0], np.float32)
    else:
        aq, sa = O.per_token_quant_fp8(x)
        sa = sa.reshape(-1)
    bias = None
    if bias_kind is not None:
        b = rng.standard_normal(N).astype(np.float32)
        bias = O.to_bf16(b) if bias_kind == "bf16" else b.astype(np.float16).astype(np.float32) if bias_kind == "f16" else b
    # a bias that is neither the activation dtype nor float32 is cast to the activation dtype first
    bias_used = O.to_bf16(bias) if bias_kind == "f16" else bias
    ref = O.fp8_scaled_mm(aq, wq, sa, sb, "f32", bias_used)

    xt = bf16_tensor(x, dev).view(*shape)
    weight = fp8_tensor(wq, dev).t()  # the layer stores weight.t(): [K, N] column-major
    t_bias = None
    if bias is not None:
        t_bias = torch.from_numpy(bias).to(dev).to({"bf16": torch.bfloat16, "f32": torch.float32, "f16": torch.float16}[bias_kind])
    out = apply_fp8_linear(
        xt, weight, torch.from_numpy(np.ascontiguousarray(w_scale)).to(dev),
        input_scale=torch.tensor([in_scale], device=dev) if mode == "static" else None, bias=t_bias,
        use_per_token_if_dynamic=(mode == "dynamic_token_forced"),
    )
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == tuple(shape[:-1]) + (N,)
    got = out.float().cpu().numpy().reshape(rows, N)
    assert _rel_err(got, ref) <= REL_TOL, _rel_err(got, ref)


@pytest.mark.parametrize("shape", [(40, 1024), (2, 3, 7, 1024), (300, 1024)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_block_fp8_linear_bias_and_nd_input(dev, shape, with_bias):
    from sglang_amd.fp8_utils import dispatch_w8a8_block_fp8_linear

    N, K = 640, shape[-1]
    rows = int(np.prod(shape[:-1]))
    x = O.make_activation(rows, K, seed=rows).reshape(shape)
    wq, ws = O.block_quant_weight(O.make_weight(N, K, 5))
    bias = O.to_bf16(np.random.default_rng(N).standard_normal(N).astype(np.float32)) if with_bias else None
    ref = O.block_fp8_linear(x, wq, ws, bias)
    fn = dispatch_w8a8_block_fp8_linear()
    out = fn(bf16_tensor(x.reshape(rows, K), dev).view(*shape), fp8_tensor(wq, dev), [128, 128], torch.from_numpy(ws).to(dev),
             None, None if bias is None else bf16_tensor(bias, dev))
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == tuple(shape[:-1]) + (N,)
    assert _rel_err(out.float().cpu().numpy(), ref) <= REL_TOL
    if with_bias:
        # the bias is one more bf16 add on top of the un-biased result: exactly that, element by element
        plain = fn(bf16_tensor(x.reshape(rows, K), dev).view(*shape), fp8_tensor(wq, dev), [128, 128], torch.from_numpy(ws).to(dev))
        assert torch.equal(out, plain + bf16_tensor(bias, dev))


@pytest.mark.parametrize("shape", [(5, 1024), (2, 37, 1024)])
def test_block_fp8_linear_takes_a_prequantised_input(dev, shape):
    """Fp8LinearMethod.apply hands an upstream-quantised `(x_q, x_scale)` pair over as input / input_scale
    (fp8.py:500-508): the same bits as quantising here (bf16 out), and <= 1e-2 against the oracle."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.fp8_utils import dispatch_w8a8_block_fp8_linear

    N, K = 384, shape[-1]
    rows = int(np.prod(shape[:-1]))
    x = O.make_activation(rows, K, seed=rows)
    wq, ws = O.block_quant_weight(O.make_weight(N, K, 6))
    fn = dispatch_w8a8_block_fp8_linear()
    xt = bf16_tensor(x, dev)
    W, Ws = fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)
    x_q, x_s = sglang_per_token_group_quant_fp8(xt, 128)  # row-major scales: any strides are taken
    out = fn(x_q.view(*shape), W, [128, 128], Ws, x_s.view(*shape[:-1], K // 128))
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == tuple(shape[:-1]) + (N,)
    assert torch.equal(out.view(rows, N), fn(xt, W, [128, 128], Ws))
    assert _rel_err(out.float().cpu().numpy().reshape(rows, N), O.block_fp8_linear(x, wq, ws)) <= REL_TOL
    with pytest.raises(RuntimeError, match="float8_e4m3fn already"):
        fn(xt, W, [128, 128], Ws, x_s)


def test_graph_capture_split_k_gemm_survives_workspace_growth(dev):
    """A K-cut GEMM (M=16, N=7168, K=16384: float partials in the workspace) captured in a graph; afterwards a GEMM
    that needs a larger workspace runs eagerly on the stream the capture used, which makes the wrapper hand out a
    bigger buffer.  The graph still owns the one it recorded: its replays must keep giving the eager result."""
    from sglang_amd import sgl_kernel as ops
    from sglang_amd._lib import lib
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul

    M, N, K = 16, 7168, 16384
    assert lib.fp8k_block_gemm_workspace_bytes(M, N, K) > 0
    x = bf16_tensor(O.make_activation(M, K, 0), dev)
    rng = np.random.default_rng(0)
    wq = rng.integers(0, 0x68, (N, K), dtype=np.uint8) | (rng.integers(0, 2, (N, K), dtype=np.uint8) << 7)
    ws = (rng.uniform(0.5, 2.0, (N // 128, K // 128)) * 1e-3).astype(np.float32)
    B, Bs = fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)

    def linear():
        q, s = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
        return w8a8_block_fp8_matmul(q, B, s, Bs, [128, 128], torch.bfloat16)

    eager = linear()
    torch.cuda.synchronize()
    xq, xs = O.per_token_group_quant_fp8(x.float().cpu().numpy(), 128)
    ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="f32", acc=np.float64)
    assert _rel_err(eager.float().cpu().numpy(), ref) <= REL_TOL

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = linear()
        key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
        captured_ws = ops._workspaces[key]
        # grow the workspace of the capture stream after the GEMM was recorded: 128 rows need several times more
        big = lib.fp8k_block_gemm_workspace_bytes(128, N, K)
        ops.reserve_workspace(dev, max(big, 2 * captured_ws.numel()))
        assert ops._workspaces[key] is not captured_ws and any(b is captured_ws for b in ops._retired)
    for _ in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        # eager work between the replays: a larger GEMM whose partials land in the (new) workspace
        q2, s2 = sglang_per_token_group_quant_fp8(bf16_tensor(O.make_activation(128, K, 1), dev), 128, column_major_scales=True)
        w8a8_block_fp8_matmul(q2, B, s2, Bs, [128, 128], torch.bfloat16)
        torch.cuda.synchronize()


@pytest.mark.parametrize("T,E,topk", [(96, 16, 4), (900, 4, 4)])
def test_graph_capture_fused_moe_layer(dev, monkeypatch, T, E, topk):
    """quant + grouped GEMMs + fused silu/requant + top-k sum of fused_experts_impl, and the dense linear, in one graph;
    three replays with eager launches between them, each compared with the eager result.  The second case has 900 slots
    per expert: several 256-slot blocks each, dealt out evenly (moe_balance_blocks) and walked; its result is also held
    bit for bit against the layer on the aligner's own table."""
    import sglang_amd.fused_moe as fm
    from sglang_amd.fp8_utils import w8a8_block_fp8_linear
    from sglang_amd.fused_moe import blocks_want_balancing, fused_experts_impl, get_default_config

    rng = np.random.default_rng(7)
    H, I = 1024, 512
    assert blocks_want_balancing(get_default_config(T, E, topk), T * topk, E) == (T == 900)
    x = O.make_activation(T, H, 7)
    w13q = np.empty((E, 2 * I, H), np.uint8); w13s = np.empty((E, 2 * I // 128, H // 128), np.float32)
    w2q = np.empty((E, H, I), np.uint8); w2s = np.empty((E, H // 128, I // 128), np.float32)
    for e in range(E):
        w13q[e], w13s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((2 * I, H)).astype(np.float32) * 0.02))
        w2q[e], w2s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((H, I)).astype(np.float32) * 0.02))
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    tw = rng.uniform(0.1, 1.0, (T, topk)).astype(np.float32)
    wq, ws = O.block_quant_weight(O.make_weight(768, H, 9))
    xt = bf16_tensor(x, dev)
    args = (xt, fp8_tensor(w13q, dev), fp8_tensor(w2q, dev), torch.from_numpy(tw).to(dev), torch.from_numpy(ids).to(dev))
    kw = dict(use_fp8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
              block_shape=[128, 128], routed_scaling_factor=2.5)
    W, Ws = fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)

    def layer():
        h = fused_experts_impl(*args, **kw)
        return h, w8a8_block_fp8_linear(h, W, [128, 128], Ws)

    eager_h, eager_y = layer()
    torch.cuda.synchronize()
    ref = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, 2.5)
    # The 900-token input holds a row with an outlier (largest entry 280 times the row's median).  In the oracle itself a
    # 0.2 % change of that row's GEMM 1 result moves some thirty fp8 codes and a few scales of the second quantisation per
    # expert and the expert's output by up to 1.7 % of its largest value, so last-bit differences in the 16-bit GEMM 1
    # result show: the row's sums over four experts differ from the oracle's by up to 1.13e-2 of the output's largest
    # value, the same on every table form and block size (measured); all but one other row stay within 5e-3.
    assert _rel_err(eager_h.float().cpu().numpy(), ref) <= (2 * REL_TOL if T == 900 else REL_TOL)
    if T == 900:
        with monkeypatch.context() as m:
            m.setattr(fm, "blocks_want_balancing", lambda *a, **k: False)
            plain_h = fused_experts_impl(*args, **kw)
        torch.cuda.synchronize()
        assert torch.equal(plain_h, eager_h)

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        h, y = layer()
    for _ in range(3):
        h.zero_(); y.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(h, eager_h) and torch.equal(y, eager_y)
        layer()  # eager launches of the same kernels between the replays
        torch.cuda.synchronize()
