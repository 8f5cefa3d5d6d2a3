"""GPU parity of the MLA absorbed-product entry points against the oracle.

per_tensor_quant_mla_fp8 (reference: python/sglang/srt/layers/quantization/fp8_kernel.py:1221-1266): bytes and the
scale bit for bit.  bmm_fp8 (sgl-kernel/python/sgl_kernel/gemm.py:66-82; the reference's own test asks for a cosine
similarity above 0.99): max relative error <= 1e-2 against the float64 product of the de-quantised operands, and the
cosine as well.  per_token_group_quant_mla_deep_gemm_masked_fp8 (fp8_kernel.py:1319-1362): bytes and scales of the
first m rows bit for bit, layout and strides as the reference returns them."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import bf16_tensor, fp8_tensor

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _codes(rng, shape):
    return rng.integers(0, 0x70, shape, dtype=np.uint8) | (rng.integers(0, 2, shape, dtype=np.uint8) << 7)


def _rel(c, ref):
    return float(np.abs(c.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


@pytest.mark.parametrize("H,S,D,transposed", [(16, 40, 512, True), (128, 7, 128, True), (4, 300, 128, False), (1, 1, 8, False),
                                              (16, 1, 512, True)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_per_tensor_quant_mla(dev, H, S, D, transposed, dtype):
    from sglang_amd.fp8_kernel import per_tensor_quant_mla_fp8

    g = torch.Generator().manual_seed(H * 1000 + S)
    base = (torch.randn((S, H, D) if transposed else (H, S, D), generator=g) * 2.5).to(dtype)
    x_cpu = base.transpose(0, 1) if transposed else base
    x = base.to(dev).transpose(0, 1) if transposed else base.to(dev)
    s_out = torch.zeros((1,), device=dev, dtype=torch.float32)
    q, s = per_tensor_quant_mla_fp8(x, s_out)
    torch.cuda.synchronize()
    assert s is s_out and q.is_contiguous() and tuple(q.shape) == (H, S, D) and q.dtype == torch.float8_e4m3fn
    oq, os_ = O.per_tensor_quant_mla_fp8(x_cpu.float().numpy())
    assert s.cpu().numpy()[0] == os_[0]
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), oq)


def test_per_tensor_quant_mla_zero_tensor_and_errors(dev):
    from sglang_amd.fp8_kernel import per_tensor_quant_mla_fp8

    s_out = torch.zeros((1,), device=dev, dtype=torch.float32)
    q, s = per_tensor_quant_mla_fp8(torch.zeros((2, 3, 64), device=dev, dtype=torch.bfloat16), s_out)
    assert s.item() == np.float32(1e-12) / np.float32(448.0) and not q.view(torch.uint8).any()
    with pytest.raises(AssertionError):
        per_tensor_quant_mla_fp8(torch.zeros((3, 64), device=dev, dtype=torch.bfloat16), s_out)
    with pytest.raises(RuntimeError, match="contiguous last dimension"):
        per_tensor_quant_mla_fp8(torch.zeros((2, 64, 3), device=dev, dtype=torch.bfloat16).transpose(1, 2), s_out)


@pytest.mark.parametrize("b,m,n,k", [(16, 48, 80, 64), (16, 70, 512, 128), (16, 70, 128, 512), (128, 1, 512, 128), (3, 300, 264, 256)])
@pytest.mark.parametrize("res_dtype", [torch.bfloat16, torch.float16])
def test_bmm_fp8(dev, b, m, n, k, res_dtype):
    """The reference test's shape (16, 48, 64) x (16, 64, 80) and the two absorbed products of DeepSeek MLA
    (q_nope . w_kc with k = 128, n = 512; attention output . w_vc with k = 512, n = 128)."""
    from sglang_amd.sgl_kernel import bmm_fp8

    rng = np.random.default_rng(b * 7 + m)
    aq, bq = _codes(rng, (b, m, k)), _codes(rng, (b, n, k))
    sa, sb = np.float32(0.0173), np.float32(0.0021)
    A = fp8_tensor(aq, dev)
    B = fp8_tensor(bq, dev).transpose(1, 2)  # [b, k, n], column-major per entry
    res = torch.full((b, m, n), 9.0, device=dev, dtype=res_dtype)
    ret = bmm_fp8(A, B, torch.tensor(sa, device=dev), torch.tensor([sb], device=dev), res_dtype, res)
    torch.cuda.synchronize()
    assert ret is res
    ref = O.bmm_fp8(aq, bq, sa, sb, "f32")
    got = res.float().cpu().numpy()
    assert _rel(got, ref) <= REL_TOL, _rel(got, ref)
    cos = float((got.ravel().astype(np.float64) @ ref.ravel().astype(np.float64)) /
                (np.linalg.norm(got.ravel().astype(np.float64)) * np.linalg.norm(ref.ravel().astype(np.float64))))
    assert cos > 0.99
    fresh = bmm_fp8(A, B, torch.tensor(sa, device=dev), torch.tensor(sb, device=dev), res_dtype)
    assert torch.equal(fresh, res)


def test_bmm_fp8_after_mla_quant_matches_bf16_product(dev):
    """The absorbed product as the model runs it: activations quantised per tensor, weights quantised per tensor offline,
    bmm_fp8 - against torch.bmm of the bf16 operands on the CPU (what the quantised path approximates)."""
    from sglang_amd.fp8_kernel import per_tensor_quant_mla_fp8
    from sglang_amd.sgl_kernel import bmm_fp8

    g = torch.Generator().manual_seed(11)
    heads, seq, k, n = 16, 33, 128, 512
    q_nope = torch.randn((seq, heads, k), generator=g).to(torch.bfloat16)
    w_kc = (torch.randn((heads, n, k), generator=g) * 0.05).to(torch.bfloat16)
    wq, ws = O.per_tensor_quant_fp8(w_kc.float().numpy().reshape(heads * n, k))
    s_out = torch.zeros((1,), device=dev, dtype=torch.float32)
    xq, xs = per_tensor_quant_mla_fp8(q_nope.to(dev).transpose(0, 1), s_out)
    out = bmm_fp8(xq, fp8_tensor(wq.reshape(heads, n, k), dev).transpose(1, 2), xs, torch.from_numpy(ws).to(dev), torch.bfloat16)
    ref = torch.bmm(q_nope.transpose(0, 1).float(), w_kc.float().transpose(1, 2))
    cos = torch.nn.functional.cosine_similarity(ref.reshape(-1), out.float().cpu().reshape(-1), dim=0)
    assert cos > 0.99


def test_bmm_fp8_errors(dev):
    from sglang_amd.sgl_kernel import bmm_fp8

    a = torch.zeros((2, 8, 128), device=dev, dtype=torch.float8_e4m3fn)
    bt = torch.zeros((2, 16, 128), device=dev, dtype=torch.float8_e4m3fn).transpose(1, 2)
    one = torch.ones((1,), device=dev)
    with pytest.raises(RuntimeError, match="column-major"):
        bmm_fp8(a, bt.contiguous(), one, one, torch.bfloat16)
    with pytest.raises(RuntimeError, match="float8_e4m3fn"):
        bmm_fp8(a.view(torch.float8_e5m2), bt, one, one, torch.bfloat16)
    with pytest.raises(RuntimeError, match="expected"):
        bmm_fp8(a, bt[:1], one, one, torch.bfloat16)
    with pytest.raises(RuntimeError, match="one scale"):
        bmm_fp8(a, bt, torch.ones((2,), device=dev), one, torch.bfloat16)
    assert bmm_fp8(a[:0], bt[:0], one, one, torch.bfloat16).shape == (0, 8, 16)


@pytest.mark.parametrize("b,m,k,transposed", [(4, 70, 512, True), (2, 256, 256, False), (3, 300, 128, True), (16, 1, 512, True)])
def test_group_quant_mla_masked(dev, b, m, k, transposed):
    from sglang_amd.fp8_kernel import per_token_group_quant_mla_deep_gemm_masked_fp8

    x = O.make_activation(b * m, k, seed=b + m)
    if transposed:  # [m, b, k] in memory, seen as [b, m, k]
        xt = bf16_tensor(x, dev).view(m, b, k).transpose(0, 1)
        x_ref = x.reshape(m, b, k).transpose(1, 0, 2)
    else:
        xt = bf16_tensor(x, dev).view(b, m, k)
        x_ref = x.reshape(b, m, k)
    x_q, x_s, masked_m, m_ret, aligned_m = per_token_group_quant_mla_deep_gemm_masked_fp8(xt)
    torch.cuda.synchronize()
    assert m_ret == m and aligned_m == (m + 255) // 256 * 256
    assert tuple(x_q.shape) == (b, aligned_m, k) and x_q.is_contiguous()
    assert tuple(x_s.shape) == (b, aligned_m, k // 128) and x_s.stride() == (k // 128 * aligned_m, 1, aligned_m)
    assert masked_m.dtype == torch.int32 and masked_m.tolist() == [m] * b
    oq, os_ = O.per_token_group_quant_fp8(np.ascontiguousarray(x_ref).reshape(b * m, k), 128)
    assert np.array_equal(x_q[:, :m].contiguous().view(torch.uint8).cpu().numpy().reshape(b * m, k), oq)
    assert np.array_equal(x_s[:, :m].contiguous().cpu().numpy().reshape(b * m, k // 128), os_)


def test_group_quant_mla_masked_feeds_the_masked_grouped_gemm(dev):
    """The quantiser's outputs go straight into the masked grouped GEMM (the reference's use, deepseek_v2.py's
    forward_absorb with DeepGEMM): the product is the oracle's on the first m rows; the padding rows stay untouched."""
    from sglang_amd.deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_masked
    from sglang_amd.fp8_kernel import per_token_group_quant_mla_deep_gemm_masked_fp8

    rng = np.random.default_rng(2)
    b, m, k, n = 4, 45, 512, 256
    x = O.make_activation(b * m, k, seed=1)
    x_q, x_s, masked_m, _, aligned_m = per_token_group_quant_mla_deep_gemm_masked_fp8(bf16_tensor(x, dev).view(b, m, k))
    wq = np.empty((b, n, k), np.uint8); ws = np.empty((b, n // 128, k // 128), np.float32)
    for e in range(b):
        wq[e], ws[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((n, k)).astype(np.float32) * 0.05))
    out = torch.full((b, aligned_m, n), 5.0, device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_masked((x_q, x_s), (fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)), out, masked_m, m)
    got = out.float().cpu().numpy()
    oq, os_ = O.per_token_group_quant_fp8(x, 128)
    for e in range(b):
        ref = O.w8a8_block_fp8_matmul(oq[e * m:(e + 1) * m], wq[e], os_[e * m:(e + 1) * m], ws[e], acc=np.float64)
        assert _rel(got[e, :m], ref) <= REL_TOL
    assert (got[:, m:] == 5.0).all()
