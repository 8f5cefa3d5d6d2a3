"""GPU parity of the FP8 GEMMs against the CPU oracle.

Tolerance (stated by the task): max relative error <= 1e-2 on bf16 output with fp32 accumulation,
measured as max|C - C_ref| / max|C_ref| against the float64 oracle; integer-valued inputs with
power-of-two scales must be reproduced exactly.
"""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import fp8_tensor

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _quantised_problem(M, N, K, seed):
    x = O.make_activation(M, K, seed)
    w = O.make_weight(N, K, seed)
    xq, xs = O.per_token_group_quant_fp8(x, 128)
    wq, ws = O.block_quant_weight(w)
    return xq, xs, wq, ws


def _rel_err(c, ref):
    return float(np.abs(c.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


def _run_block(xq, xs, wq, ws, dev, out_dtype=torch.bfloat16, col_major_as=False, api="triton"):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    A = fp8_tensor(xq, dev)
    B = fp8_tensor(wq, dev)
    As = torch.from_numpy(xs).to(dev)
    Bs = torch.from_numpy(ws).to(dev)
    if col_major_as:
        As = As.t().contiguous().t()
    if api == "triton":
        C = w8a8_block_fp8_matmul(A, B, As, Bs, [128, 128], out_dtype)
    else:
        C = fp8_blockwise_scaled_mm(A, B.t(), As.t().contiguous().t(), Bs.t(), out_dtype)
    torch.cuda.synchronize()
    return C.float().cpu().numpy()


@pytest.mark.parametrize("M", [1, 5, 32, 127, 128, 256, 300, 1024])
@pytest.mark.parametrize("N,K", [(512, 512), (4608, 1024), (1536, 2304)])
def test_block_gemm_vs_oracle(dev, M, N, K):
    xq, xs, wq, ws = _quantised_problem(M, N, K, seed=M + N)
    ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="f32", acc=np.float64)
    for api in ("triton", "sgl"):
        c = _run_block(xq, xs, wq, ws, dev, api=api)
        assert _rel_err(c, ref) <= REL_TOL, (api, _rel_err(c, ref))


def test_block_gemm_config1(dev):
    """BASELINE config 1: x [32,4096] with outliers, W [4096,4096], seed 0, through the linear entry point."""
    from sglang_amd.fp8_utils import dispatch_w8a8_block_fp8_linear
    from tests.conftest import bf16_tensor

    x = O.make_activation(32, 4096, 0)
    w = O.make_weight(4096, 4096, 0)
    wq, ws = O.block_quant_weight(w)
    ref = O.block_fp8_linear(x, wq, ws)
    fn = dispatch_w8a8_block_fp8_linear()
    out = fn(bf16_tensor(x, dev), fp8_tensor(wq, dev), [128, 128], torch.from_numpy(ws).to(dev))
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and out.shape == (32, 4096)
    assert _rel_err(out.float().cpu().numpy(), ref) <= REL_TOL


@pytest.mark.parametrize("M", [16, 1024])
@pytest.mark.parametrize("N,K", [(24576, 1536), (32768, 512), (7168, 16384), (4608, 7168), (7168, 2304)])
def test_block_gemm_deepseek_shapes(dev, M, N, K):
    """DeepSeek-V3 projection shapes; checked on a sample of output rows/columns against the oracle."""
    rng = np.random.default_rng(N + K + M)
    xq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((M, K)).astype(np.float32) * 100, -448, 448))
    wq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((N, K)).astype(np.float32) * 100, -448, 448))
    xs = rng.uniform(0.5, 2.0, (M, K // 128)).astype(np.float32) * 1e-2
    ws = rng.uniform(0.5, 2.0, (N // 128, K // 128)).astype(np.float32) * 1e-3
    c = _run_block(xq, xs, wq, ws, dev)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 6)]))
    cols = np.unique(np.concatenate([np.arange(0, 130), np.arange(N - 130, N), rng.integers(0, N, 300)]))
    ws_cols = ws[cols // 128]
    a = O.e4m3fn_to_f32(xq[rows]).astype(np.float64)
    b = O.e4m3fn_to_f32(wq[cols]).astype(np.float64)
    ref = np.zeros((rows.size, cols.size))
    for kb in range(K // 128):
        sl = slice(kb * 128, (kb + 1) * 128)
        ref += (a[:, sl] @ b[:, sl].T) * xs[rows, kb][:, None] * ws_cols[:, kb][None, :]
    got = c[np.ix_(rows, cols)]
    assert _rel_err(got, ref) <= REL_TOL


def test_block_gemm_headline_full_size(dev):
    """The benchmark's own shape (M=4096 against the [18432, 7168] gate_up weight): a sample of rows and columns
    against the oracle, and two properties that need no oracle at this size - a row of the output depends on
    nothing but its own activation row (permuting rows permutes the result bit for bit, whatever tile a row
    lands in), and power-of-two scale factors pass through exactly."""
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    M, N, K = 4096, 18432, 7168
    rng = np.random.default_rng(4096)

    def codes(shape):  # random e4m3fn bytes of moderate magnitude, no NaN codes
        b = rng.integers(0, 0x60, shape, dtype=np.uint8) | (rng.integers(0, 2, shape, dtype=np.uint8) << 7)
        return b

    xq, wq = codes((M, K)), codes((N, K))
    xs = (rng.uniform(0.5, 2.0, (M, K // 128)) * 1e-2).astype(np.float32)
    ws = (rng.uniform(0.5, 2.0, (N // 128, K // 128)) * 1e-3).astype(np.float32)
    A, B = fp8_tensor(xq, dev), fp8_tensor(wq, dev)
    As, Bs = torch.from_numpy(xs).to(dev).t().contiguous().t(), torch.from_numpy(ws).to(dev)
    C = w8a8_block_fp8_matmul(A, B, As, Bs, [128, 128], torch.bfloat16)

    rows = np.unique(np.concatenate([[0, 255, 256, M - 1], rng.integers(0, M, 6)]))
    cols = np.unique(np.concatenate([np.arange(0, 130), np.arange(N - 130, N), rng.integers(0, N, 300)]))
    a = O.e4m3fn_to_f32(xq[rows]).astype(np.float64)
    b = O.e4m3fn_to_f32(wq[cols]).astype(np.float64)
    ws_cols = ws[cols // 128]
    ref = np.zeros((rows.size, cols.size))
    for kb in range(K // 128):
        sl = slice(kb * 128, (kb + 1) * 128)
        ref += (a[:, sl] @ b[:, sl].T) * xs[rows, kb][:, None] * ws_cols[:, kb][None, :]
    got = C[torch.from_numpy(rows).to(dev)][:, torch.from_numpy(cols).to(dev)].float().cpu().numpy()
    assert _rel_err(got, ref) <= REL_TOL

    perm = torch.from_numpy(rng.permutation(M)).to(dev)
    Ap = A.view(torch.uint8)[perm].contiguous().view(torch.float8_e4m3fn)
    Cp = w8a8_block_fp8_matmul(Ap, B, As[perm].t().contiguous().t(), Bs, [128, 128], torch.bfloat16)
    assert torch.equal(Cp, C[perm])
    C4 = w8a8_block_fp8_matmul(A, B, As * 0.5, Bs * 8.0, [128, 128], torch.bfloat16)
    assert torch.equal(C4, C * 4.0)


@pytest.mark.parametrize("M,N,K", [(64, 256, 256), (256, 512, 1024), (1024, 256, 4096), (3, 384, 128)])
def test_block_gemm_exact_on_integers(dev, M, N, K):
    """Small integers and power-of-two scales: every partial sum is exactly representable."""
    rng = np.random.default_rng(K)
    xv = rng.integers(-4, 5, (M, K)).astype(np.float32)
    wv = rng.integers(-4, 5, (N, K)).astype(np.float32)
    xq, wq = O.f32_to_e4m3fn(xv), O.f32_to_e4m3fn(wv)
    xs = (2.0 ** rng.integers(-3, 3, (M, K // 128))).astype(np.float32)
    ws = (2.0 ** rng.integers(-3, 3, (N // 128, K // 128))).astype(np.float32)
    ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="bf16", acc=np.float64)
    c = _run_block(xq, xs, wq, ws, dev)
    np.testing.assert_array_equal(c, ref)
    c16 = _run_block(xq, xs, wq, ws, dev, out_dtype=torch.float16)
    np.testing.assert_array_equal(c16, O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="f16", acc=np.float64))


@pytest.mark.parametrize("M", [3700, 3840, 4000])
def test_block_gemm_last_round_in_half_tiles_exact(dev, M):
    """More 256x256 tiles than CUs with a last round that fills less than half of them: those tiles run as two
    128-row halves.  M = 3700 leaves a tile whose upper half lies past the last row, 4000 one whose upper half holds
    32 rows, 3840 (a multiple of 256) none that is ragged.  Integer data: exact."""
    N, K = 18432, 256
    rng = np.random.default_rng(M)
    xq = O.f32_to_e4m3fn(rng.integers(-4, 5, (M, K)).astype(np.float32))
    wq = O.f32_to_e4m3fn(rng.integers(-4, 5, (N, K)).astype(np.float32))
    xs = (2.0 ** rng.integers(-3, 3, (M, K // 128))).astype(np.float32)
    ws = (2.0 ** rng.integers(-3, 3, (N // 128, K // 128))).astype(np.float32)
    tiles = ((M + 255) // 256) * (N // 256)
    assert tiles > 256 and 0 < tiles % 256 <= 128
    c = _run_block(xq, xs, wq, ws, dev)
    np.testing.assert_array_equal(c, O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="bf16", acc=np.float64))


def test_block_gemm_scale_layouts_agree(dev):
    xq, xs, wq, ws = _quantised_problem(200, 512, 1024, 9)
    a = _run_block(xq, xs, wq, ws, dev, col_major_as=False)
    b = _run_block(xq, xs, wq, ws, dev, col_major_as=True)
    c = _run_block(xq, xs, wq, ws, dev, api="sgl")
    np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(a, c)


@pytest.mark.parametrize("N,K", [(1088, 512), (136, 272), (512, 144)])
def test_block_gemm_unaligned_shapes(dev, N, K):
    """N or K not multiples of 128 (the reference's Triton path admits them)."""
    M = 37
    rng = np.random.default_rng(N)
    xq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((M, K)).astype(np.float32) * 50, -448, 448))
    wq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((N, K)).astype(np.float32) * 50, -448, 448))
    kt, nt = (K + 127) // 128, (N + 127) // 128
    xs = rng.uniform(0.5, 2, (M, kt)).astype(np.float32)
    ws = rng.uniform(0.5, 2, (nt, kt)).astype(np.float32)
    ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="f32", acc=np.float64)
    c = _run_block(xq, xs, wq, ws, dev)
    assert _rel_err(c, ref) <= REL_TOL


def test_block_gemm_random_shapes_every_plan(dev):
    """Sixty seeded random shapes (M 1..1500, N a multiple of 8 up to 6144, K a multiple of 128 up to 2304) with
    random scale layouts: whatever kernel family and K cut the plan picks, exact on integer data."""
    rng = np.random.default_rng(20250101)
    for case in range(60):
        M = int(rng.choice([rng.integers(1, 40), rng.integers(40, 300), rng.integers(300, 1500)]))
        N = int(rng.integers(1, 769)) * 8
        K = int(rng.integers(1, 19)) * 128
        xq = O.f32_to_e4m3fn(rng.integers(-4, 5, (M, K)).astype(np.float32))
        wq = O.f32_to_e4m3fn(rng.integers(-4, 5, (N, K)).astype(np.float32))
        xs = (2.0 ** rng.integers(-3, 3, (M, K // 128))).astype(np.float32)
        ws = (2.0 ** rng.integers(-3, 3, ((N + 127) // 128, K // 128))).astype(np.float32)
        ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="bf16", acc=np.float64)
        c = _run_block(xq, xs, wq, ws, dev, col_major_as=bool(case & 1))
        assert np.array_equal(c, ref), "case %d: M=%d N=%d K=%d" % (case, M, N, K)


@pytest.mark.parametrize("nw", [0, 1, 2, 4, 8])
def test_decode_gemm_with_k_cut_across_waves_is_exact_on_integers(dev, nw):
    """The decode kernel that cuts K across the waves of a workgroup (partial sums meet in LDS), pinned with every
    wave layout (0 = the plan's own): K block counts that do not divide by the number of K ranges (waves with short or
    empty ranges), N not a multiple of the 16 rows of a wave, 1 .. 32 rows, both scale layouts, bf16 and fp16 output -
    integer data with power-of-two scales, so the sums are exact whatever their order - and the same through
    fp8_scaled_mm with a bias."""
    from sglang_amd._lib import lib
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    rng = np.random.default_rng(77 + nw)
    lib.fp8k_tune_force_gemm_plan(5, nw)
    try:
        for case, (M, N, K) in enumerate([(1, 4096, 4096), (7, 1000, 128 * 5), (16, 264, 128 * 19), (17, 4608, 128 * 9),
                                          (32, 7168, 2304), (3, 8, 128), (29, 520, 128 * 33)]):
            xq = O.f32_to_e4m3fn(rng.integers(-4, 5, (M, K)).astype(np.float32))
            wq = O.f32_to_e4m3fn(rng.integers(-4, 5, (N, K)).astype(np.float32))
            xs = (2.0 ** rng.integers(-3, 3, (M, K // 128))).astype(np.float32)
            ws = (2.0 ** rng.integers(-3, 3, ((N + 127) // 128, K // 128))).astype(np.float32)
            dt, name = (torch.bfloat16, "bf16") if case & 1 else (torch.float16, "f16")
            ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype=name, acc=np.float64)
            c = _run_block(xq, xs, wq, ws, dev, col_major_as=bool(case & 2), out_dtype=dt)
            assert np.array_equal(c, ref), "nw=%d M=%d N=%d K=%d" % (nw, M, N, K)
            sa = (2.0 ** rng.integers(-3, 3, (M,))).astype(np.float32)
            sb = (2.0 ** rng.integers(-3, 3, (N,))).astype(np.float32)
            bias = torch.from_numpy(rng.integers(-8, 9, (N,)).astype(np.float32))
            got = fp8_scaled_mm(fp8_tensor(xq, dev), fp8_tensor(wq, dev).t(), torch.from_numpy(sa).to(dev),
                                torch.from_numpy(sb).to(dev), torch.bfloat16, bias.to(dev)).float().cpu().numpy()
            want = O.fp8_scaled_mm(xq, wq, sa, sb, out_dtype="bf16", bias=bias.numpy())
            assert np.array_equal(got, want), "row mode nw=%d M=%d N=%d K=%d" % (nw, M, N, K)
    finally:
        lib.fp8k_tune_force_gemm_plan(-1, 0)


def _run_scaled_mm(aq, bq, sa, sb, dev, out_dtype=torch.bfloat16, bias=None):
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    A = fp8_tensor(aq, dev)
    B = fp8_tensor(bq, dev).t()
    C = fp8_scaled_mm(A, B, torch.from_numpy(sa).to(dev), torch.from_numpy(sb).to(dev), out_dtype,
                      None if bias is None else bias.to(dev))
    torch.cuda.synchronize()
    return C.float().cpu().numpy()


@pytest.mark.parametrize("M", [1, 8, 64, 512, 2048])
@pytest.mark.parametrize("N,K", [(6144, 4096), (4096, 14336)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_scaled_mm_llama_shapes(dev, M, N, K, with_bias):
    rng = np.random.default_rng(M + N)
    x = O.make_activation(M, K, M)
    aq, sa = O.per_token_quant_fp8(x)
    w = O.make_weight(N, K, N)
    bq, sbt = O.per_tensor_quant_fp8(w)
    sb = np.full((N,), sbt[0], dtype=np.float32)
    bias = torch.from_numpy(O.to_bf16(rng.standard_normal(N).astype(np.float32))).to(torch.bfloat16) if with_bias else None
    ref = O.fp8_scaled_mm(aq, bq, sa.reshape(-1), sb, "f32", None if bias is None else bias.float().numpy())
    c = _run_scaled_mm(aq, bq, sa, sb, dev, bias=bias)
    assert _rel_err(c, ref) <= REL_TOL
    if with_bias:
        c32 = _run_scaled_mm(aq, bq, sa, sb, dev, bias=bias.float())
        np.testing.assert_array_equal(c, c32)


def test_scaled_mm_exact_and_fp16(dev):
    rng = np.random.default_rng(1)
    M, N, K = 130, 512, 1024
    aq = O.f32_to_e4m3fn(rng.integers(-3, 4, (M, K)).astype(np.float32))
    bq = O.f32_to_e4m3fn(rng.integers(-3, 4, (N, K)).astype(np.float32))
    sa = (2.0 ** rng.integers(-2, 3, M)).astype(np.float32)
    sb = (2.0 ** rng.integers(-2, 3, N)).astype(np.float32)
    for dt, name in ((torch.bfloat16, "bf16"), (torch.float16, "f16")):
        c = _run_scaled_mm(aq, bq, sa, sb, dev, out_dtype=dt)
        np.testing.assert_array_equal(c, O.fp8_scaled_mm(aq, bq, sa, sb, name))


def test_gemm_errors(dev):
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm

    a = torch.zeros((4, 256), dtype=torch.float8_e4m3fn, device=dev)
    b = torch.zeros((256, 256), dtype=torch.float8_e4m3fn, device=dev)
    sa = torch.ones((4, 2), device=dev).t().contiguous().t()
    sb = torch.ones((2, 2), device=dev)
    with pytest.raises(RuntimeError, match="column major"):
        fp8_blockwise_scaled_mm(a, b, sa, sb, torch.bfloat16)
    with pytest.raises(RuntimeError, match="Half or BFloat16"):
        fp8_blockwise_scaled_mm(a, b.t(), sa, sb, torch.float32)
    with pytest.raises(RuntimeError, match="scales_a"):
        fp8_blockwise_scaled_mm(a, b.t(), sa[:, :1], sb, torch.bfloat16)
    with pytest.raises(RuntimeError, match="Float8_e4m3fn"):
        fp8_blockwise_scaled_mm(a.view(torch.uint8), b.t(), sa, sb, torch.bfloat16)
    with pytest.raises(RuntimeError, match="bias"):
        fp8_scaled_mm(a, b.t(), torch.ones(4, device=dev), torch.ones(256, device=dev), torch.bfloat16,
                      torch.ones(255, device=dev))
    out = fp8_blockwise_scaled_mm(a[:0], b.t(), sa[:0], sb, torch.bfloat16)
    assert out.shape == (0, 256)


@pytest.mark.parametrize("M,N,K", [(129, 256, 256), (300, 512, 1024), (1024, 4608, 1536), (2048, 1536, 7168), (64, 512, 512)])
def test_block_gemm_ue8m0_hardware_scales(dev, M, N, K):
    """UE8M0 path (reference: the DeepGEMM branch with DEEPGEMM_SCALE_UE8M0, fp8_utils.py:229-268): activations
    quantised with power-of-two scales (packed bytes), weight scales rounded up to powers of two; the matrix core
    applies both.  Checked against the oracle's block matmul on the very same (unpacked) scales, <= 1e-2, and
    against this library's float-scale kernel on the unpacked scales."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.sgl_kernel import mark_ue8m0, unpack_ue8m0_scales

    x = O.make_activation(M, K, seed=M)
    w = O.make_weight(N, K, seed=N)
    wq, ws = O.block_quant_weight(w)
    ws2 = O.ceil_to_ue8m0(ws)                     # power-of-two weight scales (the bytes stay as they are:
    xt = torch.from_numpy(x).to(dev).to(torch.bfloat16)  # only the GEMM's use of the scales is under test)
    xq, xs_packed = sglang_per_token_group_quant_fp8(xt, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    B, Bs = fp8_tensor(wq, dev), mark_ue8m0(torch.from_numpy(ws2).to(dev))
    c = w8a8_block_fp8_matmul(xq, B, xs_packed, Bs, [128, 128], torch.bfloat16)
    xs = unpack_ue8m0_scales(xs_packed, K // 128)
    c_float = w8a8_block_fp8_matmul(xq, B, xs, Bs, [128, 128], torch.bfloat16)
    torch.cuda.synchronize()
    ref = O.w8a8_block_fp8_matmul(xq.view(torch.uint8).cpu().numpy(), wq, xs.cpu().numpy(), ws2, acc=np.float64)
    assert _rel_err(c.float().cpu().numpy(), ref) <= REL_TOL
    assert _rel_err(c.float().cpu().numpy(), c_float.float().cpu().numpy()) <= REL_TOL


def test_ue8m0_requantised_checkpoint_end_to_end(dev):
    """A float-scale block-FP8 weight passed through requant_weight_ue8m0 (reference: fp8_utils.py:453-476) and then
    the UE8M0 linear: equal to the oracle on the requantised weight to 1e-2, and close to the float-scale linear of
    the original weight (both are 8-bit renderings of the same bf16 numbers)."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.fp8_utils import requant_weight_ue8m0, w8a8_block_fp8_linear
    from sglang_amd.sgl_kernel import mark_ue8m0, unpack_ue8m0_scales

    M, N, K = 384, 768, 1024
    x = torch.from_numpy(O.make_activation(M, K, seed=1)).to(dev).to(torch.bfloat16)
    wq, ws = O.block_quant_weight(O.make_weight(N, K, seed=2))
    W, Ws = fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)
    W2, Ws2 = requant_weight_ue8m0(W, Ws, [128, 128])
    xq, xs_packed = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    c = w8a8_block_fp8_matmul(xq, W2, xs_packed, Ws2, [128, 128], torch.bfloat16)
    ref = O.w8a8_block_fp8_matmul(xq.view(torch.uint8).cpu().numpy(), W2.view(torch.uint8).cpu().numpy(),
                                  unpack_ue8m0_scales(xs_packed, K // 128).cpu().numpy(), Ws2.cpu().numpy(), acc=np.float64)
    assert _rel_err(c.float().cpu().numpy(), ref) <= REL_TOL
    c_float = w8a8_block_fp8_linear(x, W, [128, 128], Ws)
    assert _rel_err(c.float().cpu().numpy(), c_float.float().cpu().numpy()) <= 0.08


@pytest.mark.parametrize("M", [40, 128, 129, 700])
def test_packed_ue8m0_scales_next_to_ordinary_float_weight_scales(dev, M):
    """Packed UE8M0 activation scales with float32 weight scales that are NOT powers of two: a float scale is never
    read as a bare exponent, whatever the batch size (below and above the 128 rows from which the tile kernels could
    apply exponents in hardware) - the result is the oracle's on the expanded scales (<= 1e-2) and, bit for bit, that
    of the float-scale call on the expanded scales."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.sgl_kernel import unpack_ue8m0_scales

    N, K = 768, 1024
    x = torch.from_numpy(O.make_activation(M, K, seed=M)).to(dev).to(torch.bfloat16)
    wq, ws = O.block_quant_weight(O.make_weight(N, K, seed=N))     # amax/448 scales: mantissas all over the place
    xq, xs_packed = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    B, Bs = fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)
    c = w8a8_block_fp8_matmul(xq, B, xs_packed, Bs, [128, 128], torch.bfloat16)
    xs = unpack_ue8m0_scales(xs_packed, K // 128)
    ref = O.w8a8_block_fp8_matmul(xq.view(torch.uint8).cpu().numpy(), wq, xs.cpu().numpy(), ws, acc=np.float64)
    assert _rel_err(c.float().cpu().numpy(), ref) <= REL_TOL
    assert torch.equal(c, w8a8_block_fp8_matmul(xq, B, xs, Bs, [128, 128], torch.bfloat16))


@pytest.mark.parametrize("M", [64, 300])
def test_packed_ue8m0_weight_scales(dev, M):
    """Weight scales as packed UE8M0 words, one row per weight row (the layout the reference prepares for DeepGEMM,
    fp8_kernel.py:1036-1043), with packed activation scales: equal to the float form of the same powers of two."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.sgl_kernel import mark_ue8m0, unpack_ue8m0_scales

    N, K = 512, 1280
    x = torch.from_numpy(O.make_activation(M, K, seed=M)).to(dev).to(torch.bfloat16)
    wq, ws = O.block_quant_weight(O.make_weight(N, K, seed=N))
    ws2 = O.ceil_to_ue8m0(ws)
    packed_rows = torch.from_numpy(O.pack_ue8m0_scales(np.repeat(ws2, 128, axis=0))).to(dev)   # [N, ceil(10/4)]
    xq, xs_packed = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    B = fp8_tensor(wq, dev)
    c = w8a8_block_fp8_matmul(xq, B, xs_packed, packed_rows, [128, 128], torch.bfloat16)
    c_float = w8a8_block_fp8_matmul(xq, B, xs_packed, mark_ue8m0(torch.from_numpy(ws2).to(dev)), [128, 128], torch.bfloat16)
    assert torch.equal(c, c_float)
    # the same words in the mn-major storage transform_scale_ue8m0 produces (reference: fp8_utils.py:505-515)
    from sglang_amd.fp8_utils import transform_scale_ue8m0

    mn_major = transform_scale_ue8m0(torch.from_numpy(ws2).to(dev), N)
    assert mn_major.stride(0) == 1 and torch.equal(mn_major, packed_rows)
    assert torch.equal(w8a8_block_fp8_matmul(xq, B, xs_packed, mn_major, [128, 128], torch.bfloat16), c)
    ref = O.w8a8_block_fp8_matmul(xq.view(torch.uint8).cpu().numpy(), wq,
                                  unpack_ue8m0_scales(xs_packed, K // 128).cpu().numpy(), ws2, acc=np.float64)
    assert _rel_err(c.float().cpu().numpy(), ref) <= REL_TOL


@pytest.mark.parametrize("case", ["a", "b", "c"])
def test_linear_path_against_golden_vectors(dev, case):
    """Quant and GEMM through the library against tests/golden/w8a8_vectors.npz, which torch library ops alone wrote
    (tests/golden/make_vectors.py): quantised bytes and scales bit for bit, the product within the stated tolerance."""
    import os
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul

    G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "w8a8_vectors.npz"))
    x = torch.from_numpy(G[case + "_x_bf16_bits"].view(np.int16)).view(torch.bfloat16).to(dev)
    for col in (False, True):
        q, s = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=col)
        torch.cuda.synchronize()
        assert np.array_equal(q.view(torch.uint8).cpu().numpy(), G[case + "_q"])
        assert np.array_equal(s.cpu().numpy(), G[case + "_s"])
        y = w8a8_block_fp8_matmul(q, fp8_tensor(G[case + "_wq"], dev), s, torch.from_numpy(G[case + "_ws"]).to(dev),
                                  [128, 128], torch.bfloat16)
        torch.cuda.synchronize()
        assert _rel_err(y.float().cpu().numpy(), G[case + "_y"]) <= REL_TOL


def test_stream_read_write_probe_writes_its_pattern_and_checks_its_arguments(dev):
    """The measurement aid fp8k_tune_stream_read_write: every workgroup writes 8 KB x stores_per_wave after each tile of
    stages, all of it inside the caller's buffer (words 1, 2, 3, tile index), nothing beyond; too small a destination
    is refused."""
    from sglang_amd._lib import lib, stream_ptr

    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    spt, spw, tiles = 3, 2, 4
    share = 32768 * spt * tiles
    src = torch.zeros(ncu * share + 4096, dtype=torch.uint8, device=dev)
    written = ncu * tiles * 8 * spw * 1024
    dst = torch.full((written // 4 + 1024,), -1, dtype=torch.int32, device=dev)
    rc = lib.fp8k_tune_stream_read_write(src.data_ptr(), src.numel(), dst.data_ptr(), written, spt, spw, stream_ptr(dev))
    assert rc == 0, lib.fp8k_last_error()
    torch.cuda.synchronize()
    got = dst.cpu().numpy()
    body = got[: written // 4].reshape(ncu, tiles, 8 * spw * 64, 4)
    assert (body[..., 0] == 1).all() and (body[..., 1] == 2).all() and (body[..., 2] == 3).all()
    assert (body[..., 3] == np.arange(tiles)[None, :, None]).all()
    assert (got[written // 4:] == -1).all()
    rc = lib.fp8k_tune_stream_read_write(src.data_ptr(), src.numel(), dst.data_ptr(), written - 1, spt, spw, stream_ptr(dev))
    assert rc != 0 and b"dst holds" in lib.fp8k_last_error()


def test_mfma_probes_compute_what_they_claim_and_check_their_arguments(dev):
    """The measurement aids fp8k_tune_mfma_peak / fp8k_tune_mfma_loop: on operand bytes 0x38 (1.0 in e4m3) every one of the
    bare loop's 8 x 16 accumulator values per lane is 64 x iters, on all-zero bytes every form sums to zero; the FLOP
    counts they report are those of their MFMAs; a form outside 1..6 is refused."""
    import ctypes

    from sglang_amd._lib import lib, stream_ptr

    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.full((ncu * 512,), float("nan"), dtype=torch.float32, device=dev)
    ones = torch.full((1 << 20,), 0x38, dtype=torch.uint8, device=dev)
    zeros = torch.zeros(1 << 20, dtype=torch.uint8, device=dev)
    flops = ctypes.c_int64(0)
    iters = 4
    rc = lib.fp8k_tune_mfma_peak(ones.data_ptr(), ones.numel(), iters, sink.data_ptr(), sink.numel(), ctypes.byref(flops),
                                 stream_ptr(dev))
    assert rc == 0, lib.fp8k_last_error()
    torch.cuda.synchronize()
    assert flops.value == ncu * 8 * iters * 8 * 2 * 32 * 32 * 64
    assert (sink == 128 * 64.0 * iters).all()
    for form in (1, 2, 3, 4, 5, 6):
        sink.fill_(float("nan"))
        rc = lib.fp8k_tune_mfma_loop(zeros.data_ptr(), zeros.numel(), iters, form, sink.data_ptr(), sink.numel(),
                                     ctypes.byref(flops), stream_ptr(dev))
        assert rc == 0, lib.fp8k_last_error()
        torch.cuda.synchronize()
        assert flops.value == ncu * 8 * iters * 16 * 2 * 32 * 32 * 64
        assert (sink == 0).all(), "form %d" % form
    # with ones the block-scaled forms fold 64-sums with scales within 1e-7 of one: 8 accumulators x 16 values per lane,
    # `iters` K blocks each (the products of the last block's final step are still pending in the short-lived pair)
    rc = lib.fp8k_tune_mfma_loop(ones.data_ptr(), ones.numel(), iters, 2, sink.data_ptr(), sink.numel(), ctypes.byref(flops),
                                 stream_ptr(dev))
    assert rc == 0, lib.fp8k_last_error()
    torch.cuda.synchronize()
    got = sink.cpu().numpy()
    assert np.isfinite(got).all() and (got > 0).all()
    assert np.allclose(got, got[0], rtol=1e-5)
    rc = lib.fp8k_tune_mfma_loop(zeros.data_ptr(), zeros.numel(), iters, 7, sink.data_ptr(), sink.numel(), ctypes.byref(flops),
                                 stream_ptr(dev))
    assert rc != 0 and b"form" in lib.fp8k_last_error()
