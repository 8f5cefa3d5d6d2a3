"""GPU parity of the 128x128 tile kernel (gemm_tile128_kernel), pinned through fp8k_tune_force_gemm_plan so that
every shape below runs on it whatever the automatic plan would pick: block, per-token and UE8M0 modes, ragged M and
N, odd and even numbers of K blocks, K cuts with the float-partial reduction, fp16 output, strided output rows.

Tolerance as for the other GEMM tests: max|C - C_ref| / max|C_ref| <= 1e-2 against the float64 oracle; integer-valued
inputs with power-of-two scales must be reproduced exactly.
"""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import fp8_tensor
from tests.test_gemm_gpu import REL_TOL, _quantised_problem, _rel_err, _run_block, _run_scaled_mm

pytestmark = pytest.mark.gpu


@pytest.fixture
def tile128():
    """force(splits) pins the kernel; the automatic choice is restored afterwards."""
    from sglang_amd._lib import lib

    yield lambda splits: lib.fp8k_tune_force_gemm_plan(4, splits)
    lib.fp8k_tune_force_gemm_plan(-1, 0)


@pytest.mark.parametrize("splits", [1, 2, 3])
@pytest.mark.parametrize("M,N,K", [(1, 128, 128), (37, 136, 384), (128, 512, 1024), (200, 1000, 1536), (300, 520, 2304),
                                   (640, 384, 640)])
def test_tile128_block_vs_oracle(dev, tile128, M, N, K, splits):
    xq, xs, wq, ws = _quantised_problem(M, N, K, seed=M + N + K)
    ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="f32", acc=np.float64)
    tile128(splits)
    for col_major in (False, True):
        c = _run_block(xq, xs, wq, ws, dev, col_major_as=col_major)
        assert _rel_err(c, ref) <= REL_TOL, (col_major, _rel_err(c, ref))
    c16 = _run_block(xq, xs, wq, ws, dev, out_dtype=torch.float16)
    assert _rel_err(c16, ref) <= REL_TOL


@pytest.mark.parametrize("splits", [1, 2])
def test_tile128_block_exact_on_integers(dev, tile128, splits):
    rng = np.random.default_rng(7)
    M, N, K = 257, 392, 896
    xq = O.f32_to_e4m3fn(rng.integers(-4, 5, (M, K)).astype(np.float32))
    wq = O.f32_to_e4m3fn(rng.integers(-4, 5, (N, K)).astype(np.float32))
    xs = (2.0 ** rng.integers(-3, 4, (M, K // 128))).astype(np.float32)
    ws = (2.0 ** rng.integers(-3, 4, ((N + 127) // 128, K // 128))).astype(np.float32)
    ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="bf16")
    tile128(splits)
    np.testing.assert_array_equal(_run_block(xq, xs, wq, ws, dev), ref)


@pytest.mark.parametrize("splits", [1, 2])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("M,N,K", [(70, 264, 512), (333, 640, 1152)])
def test_tile128_scaled_mm(dev, tile128, M, N, K, with_bias, splits):
    rng = np.random.default_rng(M + N)
    aq, sa = O.per_token_quant_fp8(O.make_activation(M, K, M))
    bq, sbt = O.per_tensor_quant_fp8(O.make_weight(N, K, N))
    sb = (sbt[0] * rng.uniform(0.5, 2.0, N)).astype(np.float32)
    bias = torch.from_numpy(O.to_bf16(rng.standard_normal(N).astype(np.float32))).to(torch.bfloat16) if with_bias else None
    ref = O.fp8_scaled_mm(aq, bq, sa.reshape(-1), sb, "f32", None if bias is None else bias.float().numpy())
    tile128(splits)
    assert _rel_err(_run_scaled_mm(aq, bq, sa, sb, dev, bias=bias), ref) <= REL_TOL
    bias16 = None if bias is None else bias.float()  # the bias must have the output's type or float32
    assert _rel_err(_run_scaled_mm(aq, bq, sa, sb, dev, out_dtype=torch.float16, bias=bias16), ref) <= REL_TOL


@pytest.mark.parametrize("splits", [1, 2])
@pytest.mark.parametrize("M,N,K", [(129, 256, 256), (300, 520, 1024), (512, 1536, 1664)])
def test_tile128_ue8m0(dev, tile128, M, N, K, splits):
    """Packed UE8M0 activation exponents and power-of-two weight scales applied by the matrix core."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.sgl_kernel import mark_ue8m0, unpack_ue8m0_scales

    x = O.make_activation(M, K, seed=M)
    wq, ws = O.block_quant_weight(O.make_weight(N, K, seed=N))
    ws2 = O.ceil_to_ue8m0(ws)
    xt = torch.from_numpy(x).to(dev).to(torch.bfloat16)
    xq, xs_packed = sglang_per_token_group_quant_fp8(xt, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    B, Bs = fp8_tensor(wq, dev), mark_ue8m0(torch.from_numpy(ws2).to(dev))
    tile128(splits)
    c = w8a8_block_fp8_matmul(xq, B, xs_packed, Bs, [128, 128], torch.bfloat16)
    torch.cuda.synchronize()
    xs = unpack_ue8m0_scales(xs_packed, K // 128)
    ref = O.w8a8_block_fp8_matmul(xq.view(torch.uint8).cpu().numpy(), wq, xs.cpu().numpy(), ws2, acc=np.float64)
    assert _rel_err(c.float().cpu().numpy(), ref) <= REL_TOL


def test_tile128_strided_output_rows(dev, tile128):
    """ldc that is not a multiple of 8 elements takes the 8-byte store path; the padding columns stay untouched."""
    from sglang_amd._lib import check, lib, stream_ptr

    M, N, K = 150, 264, 512
    xq, xs, wq, ws = _quantised_problem(M, N, K, seed=3)
    ref = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="f32", acc=np.float64)
    A, B = fp8_tensor(xq, dev), fp8_tensor(wq, dev)
    As, Bs = torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev)
    for ldc in (N + 4, N + 8):
        C = torch.full((M, ldc), 7.0, dtype=torch.bfloat16, device=dev)
        tile128(1)
        need = lib.fp8k_block_gemm_workspace_bytes(M, N, K)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        check(lib.fp8k_block_gemm(A.data_ptr(), B.data_ptr(), As.data_ptr(), Bs.data_ptr(), C.data_ptr(), M, N, K, K, K,
                                  As.stride(0), As.stride(1), Bs.stride(0), Bs.stride(1), ldc, 2, ws.data_ptr(), need,
                                  stream_ptr(dev)))
        torch.cuda.synchronize()
        out = C.float().cpu().numpy()
        assert _rel_err(out[:, :N], ref) <= REL_TOL
        assert (out[:, N:] == 7.0).all()


def test_automatic_plan_matches_pinned_kernels(dev):
    """Shapes on which the automatic plan takes the 128x128 kernel give the same bytes as with the kernel pinned
    (same summation order), and stay within tolerance of the other families' result."""
    from sglang_amd._lib import lib

    try:
        for (M, N, K) in ((128, 4608, 1536), (512, 1024, 1024), (256, 7168, 2304)):
            xq, xs, wq, ws = _quantised_problem(M, N, K, seed=M)
            lib.fp8k_tune_force_gemm_plan(-1, 0)
            auto = _run_block(xq, xs, wq, ws, dev)
            lib.fp8k_tune_force_gemm_plan(1, 0)
            other = _run_block(xq, xs, wq, ws, dev)
            assert _rel_err(auto, other) <= REL_TOL
    finally:
        lib.fp8k_tune_force_gemm_plan(-1, 0)
