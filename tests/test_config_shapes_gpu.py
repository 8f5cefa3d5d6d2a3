"""Every point of the benchmark configurations on the GPU, at its full size.

configs[2]: block-FP8 GEMM, M in {1, 16, 128, 1024, 4096} x the seven DeepSeek-V3 (N, K) pairs.
configs[3]: per-token fp8_scaled_mm, M in {1, 8, 64, 512, 2048, 8192} x the four Llama-3-8B (N, K) pairs, with bias.

At these sizes a float64 product of the whole problem would take minutes on the host, so the oracle is evaluated on a
sample of output rows and columns (first and last rows, tile edges, the first and last 130 columns, random ones);
every other element is covered by two properties that need no oracle: the output is finite everywhere, and doubling
one operand's scales doubles the result bit for bit (a power-of-two factor commutes with every rounding on the path),
which a kernel that skipped or repeated a K block, a tile or a row on part of the output would break against the
sampled oracle values of the first launch.

Tolerance: max|C - C_ref| / max|C_ref| <= 1e-2 against the float64 oracle (bf16 output, float32 accumulation).
"""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import fp8_tensor

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2

DSV3_NK = [(24576, 1536), (32768, 512), (7168, 16384), (4608, 7168), (7168, 2304), (18432, 7168), (7168, 18432)]
LLAMA_NK = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]


def _codes(rng, shape, top=0x68):
    """Random e4m3fn bytes of both signs, magnitudes below 2^(top/8 - 7) (no NaN codes)."""
    return rng.integers(0, top, shape, dtype=np.uint8) | (rng.integers(0, 2, shape, dtype=np.uint8) << 7)


def _rel_err(c, ref):
    return float(np.abs(c.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


def _elem_rel_err(c, ref):
    """Largest element-wise relative error over the elements that are not tiny (|ref| above 1 % of the largest): the strict
    reading of "maximum relative error"; for a bf16 output it is bounded below by the output rounding, 2^-8."""
    c, ref = c.astype(np.float64), ref.astype(np.float64)
    big = np.abs(ref) > 1e-2 * np.abs(ref).max()
    return float((np.abs(c - ref)[big] / np.abs(ref)[big]).max()) if big.any() else 0.0


def _sample(rng, M, N):
    rows = np.unique(np.concatenate([[0, M - 1, min(M - 1, 127), min(M - 1, 128), min(M - 1, 255), min(M - 1, 256)],
                                     rng.integers(0, M, 6)]))
    cols = np.unique(np.concatenate([np.arange(0, min(N, 130)), np.arange(max(0, N - 130), N), rng.integers(0, N, 300)]))
    return rows, cols


_weights = {}


def _weight(N, K):
    """One weight per (N, K), kept on the host and on the device while the cases of that shape run."""
    if (N, K) not in _weights:
        _weights.clear()
        rng = np.random.default_rng(N * 31 + K)
        wq = _codes(rng, (N, K))
        ws = (rng.uniform(0.5, 2.0, (N // 128, K // 128)) * 1e-3).astype(np.float32)
        _weights[(N, K)] = (wq, ws)
    return _weights[(N, K)]


@pytest.mark.parametrize("M", [1, 16, 128, 1024, 4096])
@pytest.mark.parametrize("N,K", DSV3_NK)
def test_block_gemm_deepseek_v3_every_config_point(dev, N, K, M):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    wq, ws = _weight(N, K)
    rng = np.random.default_rng(M * 7 + N + K)
    xq = _codes(rng, (M, K))
    xs = (rng.uniform(0.5, 2.0, (M, K // 128)) * 1e-2).astype(np.float32)
    A, B = fp8_tensor(xq, dev), fp8_tensor(wq, dev)
    As_row, Bs = torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev)
    As_col = As_row.t().contiguous().t()        # what the linear layer passes (column-major scales)
    C = w8a8_block_fp8_matmul(A, B, As_col, Bs, [128, 128], torch.bfloat16)
    torch.cuda.synchronize()
    assert C.shape == (M, N) and C.dtype == torch.bfloat16
    assert bool(torch.isfinite(C).all())

    rows, cols = _sample(rng, M, N)
    a = O.e4m3fn_to_f32(xq[rows]).astype(np.float64)
    b = O.e4m3fn_to_f32(wq[cols]).astype(np.float64)
    ws_cols = ws[cols // 128]
    ref = np.zeros((rows.size, cols.size))
    for kb in range(K // 128):
        sl = slice(kb * 128, (kb + 1) * 128)
        ref += (a[:, sl] @ b[:, sl].T) * xs[rows, kb][:, None] * ws_cols[:, kb][None, :]
    got = C[torch.from_numpy(rows).to(dev)][:, torch.from_numpy(cols).to(dev)].float().cpu().numpy()
    assert _rel_err(got, ref) <= REL_TOL, _rel_err(got, ref)
    assert _elem_rel_err(got, ref) <= REL_TOL, _elem_rel_err(got, ref)

    # row-major scales (the Triton-side layout) take the same kernels after a scale copy: same bits
    C_row = w8a8_block_fp8_matmul(A, B, As_row, Bs, [128, 128], torch.bfloat16)
    assert torch.equal(C_row, C)
    # power-of-two scale factors pass through every rounding unchanged, on the whole output
    C4 = w8a8_block_fp8_matmul(A, B, As_col * 0.5, Bs * 8.0, [128, 128], torch.bfloat16)
    assert torch.equal(C4, C * 4.0)


@pytest.mark.parametrize("M", [1, 8, 64, 512, 2048, 8192])
@pytest.mark.parametrize("N,K", LLAMA_NK)
def test_scaled_mm_llama3_every_config_point(dev, N, K, M):
    """Per-tensor weight scale broadcast to [N], per-token activation scale, bf16 bias (and the same bias as float32)."""
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    wq, _ = _weight(N, K)
    rng = np.random.default_rng(M * 11 + N + K)
    aq = _codes(rng, (M, K))
    sa = (rng.uniform(0.5, 2.0, M) * 1e-2).astype(np.float32)
    sb = np.full((N,), 3.1e-4, dtype=np.float32)
    bias = O.to_bf16(rng.standard_normal(N).astype(np.float32))
    A, B = fp8_tensor(aq, dev), fp8_tensor(wq, dev).t()
    tsa, tsb = torch.from_numpy(sa).to(dev), torch.from_numpy(sb).to(dev)
    tbias = torch.from_numpy(bias).to(dev).to(torch.bfloat16)
    C = fp8_scaled_mm(A, B, tsa, tsb, torch.bfloat16, tbias)
    C0 = fp8_scaled_mm(A, B, tsa, tsb, torch.bfloat16)
    torch.cuda.synchronize()
    assert C.shape == (M, N) and bool(torch.isfinite(C).all())

    rows, cols = _sample(rng, M, N)
    ti, tj = torch.from_numpy(rows).to(dev), torch.from_numpy(cols).to(dev)
    ref0 = O.fp8_scaled_mm(aq[rows], wq[cols], sa[rows], sb[cols], "f32")
    ref = O.fp8_scaled_mm(aq[rows], wq[cols], sa[rows], sb[cols], "f32", bias[cols])
    assert _rel_err(C0[ti][:, tj].float().cpu().numpy(), ref0) <= REL_TOL
    assert _rel_err(C[ti][:, tj].float().cpu().numpy(), ref) <= REL_TOL
    assert _elem_rel_err(C0[ti][:, tj].float().cpu().numpy(), ref0) <= REL_TOL
    # float32 bias of the same values: the same bits (the bias is added in float32 either way)
    assert torch.equal(fp8_scaled_mm(A, B, tsa, tsb, torch.bfloat16, tbias.float()), C)
    # power-of-two scale factors pass through exactly on the whole un-biased output
    assert torch.equal(fp8_scaled_mm(A, B, tsa * 4.0, tsb * 0.5, torch.bfloat16), C0 * 2.0)
