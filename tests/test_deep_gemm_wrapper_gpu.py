"""GPU parity of the DeepGEMM-shaped entry points (plain, contiguous grouped, masked grouped) against the oracle's
block matmul applied group by group.  Tolerance as for the other GEMMs: max relative error <= 1e-2 on bf16 output;
rows that the layout marks as skipped must stay untouched."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import fp8_tensor

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _codes(rng, shape):
    return rng.integers(0, 0x60, shape, dtype=np.uint8) | (rng.integers(0, 2, shape, dtype=np.uint8) << 7)


def _rel(c, ref):
    return float(np.abs(c.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


def test_gemm_nt_f8f8bf16(dev):
    from sglang_amd.deep_gemm_wrapper import gemm_nt_f8f8bf16

    rng = np.random.default_rng(1)
    M, N, K = 200, 512, 1024
    aq, bq = _codes(rng, (M, K)), _codes(rng, (N, K))
    a_s = rng.uniform(0.5, 2.0, (M, K // 128)).astype(np.float32) * 1e-2
    b_s = rng.uniform(0.5, 2.0, (N // 128, K // 128)).astype(np.float32) * 1e-2
    out = torch.empty((M, N), device=dev, dtype=torch.bfloat16)
    gemm_nt_f8f8bf16((fp8_tensor(aq, dev), torch.from_numpy(a_s).to(dev)), (fp8_tensor(bq, dev), torch.from_numpy(b_s).to(dev)), out)
    ref = O.w8a8_block_fp8_matmul(aq, bq, a_s, b_s, acc=np.float64)
    assert _rel(out.float().cpu().numpy(), ref) <= REL_TOL


@pytest.mark.parametrize("G,rows,N,K", [(4, [128, 0, 256, 128], 512, 512), (8, [128] * 8, 256, 1024), (3, [384, 128, 640], 384, 256)])
def test_grouped_contiguous(dev, G, rows, N, K):
    """Rows of each group contiguous and padded to 128 (DeepGEMM's alignment); the padding rows carry -1."""
    from sglang_amd.deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_contig

    rng = np.random.default_rng(G * 1000 + N)
    m_sum = sum(rows)
    m_indices = np.full((m_sum,), -1, dtype=np.int32)
    at = 0
    for g, r in enumerate(rows):
        real = r - (37 if r >= 128 else 0)  # the tail of every group's range is padding
        m_indices[at:at + real] = g
        at += r
    aq, bq = _codes(rng, (m_sum, K)), _codes(rng, (G, N, K))
    a_s = rng.uniform(0.5, 2.0, (m_sum, K // 128)).astype(np.float32) * 1e-2
    b_s = rng.uniform(0.5, 2.0, (G, N // 128, K // 128)).astype(np.float32) * 1e-2
    out = torch.full((m_sum, N), 7.0, device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_contig((fp8_tensor(aq, dev), torch.from_numpy(a_s).to(dev)),
                                    (fp8_tensor(bq, dev), torch.from_numpy(b_s).to(dev)), out, torch.from_numpy(m_indices).to(dev))
    got = out.float().cpu().numpy()
    for g in range(G):
        sel = np.nonzero(m_indices == g)[0]
        if sel.size:
            ref = O.w8a8_block_fp8_matmul(aq[sel], bq[g], a_s[sel], b_s[g], acc=np.float64)
            assert _rel(got[sel], ref) <= REL_TOL
    assert np.all(got[m_indices < 0] == 7.0)


@pytest.mark.parametrize("G,m_max,masked,N,K", [(4, 128, [0, 5, 128, 77], 256, 512), (6, 512, [300, 1, 512, 0, 129, 256], 512, 256)])
def test_grouped_masked(dev, G, m_max, masked, N, K):
    from sglang_amd.deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_masked

    rng = np.random.default_rng(G * 77 + m_max)
    aq, bq = _codes(rng, (G, m_max, K)), _codes(rng, (G, N, K))
    a_s = rng.uniform(0.5, 2.0, (G, m_max, K // 128)).astype(np.float32) * 1e-2
    b_s = rng.uniform(0.5, 2.0, (G, N // 128, K // 128)).astype(np.float32) * 1e-2
    out = torch.full((G, m_max, N), -3.0, device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_masked((fp8_tensor(aq, dev), torch.from_numpy(a_s).to(dev)),
                                    (fp8_tensor(bq, dev), torch.from_numpy(b_s).to(dev)), out,
                                    torch.tensor(masked, device=dev, dtype=torch.int32), max(sum(masked) // G, 1))
    got = out.float().cpu().numpy()
    for g in range(G):
        m = masked[g]
        if m:
            ref = O.w8a8_block_fp8_matmul(aq[g, :m], bq[g], a_s[g, :m], b_s[g], acc=np.float64)
            assert _rel(got[g, :m], ref) <= REL_TOL
        assert np.all(got[g, m:] == -3.0)


def test_wrapper_errors(dev):
    from sglang_amd.deep_gemm_wrapper import gemm_nt_f8f8bf16

    a = torch.zeros((8, 128), device=dev, dtype=torch.float8_e4m3fn)
    out = torch.empty((8, 8), device=dev, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="float32 or packed int32"):
        gemm_nt_f8f8bf16((a, torch.zeros((8, 1), device=dev, dtype=torch.float16)), (a, torch.ones((1, 1), device=dev)), out)
    with pytest.raises(RuntimeError, match="float8_e4m3fn"):
        gemm_nt_f8f8bf16((a.view(torch.uint8), torch.ones((8, 1), device=dev)), (a, torch.ones((1, 1), device=dev)), out)
    # packed activation scales are taken (exponent 127 = scale 1)
    s_packed = torch.full((8, 1), 127, device=dev, dtype=torch.int32)
    gemm_nt_f8f8bf16((a, s_packed), (a, torch.ones((1, 1), device=dev)), out)
    assert bool((out == 0).all())


def test_grouped_masked_with_packed_ue8m0_scales(dev):
    """Both scale tensors as packed UE8M0 words (activations per row, weights per weight row): the result is the
    oracle's on the powers of two they encode."""
    from sglang_amd.deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_masked

    rng = np.random.default_rng(9)
    G, m_max, N, K = 4, 96, 256, 640
    masked = np.array([96, 0, 40, 7], dtype=np.int32)
    aq, bq = _codes(rng, (G, m_max, K)), _codes(rng, (G, N, K))
    a_s = (2.0 ** rng.integers(-9, -4, (G, m_max, K // 128))).astype(np.float32)
    b_s = (2.0 ** rng.integers(-9, -4, (G, N // 128, K // 128))).astype(np.float32)
    a_p = torch.from_numpy(np.stack([O.pack_ue8m0_scales(x) for x in a_s])).to(dev)
    b_p = torch.from_numpy(np.stack([O.pack_ue8m0_scales(np.repeat(x, 128, axis=0)) for x in b_s])).to(dev)
    out = torch.full((G, m_max, N), 7.0, device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_masked((fp8_tensor(aq, dev), a_p), (fp8_tensor(bq, dev), b_p), out, torch.from_numpy(masked).to(dev), 40)
    got = out.float().cpu().numpy()
    for g in range(G):
        m = int(masked[g])
        if m:
            ref = O.w8a8_block_fp8_matmul(aq[g, :m], bq[g], a_s[g, :m], b_s[g], acc=np.float64)
            assert _rel(got[g, :m], ref) <= REL_TOL
        assert (got[g, m:] == 7.0).all()


@pytest.mark.parametrize("G,m_max,masked,N,K,expected_m", [
    (4, 320, [320, 0, 131, 257], 256, 640, 300),      # 256-row blocks, ragged tails, an empty group
    (2, 512, [512, 100], 384, 256, 512),              # two trips of K only; N not a multiple of 256
    (3, 200, [200, 199, 1], 128, 2048, 128),          # one 128-column tile, long K
])
def test_grouped_masked_packed_scales_on_the_hardware_scaled_kernel(dev, G, m_max, masked, N, K, expected_m):
    """Both scale tensors packed and enough rows per group for 256-row blocks: the matrix cores apply the exponents
    (fp8k_moe_block_gemm_ue8m0).  Oracle parity to the tolerance of the other GEMMs, untouched rows stay untouched,
    and the result agrees with the float-scale kernels on the same powers of two to bf16 rounding."""
    from sglang_amd.deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_masked
    from sglang_amd.fused_moe import get_default_config

    assert get_default_config(expected_m * G, G, 1)["BLOCK_SIZE_M"] == 256
    rng = np.random.default_rng(G * 1000 + K)
    masked = np.array(masked, dtype=np.int32)
    aq, bq = _codes(rng, (G, m_max, K)), _codes(rng, (G, N, K))
    a_s = (2.0 ** rng.integers(-12, 3, (G, m_max, K // 128))).astype(np.float32)
    b_s = (2.0 ** rng.integers(-12, 3, (G, N // 128, K // 128))).astype(np.float32)
    a_p = torch.from_numpy(np.stack([O.pack_ue8m0_scales(x) for x in a_s])).to(dev)
    b_p = torch.from_numpy(np.stack([O.pack_ue8m0_scales(np.repeat(x, 128, axis=0)) for x in b_s])).to(dev)
    A, B = fp8_tensor(aq, dev), fp8_tensor(bq, dev)
    mm = torch.from_numpy(masked).to(dev)
    out = torch.full((G, m_max, N), 7.0, device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_masked((A, a_p), (B, b_p), out, mm, expected_m)
    out_f = torch.full((G, m_max, N), 7.0, device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_masked((A, torch.from_numpy(a_s).to(dev)), (B, torch.from_numpy(b_s).to(dev)), out_f, mm, expected_m)
    got, got_f = out.float().cpu().numpy(), out_f.float().cpu().numpy()
    for g in range(G):
        m = int(masked[g])
        if m:
            ref = O.w8a8_block_fp8_matmul(aq[g, :m], bq[g], a_s[g, :m], b_s[g], acc=np.float64)
            assert _rel(got[g, :m], ref) <= REL_TOL
            assert _rel(got[g, :m], got_f[g, :m]) <= 2.0 ** -7
        assert (got[g, m:] == 7.0).all()


def test_grouped_contiguous_packed_scales_on_the_hardware_scaled_kernel(dev):
    """The contiguous layout with packed scales and 256-row blocks; rows marked -1 stay untouched."""
    from sglang_amd.deep_gemm_wrapper import grouped_gemm_nt_f8f8bf16_contig

    rng = np.random.default_rng(77)
    G, N, K = 3, 512, 1024
    rows = [384, 256, 640]
    real = [300, 256, 513]
    M = sum(rows)
    idx = np.full(M, -1, dtype=np.int32)
    start = 0
    for g in range(G):
        idx[start:start + real[g]] = g
        start += rows[g]
    aq, bq = _codes(rng, (M, K)), _codes(rng, (G, N, K))
    a_s = (2.0 ** rng.integers(-10, 0, (M, K // 128))).astype(np.float32)
    b_s = (2.0 ** rng.integers(-10, 0, (G, N // 128, K // 128))).astype(np.float32)
    a_p = torch.from_numpy(O.pack_ue8m0_scales(a_s)).to(dev)
    b_p = torch.from_numpy(np.stack([O.pack_ue8m0_scales(np.repeat(x, 128, axis=0)) for x in b_s])).to(dev)
    out = torch.full((M, N), 7.0, device=dev, dtype=torch.bfloat16)
    grouped_gemm_nt_f8f8bf16_contig((fp8_tensor(aq, dev), a_p), (fp8_tensor(bq, dev), b_p), out, torch.from_numpy(idx).to(dev))
    got = out.float().cpu().numpy()
    for g in range(G):
        sel = np.nonzero(idx == g)[0]
        ref = O.w8a8_block_fp8_matmul(aq[sel], bq[g], a_s[sel], b_s[g], acc=np.float64)
        assert _rel(got[sel], ref) <= REL_TOL
    assert (got[idx < 0] == 7.0).all()
