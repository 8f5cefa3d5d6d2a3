"""GPU parity of the fused-MoE stages against the CPU oracle.

Integer stage (moe_align_block_size): exact, compared through the invariants the reference's own test
uses (sgl-kernel/tests/test_moe_align.py:210-254) because the order inside an expert is unspecified.
Floating-point stages: silu within one bf16 ulp of the oracle's (hardware exp2 and reciprocal vs numpy exp),
moe_sum_reduce exact (same float32 summation order), grouped GEMM and the whole layer within the
path's 1e-2 max-relative-error bound.
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


def _random_ids(rng, T, E, topk, frac_minus1=0.0):
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    if frac_minus1:
        ids[rng.random(ids.shape) < frac_minus1] = -1
    return ids


def _check_align(ids, E, block, sorted_ids, expert_ids, npad):
    numel = ids.size
    flat = ids.reshape(-1)
    counts = np.bincount(flat + 1, minlength=E + 1)
    assert npad == sum((c + block - 1) // block * block for c in counts)
    ref_sorted, ref_experts, ref_npad = O.moe_align_block_size(ids, block, E)
    assert npad == ref_npad
    used = expert_ids[: npad // block]
    np.testing.assert_array_equal(used, ref_experts[: npad // block])
    for b in range(npad // block):
        blk = sorted_ids[b * block : (b + 1) * block]
        ref_blk = ref_sorted[b * block : (b + 1) * block]
        # same members, real slots first then padding
        nreal = int((ref_blk < numel).sum())
        assert (blk[nreal:] == numel).all()
        assert (blk[:nreal] < numel).all()
    # every slot appears exactly once; per-expert ranges hold exactly that expert's slots (as sets)
    real = sorted_ids[:npad][sorted_ids[:npad] < numel]
    np.testing.assert_array_equal(np.sort(real), np.arange(numel))
    start = 0
    for bkt in range(E + 1):
        c = counts[bkt]
        padded = (c + block - 1) // block * block
        seg = sorted_ids[start : start + padded]
        np.testing.assert_array_equal(np.sort(seg[:c]), np.nonzero(flat + 1 == bkt)[0])
        assert (seg[c:] == numel).all()
        start += padded


@pytest.mark.parametrize("T,E,topk,block", [(1, 256, 8, 32), (7, 8, 2, 16), (97, 64, 6, 64), (4096, 256, 8, 128),
                                           (333, 257, 8, 64), (9000, 256, 8, 64), (33, 16, 1, 128)])
@pytest.mark.parametrize("id_dtype", [torch.int32, torch.int64])
def test_moe_align_block_size(dev, T, E, topk, block, id_dtype):
    from sglang_amd.fused_moe import moe_align_block_size

    rng = np.random.default_rng(T + E)
    ids = _random_ids(rng, T, E, topk, 0.05 if T > 1 else 0.0)
    t_ids = torch.from_numpy(ids).to(dev).to(id_dtype)
    sorted_ids, expert_ids, npad = moe_align_block_size(t_ids, block, E)
    torch.cuda.synchronize()
    assert sorted_ids.numel() == ids.size + (E + 1) * (block - 1)
    assert expert_ids.numel() == (sorted_ids.numel() + block - 1) // block
    _check_align(ids, E, block, sorted_ids.cpu().numpy(), expert_ids.cpu().numpy(), int(npad.item()))


def test_moe_align_skewed_and_unpadded(dev):
    """All ids on one expert; pad_sorted_token_ids=False leaves the padding slots untouched."""
    from sglang_amd import sgl_kernel as ops

    E, block = 32, 64
    ids = np.full((500, 4), 5, dtype=np.int32)
    t_ids = torch.from_numpy(ids).to(dev)
    cap = ids.size + (E + 1) * (block - 1)
    sorted_ids = torch.full((cap,), -7, dtype=torch.int32, device=dev)
    expert_ids = torch.full(((cap + block - 1) // block,), -9, dtype=torch.int32, device=dev)
    npad = torch.zeros(1, dtype=torch.int32, device=dev)
    cumsum = torch.zeros(E + 2, dtype=torch.int32, device=dev)
    ops.moe_align_block_size(t_ids, E + 1, block, sorted_ids, expert_ids, npad, cumsum, False)
    torch.cuda.synchronize()
    n = int(npad.item())
    assert n == (2000 + block - 1) // block * block
    s = sorted_ids.cpu().numpy()
    np.testing.assert_array_equal(np.sort(s[:2000]), np.arange(2000))
    assert (s[2000:] == -7).all()
    e = expert_ids.cpu().numpy()
    assert (e[: n // block] == 5).all() and (e[n // block :] == -9).all()
    with pytest.raises(RuntimeError, match="sorted_token_ids holds"):
        ops.moe_align_block_size(t_ids, E + 1, block, sorted_ids[:100], expert_ids, npad, cumsum, True)


@pytest.mark.parametrize("rows,d", [(1, 2048), (37, 256), (32768, 2048)])
def test_silu_and_mul(dev, rows, d):
    from sglang_amd.sgl_kernel import silu_and_mul

    rng = np.random.default_rng(rows)
    x = O.to_bf16(rng.standard_normal((rows, 2 * d)).astype(np.float32) * 4)
    out = silu_and_mul(bf16_tensor(x, dev))
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    ref = O.silu_and_mul(x)
    # a silu value one bf16 ulp off (at most 2^-7 relative) carried through the product and its rounding
    tol = np.abs(ref) * 2.0**-6 + 1e-30
    assert (np.abs(got - ref) <= tol).all()
    # bf16 inputs take few distinct values: one whose silu lies within a float32 ulp of a bf16 tie (5.9375 ->
    # 5.92187444, tie 5.921875) repeats a dozen times in the small case
    assert (got != ref).mean() < 2e-3
    # the library routine on the same device agrees with the same bound
    xt = bf16_tensor(x, dev)
    lib_ref = (torch.nn.functional.silu(xt[:, :d].float()).to(torch.bfloat16) * xt[:, d:]).float().cpu().numpy()
    assert (np.abs(got - lib_ref) <= np.abs(lib_ref) * 2.0**-6 + 1e-30).all()


def test_silu_and_mul_other_dtypes_and_errors(dev):
    from sglang_amd.sgl_kernel import silu_and_mul

    x = torch.randn(9, 64, device=dev)
    ref = torch.nn.functional.silu(x[:, :32]) * x[:, 32:]
    torch.testing.assert_close(silu_and_mul(x), ref, rtol=1e-5, atol=1e-6)
    xh = x.half()
    refh = torch.nn.functional.silu(xh[:, :32].float()).half() * xh[:, 32:]
    torch.testing.assert_close(silu_and_mul(xh), refh, rtol=2e-3, atol=1e-6)
    # the ends of the range: exp(-v) over- and underflows, infinities and NaN behave as v / (1 + exp(-v)) does
    edge = torch.tensor([0.0, -0.0, 1e-30, -1e-30, 20.0, -20.0, 80.0, -80.0, 88.0, -88.0, 90.0, -90.0, 104.0, -104.0, 1e4, -1e4,
                         3e38, -3e38, float("inf"), float("-inf"), float("nan"), 1.0, -1.0, 0.5, -0.5, 7.0, -7.0, 15.0, -15.0,
                         30.0, -30.0, 60.0, -60.0], device=dev)
    xe = torch.cat([edge, torch.ones_like(edge)]).reshape(1, -1)
    xe = torch.cat([xe[:, :edge.numel()], torch.zeros(1, (-edge.numel()) % 8, device=dev), xe[:, edge.numel():],
                    torch.zeros(1, (-edge.numel()) % 8, device=dev)], dim=1)
    got = silu_and_mul(xe)[0, :edge.numel()]
    want = edge / (1.0 + torch.exp(-edge))
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-37, equal_nan=True)
    with pytest.raises(ValueError, match="multiple of 16 bytes"):
        silu_and_mul(torch.zeros(3, 12, device=dev, dtype=torch.bfloat16))
    assert silu_and_mul(torch.zeros(0, 64, device=dev, dtype=torch.bfloat16)).shape == (0, 32)


@pytest.mark.parametrize("rows,d", [(1, 2048), (37, 256), (32768, 2048)])
def test_gelu_and_mul(dev, rows, d):
    """gelu_and_mul (erf form) against the oracle and against the library routine on the device.  The device erf and a
    correctly rounded one differ by a few float32 ulp: that can move a result across a bf16 tie (one bf16 ulp, carried
    through the product: 2^-6 relative), and for gates below -3 it is magnified by the cancellation in 1 + erf - an
    absolute error of a few 2^-24 in a sum of 1e-3 and less, |gate up| 2^-20 in the result."""
    from sglang_amd.sgl_kernel import gelu_and_mul

    rng = np.random.default_rng(rows)
    x = O.to_bf16(rng.standard_normal((rows, 2 * d)).astype(np.float32) * 3)
    out = gelu_and_mul(bf16_tensor(x, dev))
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    ref = O.gelu_and_mul(x)
    gate, up = x[:, :d], x[:, d:]
    tol = np.abs(ref) * 2.0**-6 + np.abs(gate * up) * 2.0**-20 + 1e-30
    assert (np.abs(got - ref) <= tol).all()
    assert (got != ref)[gate > -3].mean() < 2e-3
    xt = bf16_tensor(x, dev)
    lib_ref = (torch.nn.functional.gelu(xt[:, :d].float()).to(torch.bfloat16) * xt[:, d:]).float().cpu().numpy()
    assert (np.abs(got - lib_ref) <= np.abs(lib_ref) * 2.0**-6 + np.abs(gate * up) * 2.0**-20 + 1e-30).all()
    # not the other activations
    assert not np.allclose(got, O.silu_and_mul(x), rtol=2e-2)


def test_gelu_and_mul_other_dtypes_and_errors(dev):
    from sglang_amd.sgl_kernel import gelu_and_mul

    x = torch.randn(9, 64, device=dev)
    ref = torch.nn.functional.gelu(x[:, :32]) * x[:, 32:]
    torch.testing.assert_close(gelu_and_mul(x), ref, rtol=1e-5, atol=1e-6)
    xh = x.half()
    refh = torch.nn.functional.gelu(xh[:, :32].float()).half() * xh[:, 32:]
    torch.testing.assert_close(gelu_and_mul(xh), refh, rtol=2e-3, atol=1e-6)
    out = torch.empty(9, 32, device=dev)
    assert gelu_and_mul(x, out) is out
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-6)
    # the ends of the range: v for large v (no overflow in v * (0.5 * (1 + erf))), -0 for large negative v, NaN kept
    edge = torch.tensor([0.0, -0.0, 1e-30, -1e-30, 6.0, -6.0, 20.0, -20.0, 1e4, -1e4, 3e38, -3e38, float("inf"), float("nan"),
                         1.0, -1.0], device=dev)
    xe = torch.cat([edge, torch.ones_like(edge)]).reshape(1, -1)
    got = gelu_and_mul(xe)[0]
    want = torch.tensor([0.0, -0.0, 5e-31, -5e-31, 6.0, -0.0, 20.0, -0.0, 1e4, -0.0, 3e38, -0.0, float("inf"), float("nan"),
                         0.8413447, -0.1586553], device=dev)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-8, equal_nan=True)
    with pytest.raises(ValueError, match="multiple of 16 bytes"):
        gelu_and_mul(torch.zeros(3, 12, device=dev, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="dtype of input"):
        gelu_and_mul(torch.zeros(3, 16, device=dev, dtype=torch.bfloat16), torch.zeros(3, 8, device=dev))
    assert gelu_and_mul(torch.zeros(0, 64, device=dev, dtype=torch.bfloat16)).shape == (0, 32)


@pytest.mark.parametrize("kind", ["silu", "gelu", "relu2"])
def test_activation_without_gate(dev, kind):
    """The activation of ungated experts against the oracle (bounds as for the gated kernels: one bf16 ulp where a
    float32 result sits on a tie, and for gelu the cancellation in 1 + erf below -3) and against the tensor library's
    op on the device; relu2 is exact."""
    from sglang_amd.sgl_kernel import activation

    rng = np.random.default_rng(len(kind))
    x = O.to_bf16(rng.standard_normal((300, 512)).astype(np.float32) * 3)
    xt = bf16_tensor(x, dev)
    out = activation(xt, kind)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    ref = O.activation_only(x, kind)
    lib_ref = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu,
               "relu2": lambda t: torch.square(torch.relu(t))}[kind](xt).float().cpu().numpy()
    if kind == "relu2":
        assert np.array_equal(got, ref) and np.array_equal(got, lib_ref)
    else:
        tol = np.abs(ref) * 2.0**-7 + (np.abs(x) * 2.0**-20 if kind == "gelu" else 0) + 1e-30
        assert (np.abs(got - ref) <= tol).all() and (np.abs(got - lib_ref) <= tol).all()
        assert (got != ref)[x > -3].mean() < 2e-3
    # float32 and float16, an output tensor, the edges, the errors
    xf = torch.randn(9, 64, device=dev)
    want = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu2": lambda t: torch.square(torch.relu(t))}[kind]
    torch.testing.assert_close(activation(xf, kind), want(xf), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(activation(xf.half(), kind), want(xf.half().float()).half(), rtol=2e-3, atol=1e-6)
    o = torch.empty_like(xf)
    assert activation(xf, kind, o) is o
    edge = torch.tensor([0.0, -0.0, 1e-30, -1e-30, 30.0, -30.0, 3e38, -3e38, float("inf"), float("-inf"), float("nan"), 1.0,
                         -1.0, 0.5, -0.5, 100.0], device=dev).reshape(1, -1)
    e = activation(edge, kind)[0]
    if kind == "relu2":
        torch.testing.assert_close(e, torch.square(torch.relu(edge[0])), rtol=0, atol=0, equal_nan=True)
    elif kind == "silu":
        torch.testing.assert_close(e, edge[0] / (1.0 + torch.exp(-edge[0])), rtol=1e-5, atol=1e-37, equal_nan=True)
    else:
        assert e[4] == 30.0 and e[5] == 0.0 and e[6] == 3e38 and e[7] == 0.0 and e[8] == float("inf") and torch.isnan(e[10])
        torch.testing.assert_close(e[11:15], torch.tensor([0.8413447, -0.1586553, 0.3457312, -0.1542688], device=dev), rtol=1e-5, atol=1e-8)
    with pytest.raises(ValueError, match="Unsupported activation"):
        activation(xf, "tanh")
    with pytest.raises(ValueError, match="multiple of 16 bytes"):
        activation(torch.zeros(3, 12, device=dev, dtype=torch.bfloat16), kind)
    with pytest.raises(RuntimeError, match="shape and dtype"):
        activation(xf, kind, torch.empty(9, 32, device=dev))
    assert activation(torch.zeros(0, 64, device=dev, dtype=torch.bfloat16), kind).shape == (0, 64)


@pytest.mark.parametrize("T,topk,H,scale", [(1, 8, 7168, 2.5), (19, 8, 128, 1.0), (4096, 8, 7168, 2.5), (5, 1, 64, 0.5)])
def test_moe_sum_reduce_exact(dev, T, topk, H, scale):
    from sglang_amd.sgl_kernel import moe_sum_reduce

    rng = np.random.default_rng(T)
    x = O.to_bf16(rng.standard_normal((T, topk, H)).astype(np.float32))
    out = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    moe_sum_reduce(bf16_tensor(x, dev), out, scale)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.float().cpu().numpy(), O.moe_sum_reduce(x, scale))


@pytest.mark.parametrize("topk", [1, 2, 3, 4, 8])
def test_moe_sum_exact(dev, topk):
    from sglang_amd.sgl_kernel import moe_sum

    rng = np.random.default_rng(topk)
    x = O.to_bf16(rng.standard_normal((37, topk, 256)).astype(np.float32) * 3)
    out = torch.empty((37, 256), dtype=torch.bfloat16, device=dev)
    moe_sum(bf16_tensor(x, dev), out)
    np.testing.assert_array_equal(out.float().cpu().numpy(), O.moe_sum(x))


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_grouped_gemm_hardware_scaled_is_exact_on_integer_data(dev, seed):
    """fp8k_moe_block_gemm_ue8m0 (256-slot blocks, sorted power-of-two scales): on small integers with power-of-two
    scales every product and sum is exact, so the matrix cores' own scaling must give the oracle's bf16 values bit
    for bit, and so must the float-scale kernel."""
    from sglang_amd.fused_moe import moe_align_block_size
    from sglang_amd.sgl_kernel import moe_block_gemm, moe_sort_scales

    rng = np.random.default_rng(seed)
    T, E, topk = int(rng.integers(200, 900)), int(rng.integers(2, 9)), 2
    N, K = int(rng.integers(1, 6)) * 128, int(rng.integers(2, 7)) * 128
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    ids[rng.random(ids.shape) < 0.05] = -1
    wq = O.f32_to_e4m3fn(rng.integers(-4, 5, (E, N, K)).astype(np.float32))
    ws = (2.0 ** rng.integers(-3, 3, (E, N // 128, K // 128))).astype(np.float32)
    xq = O.f32_to_e4m3fn(rng.integers(-4, 5, (T, K)).astype(np.float32))
    xs = (2.0 ** rng.integers(-3, 3, (T, K // 128))).astype(np.float32)
    sorted_ids, expert_ids, npad = moe_align_block_size(torch.from_numpy(ids).to(dev), 256, E)
    A, B = fp8_tensor(xq, dev), fp8_tensor(wq, dev)
    As, Bs = torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev)
    sc = moe_sort_scales(As, sorted_ids, npad, topk, ids.size)
    tw = torch.ones((T, topk), device=dev)
    flat = ids.reshape(-1)
    for pow2 in (False, True):
        C = torch.full((T * topk, N), float("nan"), dtype=torch.bfloat16, device=dev)
        moe_block_gemm(A, B, C, sc, Bs, tw, sorted_ids, expert_ids, npad, False, topk, 256, ids.size, scales_sorted=True,
                       pow2_scales=pow2)
        got = C.float().cpu().numpy()
        assert (got[flat == -1] == 0).all()
        for e in range(E):
            slots = np.nonzero(flat == e)[0]
            if slots.size:
                ref = O.w8a8_block_fp8_matmul(xq[slots // topk], wq[e], xs[slots // topk], ws[e], acc=np.float64)
                np.testing.assert_array_equal(got[slots], ref)


def _expert_weights(rng, E, N, K):
    wq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((E, N, K)).astype(np.float32) * 100, -448, 448))
    ws = (rng.uniform(0.5, 2.0, (E, (N + 127) // 128, K // 128)) * 1e-3).astype(np.float32)
    return wq, ws


@pytest.mark.parametrize("T,E,topk,N,K,block", [(5, 8, 2, 512, 256, 16), (64, 8, 2, 384, 512, 32), (300, 16, 4, 1024, 1024, 64),
                                               (700, 4, 2, 256, 384, 128), (3, 16, 8, 1024, 7168, 32),
                                               (700, 4, 2, 512, 384, 256), (300, 16, 4, 1024, 1024, 256)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_grouped_gemm_vs_oracle(dev, T, E, topk, N, K, block, out_dtype):
    """GEMM1 form (row = slot // top_k, no routed weight) and GEMM2 form (row = slot, times routed weight)."""
    from sglang_amd.fused_moe import moe_align_block_size
    from sglang_amd.sgl_kernel import moe_block_gemm, moe_sort_scales

    rng = np.random.default_rng(T * 7 + N)
    ids = _random_ids(rng, T, E, topk, 0.1 if T > 5 else 0.0)
    wq, ws = _expert_weights(rng, E, N, K)
    t_ids = torch.from_numpy(ids).to(dev)
    sorted_ids, expert_ids, npad = moe_align_block_size(t_ids, block, E)
    tw = rng.uniform(0.1, 1.0, (T, topk)).astype(np.float32)
    Bq, Bs = fp8_tensor(wq, dev), torch.from_numpy(ws).to(dev)
    for top_k, rows in ((topk, T), (1, T * topk)):
        xq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((rows, K)).astype(np.float32) * 100, -448, 448))
        xs = (rng.uniform(0.5, 2.0, (rows, K // 128)) * 1e-2).astype(np.float32)
        C = torch.full((T * topk, N), float("nan"), dtype=out_dtype, device=dev)
        mul = top_k == 1
        moe_block_gemm(fp8_tensor(xq, dev), Bq, C, torch.from_numpy(xs).to(dev), Bs, torch.from_numpy(tw).to(dev),
                       sorted_ids, expert_ids, npad, mul, top_k, block, ids.size)
        torch.cuda.synchronize()
        got = C.float().cpu().numpy()
        assert np.isfinite(got).all(), "some output row was not written"
        ref = np.zeros((T * topk, N), dtype=np.float64)
        flat = ids.reshape(-1)
        for e in range(E):
            slots = np.nonzero(flat == e)[0]
            if slots.size == 0:
                continue
            r = slots // top_k
            part = O.w8a8_block_fp8_matmul(xq[r], wq[e], xs[r], ws[e], out_dtype="f32", acc=np.float64)
            ref[slots] = part * (tw.reshape(-1)[slots][:, None] if mul else 1.0)
        assert (got[flat == -1] == 0).all()
        assert _rel_err(got, ref) <= REL_TOL
        if block >= 64:
            # scales gathered into sorted-slot order first: same arithmetic, so the same bits
            for xs_dev in (torch.from_numpy(xs).to(dev), torch.from_numpy(np.ascontiguousarray(xs.T)).to(dev).t()):
                srt = moe_sort_scales(xs_dev, sorted_ids, npad, top_k, ids.size)
                n_used = int(npad.item())
                sid = sorted_ids.cpu().numpy()[:n_used]
                live = sid < ids.size
                assert srt.shape == (sorted_ids.numel(), K // 128)
                np.testing.assert_array_equal(srt.cpu().numpy()[:n_used][live], xs[sid[live] // top_k])
                C2 = torch.full((T * topk, N), float("nan"), dtype=out_dtype, device=dev)
                moe_block_gemm(fp8_tensor(xq, dev), Bq, C2, srt, Bs, torch.from_numpy(tw).to(dev),
                               sorted_ids, expert_ids, npad, mul, top_k, block, ids.size, scales_sorted=True)
                torch.cuda.synchronize()
                assert torch.equal(C2, C)


def test_grouped_gemm_256_slot_blocks_every_group_count(dev):
    """Experts whose last 256-slot block holds 1..8 groups of 32 slots (the kernel skips the padding groups)."""
    from sglang_amd.fused_moe import moe_align_block_size
    from sglang_amd.sgl_kernel import moe_block_gemm

    rng = np.random.default_rng(11)
    counts = [1, 32, 33, 65, 97, 128, 129, 161, 193, 225, 256, 257, 0, 300]
    E, N, K, block = len(counts), 512, 384, 256
    ids = rng.permutation(np.repeat(np.arange(E, dtype=np.int32), counts))[:, None]
    T = ids.shape[0]
    wq, ws = _expert_weights(rng, E, N, K)
    xq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((T, K)).astype(np.float32) * 100, -448, 448))
    xs = (rng.uniform(0.5, 2.0, (T, K // 128)) * 1e-2).astype(np.float32)
    sorted_ids, expert_ids, npad = moe_align_block_size(torch.from_numpy(ids).to(dev), block, E)
    C = torch.full((T, N), float("nan"), dtype=torch.bfloat16, device=dev)
    moe_block_gemm(fp8_tensor(xq, dev), fp8_tensor(wq, dev), C, torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev),
                   torch.ones((T, 1), device=dev), sorted_ids, expert_ids, npad, False, 1, block, T)
    torch.cuda.synchronize()
    got = C.float().cpu().numpy()
    assert np.isfinite(got).all(), "some output row was not written"
    for e in range(E):
        rows = np.nonzero(ids[:, 0] == e)[0]
        if rows.size:
            ref = O.w8a8_block_fp8_matmul(xq[rows], wq[e], xs[rows], ws[e], out_dtype="f32", acc=np.float64)
            assert _rel_err(got[rows], ref) <= REL_TOL, "expert %d with %d slots" % (e, rows.size)
    # the same through the form with scales in sorted-slot order (its K loop is the software-pipelined one, one copy per
    # group count), at one, two and three K blocks: the same arithmetic in the same order, so the same bits
    from sglang_amd.sgl_kernel import moe_sort_scales

    for kb in (3, 2, 1):
        Kc = kb * 128
        A = fp8_tensor(np.ascontiguousarray(xq[:, :Kc]), dev)
        B = fp8_tensor(np.ascontiguousarray(wq[:, :, :Kc]), dev)
        As = torch.from_numpy(np.ascontiguousarray(xs[:, :kb])).to(dev)
        Bs = torch.from_numpy(np.ascontiguousarray(ws[:, :, :kb])).to(dev)
        outs = []
        for sort in (False, True):
            Ck = torch.full((T, N), float("nan"), dtype=torch.bfloat16, device=dev)
            sc = moe_sort_scales(As, sorted_ids, npad, 1, T) if sort else As
            moe_block_gemm(A, B, Ck, sc, Bs, torch.ones((T, 1), device=dev), sorted_ids, expert_ids, npad, False, 1, block, T,
                           scales_sorted=sort)
            torch.cuda.synchronize()
            outs.append(Ck)
        assert torch.equal(outs[0], outs[1]), "K = %d" % Kc
        if kb == 3:
            assert torch.equal(outs[0], C)


def test_grouped_gemm_random_routings_exact(dev):
    """Forty seeded random routings (1..600 tokens, 2..40 experts, top-1..6, every block size, skewed and absent
    experts, ids of -1) on integer data with power-of-two scales: exact, with per-token and with sorted scales."""
    from sglang_amd.fused_moe import moe_align_block_size
    from sglang_amd.sgl_kernel import moe_block_gemm, moe_sort_scales

    rng = np.random.default_rng(20250102)
    for case in range(40):
        T = int(rng.choice([rng.integers(1, 8), rng.integers(8, 100), rng.integers(100, 600)]))
        E = int(rng.integers(2, 41))
        topk = int(rng.integers(1, min(6, E) + 1))
        block = int(rng.choice([16, 32, 64, 128, 256]))
        N, K = int(rng.integers(1, 9)) * 128, int(rng.integers(1, 7)) * 128
        p = rng.dirichlet(np.full(E, 0.5))  # skewed: some experts get nothing
        ids = np.stack([rng.choice(E, size=topk, replace=False, p=p / p.sum()) if (p > 0).sum() >= topk
                        else rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
        ids[rng.random(ids.shape) < 0.05] = -1
        wq = O.f32_to_e4m3fn(rng.integers(-4, 5, (E, N, K)).astype(np.float32))
        ws = (2.0 ** rng.integers(-3, 3, (E, N // 128, K // 128))).astype(np.float32)
        xq = O.f32_to_e4m3fn(rng.integers(-4, 5, (T, K)).astype(np.float32))
        xs = (2.0 ** rng.integers(-3, 3, (T, K // 128))).astype(np.float32)
        sorted_ids, expert_ids, npad = moe_align_block_size(torch.from_numpy(ids).to(dev), block, E)
        A, B = fp8_tensor(xq, dev), fp8_tensor(wq, dev)
        As, Bs = torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev)
        tw = torch.ones((T, topk), device=dev)
        outs = []
        for sort in ([False, True] if block >= 64 else [False]):
            C = torch.full((T * topk, N), float("nan"), dtype=torch.bfloat16, device=dev)
            sc = moe_sort_scales(As, sorted_ids, npad, topk, ids.size) if sort else As
            moe_block_gemm(A, B, C, sc, Bs, tw, sorted_ids, expert_ids, npad, False, topk, block, ids.size, scales_sorted=sort)
            torch.cuda.synchronize()
            outs.append(C.float().cpu().numpy())
        flat = ids.reshape(-1)
        for got in outs:
            for e in range(E):
                slots = np.nonzero(flat == e)[0]
                if slots.size:
                    ref = O.w8a8_block_fp8_matmul(xq[slots // topk], wq[e], xs[slots // topk], ws[e], out_dtype="bf16", acc=np.float64)
                    assert np.array_equal(got[slots], ref), "case %d: T=%d E=%d topk=%d block=%d N=%d K=%d expert %d" % (
                        case, T, E, topk, block, N, K, e)
            assert (got[flat == -1] == 0).all(), "case %d: rows of dropped slots must be zero" % case


def test_grouped_gemm_exact_on_integers(dev):
    from sglang_amd.fused_moe import moe_align_block_size
    from sglang_amd.sgl_kernel import moe_block_gemm

    rng = np.random.default_rng(3)
    T, E, topk, N, K, block = 90, 6, 3, 512, 512, 64
    ids = _random_ids(rng, T, E, topk)
    wq = O.f32_to_e4m3fn(rng.integers(-4, 5, (E, N, K)).astype(np.float32))
    ws = (2.0 ** rng.integers(-3, 3, (E, N // 128, K // 128))).astype(np.float32)
    xq = O.f32_to_e4m3fn(rng.integers(-4, 5, (T, K)).astype(np.float32))
    xs = (2.0 ** rng.integers(-3, 3, (T, K // 128))).astype(np.float32)
    sorted_ids, expert_ids, npad = moe_align_block_size(torch.from_numpy(ids).to(dev), block, E)
    C = torch.empty((T * topk, N), dtype=torch.bfloat16, device=dev)
    moe_block_gemm(fp8_tensor(xq, dev), fp8_tensor(wq, dev), C, torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev),
                   torch.ones((T, topk), device=dev), sorted_ids, expert_ids, npad, False, topk, block, ids.size)
    torch.cuda.synchronize()
    got = C.float().cpu().numpy()
    flat = ids.reshape(-1)
    for e in range(E):
        slots = np.nonzero(flat == e)[0]
        ref = O.w8a8_block_fp8_matmul(xq[slots // topk], wq[e], xs[slots // topk], ws[e], out_dtype="bf16", acc=np.float64)
        np.testing.assert_array_equal(got[slots], ref)


def _moe_problem(rng, T, E, H, I, topk, grouped_routing):
    x = O.make_activation(T, H, int(rng.integers(1 << 30)))
    w13 = O.to_bf16(rng.standard_normal((E, 2 * I, H)).astype(np.float32) * 0.02)
    w2 = O.to_bf16(rng.standard_normal((E, H, I)).astype(np.float32) * 0.02)
    w13q = np.empty((E, 2 * I, H), np.uint8); w13s = np.empty((E, 2 * I // 128, H // 128), np.float32)
    w2q = np.empty((E, H, I), np.uint8); w2s = np.empty((E, H // 128, I // 128), np.float32)
    for e in range(E):
        w13q[e], w13s[e] = O.block_quant_weight(w13[e])
        w2q[e], w2s[e] = O.block_quant_weight(w2[e])
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if grouped_routing:
        bias = (rng.standard_normal(E) * 0.1).astype(np.float32)
        tw, ids = O.biased_grouped_topk(logits, bias, 8, 4, topk)
    else:
        ids = np.argsort(-logits, axis=1)[:, :topk].astype(np.int32)
        sc = 1 / (1 + np.exp(-np.take_along_axis(logits, ids, 1)))
        tw = (sc / sc.sum(-1, keepdims=True)).astype(np.float32)
    return x, w13q, w13s, w2q, w2s, tw, ids


@pytest.mark.parametrize("T,E,H,I,topk,grouped", [(1, 8, 512, 256, 2, False), (40, 8, 512, 256, 2, False),
                                                 (300, 32, 1024, 512, 8, True), (1000, 8, 256, 128, 4, False)])
def test_fused_experts_vs_oracle(dev, T, E, H, I, topk, grouped):
    from sglang_amd.fused_moe import fused_experts_impl

    rng = np.random.default_rng(T + E)
    x, w13q, w13s, w2q, w2s, tw, ids = _moe_problem(rng, T, E, H, I, topk, grouped)
    rsf = 2.5
    ref = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, rsf)
    out = fused_experts_impl(
        bf16_tensor(x, dev), fp8_tensor(w13q, dev), fp8_tensor(w2q, dev), torch.from_numpy(tw).to(dev),
        torch.from_numpy(ids).to(dev), use_fp8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev),
        w2_scale=torch.from_numpy(w2s).to(dev), block_shape=[128, 128], routed_scaling_factor=rsf,
    )
    torch.cuda.synchronize()
    assert out.shape == (T, H) and out.dtype == torch.bfloat16
    got = out.float().cpu().numpy()
    assert _rel_err(got, ref) <= REL_TOL
    # the reference's own acceptance metric for this layer (python/sglang/test/test_block_fp8.py:519-523)
    assert np.abs(got - ref).mean() / np.abs(ref).mean() < 0.02


@pytest.mark.parametrize("T,E,H,I", [(40, 8, 512, 256), (1100, 4, 256, 128)])
def test_fused_experts_router_weight_on_input(dev, T, E, H, I):
    """apply_router_weight_on_input (one expert per token, as the reference requires): the routed weight multiplies
    the result of GEMM 1; 1100 tokens on 4 experts take 256-slot blocks, where the default form would fuse GEMM 1's
    write-out and this one keeps the three steps."""
    from sglang_amd.fused_moe import fused_experts_impl

    rng = np.random.default_rng(T)
    x, w13q, w13s, w2q, w2s, tw, ids = _moe_problem(rng, T, E, H, I, 1, False)
    tw = rng.uniform(0.2, 1.0, tw.shape).astype(np.float32)
    ref = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, 1.0, apply_router_weight_on_input=True)
    out = fused_experts_impl(
        bf16_tensor(x, dev), fp8_tensor(w13q, dev), fp8_tensor(w2q, dev), torch.from_numpy(tw).to(dev),
        torch.from_numpy(ids).to(dev), use_fp8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev),
        w2_scale=torch.from_numpy(w2s).to(dev), block_shape=[128, 128], apply_router_weight_on_input=True,
    )
    torch.cuda.synchronize()
    assert _rel_err(out.float().cpu().numpy(), ref) <= REL_TOL


@pytest.mark.parametrize("T,E,H,I,topk", [(40, 8, 512, 256, 2), (1100, 4, 256, 128, 2), (300, 32, 1024, 512, 8)])
def test_fused_experts_gelu_and_ignored_activation_scales(dev, T, E, H, I, topk):
    """activation="gelu" (fused_moe.py:561-565 of the reference) at block sizes 16, 256 (where silu would take the fused
    write-out of GEMM 1) and 32; a1_scale / a2_scale change nothing on the block-quantised path, as in the reference
    (fused_moe_triton_kernels.py:619-637 replaces the scale it is handed by the per-token-group one)."""
    from sglang_amd.fused_moe import fused_experts_impl

    rng = np.random.default_rng(T + E)
    x, w13q, w13s, w2q, w2s, tw, ids = _moe_problem(rng, T, E, H, I, topk, False)
    ref = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, 2.5, activation="gelu")
    args = (bf16_tensor(x, dev), fp8_tensor(w13q, dev), fp8_tensor(w2q, dev), torch.from_numpy(tw).to(dev),
            torch.from_numpy(ids).to(dev))
    kw = dict(use_fp8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
              block_shape=[128, 128], routed_scaling_factor=2.5)
    out = fused_experts_impl(*args, activation="gelu", **kw)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert _rel_err(got, ref) <= REL_TOL
    assert np.abs(got - ref).mean() / np.abs(ref).mean() < 0.02
    silu = fused_experts_impl(*args, **kw)
    assert _rel_err(silu.float().cpu().numpy(), ref) > 3 * REL_TOL      # the two activations are told apart
    one = torch.full((1,), 0.37, device=dev)
    assert torch.equal(fused_experts_impl(*args, activation="gelu", a1_scale=one, a2_scale=one, **kw), out)
    assert torch.equal(fused_experts_impl(*args, a1_scale=one, a2_scale=one, **kw), silu)
    with pytest.raises(AssertionError, match="gemm1_alpha is not supported for gelu"):
        fused_experts_impl(*args, activation="gelu", gemm1_alpha=1.7, gemm1_limit=7.0, **kw)
    with pytest.raises(RuntimeError, match="alpha and limit"):
        fused_experts_impl(*args, gemm1_alpha=1.7, gemm1_limit=7.0, **kw)
    with pytest.raises(ValueError, match="Unsupported activation"):
        fused_experts_impl(*args, activation="relu2", is_gated=True, **kw)
    with pytest.raises(ValueError, match="Unsupported activation"):
        fused_experts_impl(*args, activation="swish", **kw)


@pytest.mark.parametrize("T,E,H,I,topk", [(40, 8, 512, 256, 2), (1100, 4, 256, 128, 2)])
@pytest.mark.parametrize("kind", ["silu", "gelu", "relu2"])
def test_fused_experts_without_gate(dev, T, E, H, I, topk, kind):
    """is_gated=False (fused_moe.py:566-572 of the reference): w1 is [E, I, H], the activation keeps the width; block
    sizes 16 and 256 (where the gated silu form would take the fused write-out of GEMM 1)."""
    from sglang_amd.fused_moe import fused_experts_impl

    rng = np.random.default_rng(T + E)
    x, w13q, w13s, w2q, w2s, tw, ids = _moe_problem(rng, T, E, H, I, topk, False)
    w1q, w1s = w13q[:, :I].copy(), w13s[:, : I // 128].copy()          # an [E, I, H] projection
    ref = O.fused_moe_block_fp8(x, w1q, w1s, w2q, w2s, tw, ids, 1.5, activation=kind, is_gated=False)
    out = fused_experts_impl(
        bf16_tensor(x, dev), fp8_tensor(w1q, dev), fp8_tensor(w2q, dev), torch.from_numpy(tw).to(dev),
        torch.from_numpy(ids).to(dev), use_fp8_w8a8=True, w1_scale=torch.from_numpy(w1s).to(dev),
        w2_scale=torch.from_numpy(w2s).to(dev), block_shape=[128, 128], routed_scaling_factor=1.5, activation=kind,
        is_gated=False,
    )
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert out.shape == (T, H)
    assert _rel_err(got, ref) <= REL_TOL
    assert np.abs(got - ref).mean() / np.abs(ref).mean() < 0.02
    others = [k for k in ("silu", "gelu", "relu2") if k != kind]
    for k in others:
        assert _rel_err(got, O.fused_moe_block_fp8(x, w1q, w1s, w2q, w2s, tw, ids, 1.5, activation=k, is_gated=False)) > 2 * REL_TOL


def test_fused_experts_with_absent_experts_and_no_combine(dev):
    """ids == -1 (expert on another rank) contribute zero; no_combine returns the per-slot rows."""
    from sglang_amd.fused_moe import fused_experts_impl

    rng = np.random.default_rng(5)
    T, E, H, I, topk = 50, 8, 256, 128, 2
    x, w13q, w13s, w2q, w2s, tw, ids = _moe_problem(rng, T, E, H, I, topk, False)
    ids[rng.random(ids.shape) < 0.3] = -1
    ref = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, 1.0)
    args = (bf16_tensor(x, dev), fp8_tensor(w13q, dev), fp8_tensor(w2q, dev), torch.from_numpy(tw).to(dev),
            torch.from_numpy(ids).to(dev))
    kw = dict(use_fp8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
              block_shape=[128, 128])
    out = fused_experts_impl(*args, **kw)
    per_slot = fused_experts_impl(*args, no_combine=True, **kw)
    torch.cuda.synchronize()
    assert _rel_err(out.float().cpu().numpy(), ref) <= REL_TOL
    assert per_slot.shape == (T, topk, H)
    assert (per_slot.float().cpu().numpy()[ids == -1] == 0).all()
    np.testing.assert_array_equal(out.float().cpu().numpy(), O.moe_sum_reduce(per_slot.float().cpu().numpy(), 1.0))


class _LazyExperts:
    """Expert-indexed view of a device tensor that copies one expert to the host when the oracle asks for it."""

    def __init__(self, t, as_u8):
        self.t, self.as_u8, self.shape = t, as_u8, tuple(t.shape)

    def __getitem__(self, e):
        v = self.t[e]
        return (v.view(torch.uint8) if self.as_u8 else v).cpu().numpy()


@pytest.fixture(scope="module")
def deepseek_experts(dev):
    """256 experts, hidden 7168, intermediate 2048: 11 GB of random e4m3fn weights generated on the device (no NaN
    codes) with float32 block scales; shared by the full-size tests below and released afterwards."""
    E, H, I = 256, 7168, 2048
    g = torch.Generator(device=dev)
    g.manual_seed(0)

    def rand_fp8(shape):
        b = torch.randint(0, 256, shape, generator=g, device=dev, dtype=torch.uint8)
        return torch.where((b & 0x7F) == 0x7F, b & 0xFE, b).view(torch.float8_e4m3fn)

    w1 = rand_fp8((E, 2 * I, H))
    w2 = rand_fp8((E, H, I))
    w1s = torch.rand((E, 2 * I // 128, H // 128), generator=g, device=dev) * 2e-4 + 1e-4
    w2s = torch.rand((E, H // 128, I // 128), generator=g, device=dev) * 2e-4 + 1e-4
    bias = torch.randn((E,), generator=g, device=dev) * 0.1
    yield dict(E=E, H=H, I=I, w1=w1, w2=w2, w1s=w1s, w2s=w2s, bias=bias, gen=g)
    del w1, w2
    torch.cuda.empty_cache()


@pytest.mark.parametrize("T", [1, 3, 32, 256, 4096, 16384])
def test_fused_experts_deepseek_dims(dev, deepseek_experts, T):
    """The fused MoE layer at its full DeepSeek-V3 dimensions (256 experts, hidden 7168, intermediate 2048, top-8
    grouped-sigmoid routing over 8 groups / 4 groups kept) for 1, 3, 32, 256, 4096 and 16384 tokens: these token counts
    take the 16-, 32- and 256-slot grouped kernels in turn (asserted below), the last on a table that
    moe_balance_blocks has dealt out evenly (several blocks per expert).  A token's output depends on
    nothing but its own row, its eight experts and its routed weights, so the oracle is evaluated on a sample of
    tokens (all of them up to 3 tokens) with only the experts those tokens hit copied back; the whole output must
    be finite, and permuting the tokens must permute the result (exactly where the kernel choice per expert is
    unchanged, which holds for a permutation: every expert keeps its slot count)."""
    from sglang_amd.fused_moe import biased_grouped_topk, blocks_want_balancing, fused_experts_impl, get_default_config

    d = deepseek_experts
    E, H, topk = d["E"], d["H"], 8
    want_block = {1: 16, 3: 16, 32: 16, 256: 32, 4096: 256, 16384: 256}[T]
    assert get_default_config(T, E, topk)["BLOCK_SIZE_M"] == want_block
    assert blocks_want_balancing(get_default_config(T, E, topk), T * topk, E) == (T == 16384)
    x = O.make_activation(T, H, T)
    logits = torch.randn((T, E), generator=d["gen"], device=dev)
    xt = bf16_tensor(x, dev)
    tw, ids = biased_grouped_topk(xt, logits, d["bias"], topk, True, 8, 4)
    kw = dict(use_fp8_w8a8=True, w1_scale=d["w1s"], w2_scale=d["w2s"], block_shape=[128, 128], routed_scaling_factor=2.5)
    out = fused_experts_impl(xt, d["w1"], d["w2"], tw, ids, **kw)
    torch.cuda.synchronize()
    assert out.shape == (T, H) and out.dtype == torch.bfloat16
    assert bool(torch.isfinite(out).all())
    ids_np, tw_np = ids.cpu().numpy(), tw.cpu().numpy()

    rng = np.random.default_rng(T)
    sample = np.arange(T) if T <= 3 else np.unique(np.concatenate([[0, T - 1], rng.integers(0, T, 4)]))
    ref = O.fused_moe_block_fp8(x[sample], _LazyExperts(d["w1"], True), _LazyExperts(d["w1s"], False),
                                _LazyExperts(d["w2"], True), _LazyExperts(d["w2s"], False), tw_np[sample], ids_np[sample], 2.5)
    got = out[torch.from_numpy(sample).to(dev)].float().cpu().numpy()
    assert _rel_err(got, ref) <= REL_TOL, _rel_err(got, ref)
    # routing agrees with the numpy restatement (as sets; top-k order is unspecified)
    _, ids_ref = O.biased_grouped_topk(logits.cpu().numpy()[sample], d["bias"].cpu().numpy(), 8, 4, topk)
    np.testing.assert_array_equal(np.sort(ids_np[sample], 1), np.sort(ids_ref, 1))
    if T > 3:
        perm = torch.from_numpy(rng.permutation(T)).to(dev)
        out_p = fused_experts_impl(xt[perm].contiguous(), d["w1"], d["w2"], tw[perm].contiguous(), ids[perm].contiguous(), **kw)
        torch.cuda.synchronize()
        assert torch.equal(out_p, out[perm])


@pytest.mark.parametrize("T", [4096, 16384])
def test_cutlass_fused_experts_deepseek_dims(dev, deepseek_experts, T):
    """The expert-major layer (cutlass_fused_experts_fp8) at the full DeepSeek-V3 dimensions: 32768 and 131072 ids take
    the multi-workgroup forms of prepare_moe_input and of the block table, GEMM 1 writes the requantised activation out
    itself, and at 16384 tokens the table is dealt out evenly and walked.  Oracle (expert-major composite) on a sample of
    tokens; the whole output against the slot-ordered layer of this library on the same inputs, as
    python/sglang/test/test_cutlass_moe.py compares the two paths."""
    from sglang_amd.cutlass_moe import cutlass_fused_experts_fp8
    from sglang_amd.fused_moe import biased_grouped_topk, fused_experts_impl

    d = deepseek_experts
    E, H, I, topk = d["E"], d["H"], d["I"], 8
    x = O.make_activation(T, H, T + 1)
    logits = torch.randn((T, E), generator=d["gen"], device=dev)
    xt = bf16_tensor(x, dev)
    tw, ids = biased_grouped_topk(xt, logits, d["bias"], topk, True, 8, 4)
    i64 = lambda: torch.empty((E,), device=dev, dtype=torch.int64)  # noqa: E731
    out = cutlass_fused_experts_fp8(
        xt, d["w1"].transpose(1, 2), d["w2"].transpose(1, 2), d["w1s"].transpose(1, 2), d["w2s"].transpose(1, 2), tw, ids,
        torch.full((E,), H, device=dev, dtype=torch.int64), torch.full((E,), 2 * I, device=dev, dtype=torch.int64),
        torch.full((E,), I, device=dev, dtype=torch.int64), torch.full((E,), H, device=dev, dtype=torch.int64),
        torch.empty((1024,), device=dev, dtype=torch.uint8), i64(), i64(), i64(), i64(), i64(),
        torch.empty((E + 1,), device=dev, dtype=torch.int32), torch.empty((E, 3), device=dev, dtype=torch.int32),
        torch.empty((E, 3), device=dev, dtype=torch.int32), use_fp8_blockscale=True)
    torch.cuda.synchronize()
    assert out.shape == (T, H) and out.dtype == torch.bfloat16 and bool(torch.isfinite(out).all())
    rng = np.random.default_rng(T)
    sample = np.unique(np.concatenate([[0, T - 1], rng.integers(0, T, 4)]))
    ref = O.cutlass_fused_experts_fp8(x[sample], _LazyExperts(d["w1"], True), _LazyExperts(d["w1s"], False),
                                      _LazyExperts(d["w2"], True), _LazyExperts(d["w2s"], False),
                                      tw.cpu().numpy()[sample], ids.cpu().numpy()[sample])
    got = out[torch.from_numpy(sample).to(dev)].float().cpu().numpy()
    assert _rel_err(got, ref) <= REL_TOL, _rel_err(got, ref)
    slot_order = fused_experts_impl(xt, d["w1"], d["w2"], tw, ids, use_fp8_w8a8=True, w1_scale=d["w1s"], w2_scale=d["w2s"],
                                    block_shape=[128, 128]).double()
    o = out.double()
    assert float(1 - 2 * (o * slot_order).sum() / ((o * o).sum() + (slot_order * slot_order).sum())) < 1e-3


@pytest.mark.parametrize("T,block", [(1024, 64), (2048, 128), (1024, 256)])
def test_fused_experts_deepseek_dims_other_block_sizes(dev, deepseek_experts, T, block, monkeypatch):
    """The 64- and 128-slot grouped streaming kernels at the full expert dimensions (a caller's own BLOCK_SIZE_M; the
    default choice goes from 32-slot blocks straight to 256-slot ones, which 1024 tokens take half empty): a sample of
    tokens against the oracle."""
    import sglang_amd.fused_moe as fm
    from sglang_amd.fused_moe import biased_grouped_topk, fused_experts_impl

    d = deepseek_experts
    E, H, topk = d["E"], d["H"], 8
    if block == 256:
        assert fm.get_default_config(T, E, topk)["BLOCK_SIZE_M"] == 256
    else:
        monkeypatch.setattr(fm, "get_default_config", lambda M_, E_, k_: {"BLOCK_SIZE_M": block, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 128})
    x = O.make_activation(T, H, T)
    logits = torch.randn((T, E), generator=d["gen"], device=dev)
    xt = bf16_tensor(x, dev)
    tw, ids = biased_grouped_topk(xt, logits, d["bias"], topk, True, 8, 4)
    out = fused_experts_impl(xt, d["w1"], d["w2"], tw, ids, use_fp8_w8a8=True, w1_scale=d["w1s"], w2_scale=d["w2s"],
                             block_shape=[128, 128], routed_scaling_factor=2.5)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    rng = np.random.default_rng(T)
    sample = np.unique(np.concatenate([[0, T - 1], rng.integers(0, T, 3)]))
    ref = O.fused_moe_block_fp8(x[sample], _LazyExperts(d["w1"], True), _LazyExperts(d["w1s"], False),
                                _LazyExperts(d["w2"], True), _LazyExperts(d["w2s"], False), tw.cpu().numpy()[sample],
                                ids.cpu().numpy()[sample], 2.5)
    got = out[torch.from_numpy(sample).to(dev)].float().cpu().numpy()
    assert _rel_err(got, ref) <= REL_TOL, _rel_err(got, ref)


@pytest.mark.parametrize("rows", [1, 7, 64, 1000])
@pytest.mark.parametrize("params", [(128, 4, 2, 4), (256, 8, 4, 8), (512, 16, 8, 16), (64, 8, 3, 6)])
@pytest.mark.parametrize("shared,scale_out", [(0, False), (1, True), (2, False)])
def test_moe_fused_gate_vs_oracle(dev, rows, params, shared, scale_out):
    """Reference: sgl-kernel/tests/test_moe_fused_gate.py:8-101 (float32 inputs, the DeepSeek-V3 tuple among them).
    Ids must equal the oracle's in order (same tie rules), weights to 1e-5 (expf may differ in the last bit)."""
    from sglang_amd.sgl_kernel import moe_fused_gate

    E, G, tg, topk = params
    g = torch.Generator().manual_seed(rows * 7 + E)
    x = torch.rand((rows, E), generator=g)
    bias = torch.rand((E,), generator=g)
    w, ids = moe_fused_gate(x.to(dev), bias.to(dev), G, tg, topk + shared, shared, 2.5, scale_out)
    torch.cuda.synchronize()
    w_ref, ids_ref = O.moe_fused_gate(x.numpy(), bias.numpy(), G, tg, topk + shared, shared, 2.5, scale_out)
    assert w.dtype == torch.float32 and ids.dtype == torch.int32 and tuple(w.shape) == (rows, topk + shared)
    got_i, got_w = ids.cpu().numpy(), w.cpu().numpy()
    same = (got_i == ids_ref).all(axis=1)
    # a last-bit difference in expf can swap two near-equal choices: such rows must still hold the same set
    for r in np.nonzero(~same)[0]:
        assert sorted(got_i[r].tolist()) == sorted(ids_ref[r].tolist())
    assert same.mean() >= 0.99
    np.testing.assert_allclose(np.sort(got_w, axis=1), np.sort(w_ref, axis=1), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16")])
def test_moe_fused_gate_bf16_and_ties(dev, dtype, name):
    """16-bit inputs make ties common (the arithmetic is done in the input type): the tie rules must hold."""
    from sglang_amd.sgl_kernel import moe_fused_gate

    g = torch.Generator().manual_seed(5)
    x = torch.randn((300, 256), generator=g).to(dtype)
    bias = (torch.randn((256,), generator=g) * 0.1).to(dtype)
    w, ids = moe_fused_gate(x.to(dev), bias.to(dev), 8, 4, 8)
    w_ref, ids_ref = O.moe_fused_gate(x.float().numpy(), bias.float().numpy(), 8, 4, 8, in_dtype=name)
    got_i = ids.cpu().numpy()
    same = (got_i == ids_ref).all(axis=1)
    for r in np.nonzero(~same)[0]:
        assert sorted(got_i[r].tolist()) == sorted(ids_ref[r].tolist())
    assert same.mean() >= 0.97
    np.testing.assert_allclose(np.sort(w.cpu().numpy(), axis=1), np.sort(w_ref, axis=1), rtol=2e-2, atol=1e-3)
    # all-equal inputs: groups 7..4 are dropped, experts 0..7 win
    z = torch.zeros((3, 256), device=dev, dtype=dtype)
    w0, i0 = moe_fused_gate(z, torch.zeros((256,), device=dev, dtype=dtype), 8, 4, 8)
    assert i0.cpu().tolist() == [list(range(8))] * 3
    assert torch.allclose(w0, torch.full_like(w0, 0.125))


def test_biased_grouped_topk_is_the_gate_kernel_and_matches_the_tensor_op_restatement(dev):
    """The layer-level routing entry point runs the fused gate kernel; on well-separated float32 logits its expert sets
    and weights are those of the tensor-op restatement of topk.py:665-738 kept with the tests.  Shapes the kernel does
    not take are refused (the product path has no second implementation)."""
    from sglang_amd.fused_moe import biased_grouped_topk
    from tests.routing_torch import biased_grouped_topk_impl

    g = torch.Generator(device=dev)
    g.manual_seed(3)
    logits = torch.randn((513, 256), generator=g, device=dev)
    bias = torch.randn((256,), generator=g, device=dev) * 0.01
    x = torch.empty((513, 16), device=dev, dtype=torch.bfloat16)
    w, ids = biased_grouped_topk(x, logits, bias, 8, True, 8, 4)
    w_t, ids_t = biased_grouped_topk_impl(x, logits, bias, 8, True, 8, 4)
    order, order_t = ids.argsort(dim=1), ids_t.argsort(dim=1)
    same = (ids.gather(1, order) == ids_t.gather(1, order_t)).all(dim=1)
    assert float(same.float().mean()) >= 0.99  # a last-bit difference in the sigmoid can swap two near-equal choices
    torch.testing.assert_close(w.gather(1, order)[same], w_t.gather(1, order_t)[same], rtol=1e-5, atol=1e-7)
    with pytest.raises(RuntimeError, match="power-of-two expert count"):
        biased_grouped_topk(x, logits[:, :96].contiguous(), bias[:96].contiguous(), 4, True, 4, 2)
    with pytest.raises(RuntimeError, match="renormalised"):
        biased_grouped_topk(x, logits, bias, 8, False, 8, 4)


def test_moe_fused_gate_errors(dev):
    from sglang_amd.sgl_kernel import moe_fused_gate

    x = torch.zeros((4, 96), device=dev)
    with pytest.raises(RuntimeError, match="power of 2"):
        moe_fused_gate(x, torch.zeros((96,), device=dev), 4, 2, 4)
    x = torch.zeros((4, 256), device=dev)
    with pytest.raises(RuntimeError, match="exceeds the maximum supported"):
        moe_fused_gate(x, torch.zeros((256,), device=dev), 4, 2, 4)
    with pytest.raises(RuntimeError, match="same dtype"):
        moe_fused_gate(x, torch.zeros((256,), device=dev, dtype=torch.bfloat16), 8, 4, 8)


@pytest.mark.parametrize("T,E,H,I,topk", [(1024, 8, 512, 256, 2), (700, 4, 256, 128, 4), (2100, 8, 384, 384, 3)])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_gemm1_with_fused_activation_quant_is_the_three_step_sequence(dev, T, E, H, I, topk, dt):
    """256-slot blocks: the first grouped GEMM with silu_and_mul and the requantisation in its write-out against the same
    GEMM into a 16-bit tensor followed by the fused silu + group quant kernel - bytes and scales of every real slot bit
    for bit, and the whole layer (fused by default at this block size) bit for bit the sequence continued by hand.  The
    layer with the fusion on is held against the oracle at the full DeepSeek-V3 dimensions by
    test_fused_experts_deepseek_dims (4096 tokens take 256-slot blocks)."""
    import sglang_amd.fused_moe as fm
    from sglang_amd import custom_ops as ops
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    rng = np.random.default_rng(T + I)
    x = torch.from_numpy(O.make_activation(T, H, T)).to(dev).to(dt)
    w13q = np.empty((E, 2 * I, H), np.uint8); w13s = np.empty((E, 2 * I // 128, H // 128), np.float32)
    w2q = np.empty((E, H, I), np.uint8); w2s = np.empty((E, H // 128, I // 128), np.float32)
    for e in range(E):
        w13q[e], w13s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((2 * I, H)).astype(np.float32) * 0.05))
        w2q[e], w2s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((H, I)).astype(np.float32) * 0.05))
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    if E > 4:
        ids[ids == 1] = 0  # one expert without tokens, one with twice the share (more than one block)
    tw = rng.uniform(0.1, 1.0, (T, topk)).astype(np.float32)
    w1, w2 = fp8_tensor(w13q, dev), fp8_tensor(w2q, dev)
    s1, s2 = torch.from_numpy(w13s).to(dev), torch.from_numpy(w2s).to(dev)
    idt, twt = torch.from_numpy(ids).to(dev), torch.from_numpy(tw).to(dev)
    slots = T * topk

    sorted_ids, expert_ids, post_pad = fm.moe_align_block_size(idt, 256, E)
    a1_q, a1_s = sglang_per_token_group_quant_fp8(x, 128)
    a1_ss = ops.moe_sort_scales(a1_s, sorted_ids, post_pad, topk, slots)
    c1 = torch.empty((slots, 2 * I), device=dev, dtype=dt)
    ops.moe_block_gemm(a1_q, w1, c1, a1_ss, s1, None, sorted_ids, expert_ids, post_pad, False, topk, 256, slots, scales_sorted=True)
    ref_q, ref_s = sglang_per_token_group_quant_fp8(c1, 128, fuse_silu_and_mul=True)
    got_q = torch.zeros((slots, I), device=dev, dtype=torch.float8_e4m3fn)
    got_s = torch.full((I // 128, sorted_ids.numel()), -1.0, device=dev, dtype=torch.float32).t()
    ops.moe_block_gemm_silu_quant(a1_q, w1, a1_ss, s1, got_q, got_s, sorted_ids, expert_ids, post_pad, topk, slots, dt)
    torch.cuda.synchronize()
    assert torch.equal(got_q.view(torch.uint8), ref_q.view(torch.uint8))
    sid = sorted_ids[: int(post_pad.item())].long()
    real = sid < slots
    assert torch.equal(got_s[: sid.numel()][real], ref_s[sid[real]])
    assert bool((got_s[: sid.numel()][~real] == 0).all())

    # the whole layer (which takes the fused GEMM 1 with 256-slot blocks) against the three-step sequence continued by hand
    a2_ss = ops.moe_sort_scales(ref_s, sorted_ids, post_pad, 1, slots)
    c3 = torch.empty((T, topk, H), device=dev, dtype=dt)
    ops.moe_block_gemm(ref_q, w2, c3, a2_ss, s2, twt, sorted_ids, expert_ids, post_pad, True, 1, 256, slots, scales_sorted=True)
    plain = torch.empty((T, H), device=dev, dtype=dt)
    ops.moe_sum_reduce(c3, plain, 1.0)
    kw = dict(use_fp8_w8a8=True, w1_scale=s1, w2_scale=s2, block_shape=[128, 128])
    old = fm.get_default_config
    fm.get_default_config = lambda M_, E_, t_: {"BLOCK_SIZE_M": 256, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 128}
    try:
        assert fm.gemm1_fuses_activation(fm.get_default_config(T, E, topk), 2 * I)
        fused = fm.fused_experts_impl(x, w1, w2, twt, idt, **kw)
    finally:
        fm.get_default_config = old
    assert torch.equal(fused, plain)


@pytest.mark.parametrize("T,E,topk,block", [(700, 4, 2, 256), (2100, 8, 3, 256), (300, 16, 4, 64), (16384, 256, 8, 256), (5, 8, 2, 16)])
def test_moe_balance_blocks_deals_every_experts_slots_out_evenly(dev, T, E, topk, block):
    """moe_balance_blocks: the same blocks per expert and the same slots per expert (as sets), every block of an expert
    holding floor or ceil of slots / blocks of them, real slots first in every block, padding value elsewhere; the
    grouped GEMM on the balanced table gives the same rows as on the aligner's."""
    from sglang_amd.fused_moe import moe_align_block_size
    from sglang_amd.sgl_kernel import moe_balance_blocks, moe_block_gemm, moe_sort_scales

    rng = np.random.default_rng(T + E)
    ids = _random_ids(rng, T, E, topk, 0.1 if T > 5 else 0.0)
    numel = ids.size
    sorted_ids, expert_ids, npad = moe_align_block_size(torch.from_numpy(ids).to(dev), block, E)
    bal = moe_balance_blocks(sorted_ids, expert_ids, npad, block, numel, E)
    torch.cuda.synchronize()
    used = int(npad.item())
    a, b, eid = sorted_ids.cpu().numpy(), bal.cpu().numpy(), expert_ids.cpu().numpy()[: used // block]
    assert (b[used:] == numel).all()
    flat = ids.reshape(-1)
    for e in np.unique(eid):
        blocks = np.nonzero(eid == e)[0]
        assert np.array_equal(blocks, np.arange(blocks[0], blocks[0] + blocks.size))
        seg_a = a[blocks[0] * block:(blocks[-1] + 1) * block]
        seg_b = b[blocks[0] * block:(blocks[-1] + 1) * block].reshape(blocks.size, block)
        real_a = seg_a[seg_a < numel]
        assert np.array_equal(np.sort(seg_b[seg_b < numel]), np.sort(real_a))
        if e >= 0:
            assert np.array_equal(np.sort(real_a), np.nonzero(flat == e)[0])
        per_block = (seg_b < numel).sum(axis=1)
        assert per_block.max() - per_block.min() <= 1 and per_block.sum() == real_a.size
        for row, n_real in zip(seg_b, per_block):
            assert (row[:n_real] < numel).all() and (row[n_real:] == numel).all()
    if block < 64:
        return
    # the grouped GEMM does not care which table it walks
    N, K = 256, 256
    wq, ws = _expert_weights(rng, E, N, K)
    xq = O.f32_to_e4m3fn(np.clip(rng.standard_normal((T, K)).astype(np.float32) * 100, -448, 448))
    xs = (rng.uniform(0.5, 2.0, (T, K // 128)) * 1e-2).astype(np.float32)
    A, B = fp8_tensor(xq, dev), fp8_tensor(wq, dev)
    As, Bs = torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev)
    outs = []
    for table in (sorted_ids, bal):
        C = torch.zeros((numel, N), dtype=torch.bfloat16, device=dev)
        sc = moe_sort_scales(As, table, npad, topk, numel)
        moe_block_gemm(A, B, C, sc, Bs, torch.ones((T, topk), device=dev), table, expert_ids, npad, False, topk, block, numel,
                       scales_sorted=True)
        torch.cuda.synchronize()
        outs.append(C)
    assert torch.equal(outs[0], outs[1])
