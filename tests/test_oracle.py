"""Pins of the CPU oracle (no GPU): every oracle function is checked against something that does
not share its formula - torch's CPU conversions, closed forms from the reference's own tests,
exhaustive tables, float64 arithmetic, brute force on tiny inputs, or integer invariants."""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import fp8_oracle as O


# ---------------------------------------------------------------- formats
def test_e4m3fn_encode_matches_torch_on_every_16bit_prefix():
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    for low in (0x0000, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1234):
        x = (hi | low).view(np.float32)
        ref = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        got = O.f32_to_e4m3fn(x)
        ok = (ref == got) | np.isnan(x)  # NaN sign is unspecified
        assert ok.all()


def test_e4m3fn_known_answers():
    # OCP table: max 448, no Inf, 0x7F NaN, subnormal step 2^-9, ties to even
    x = np.array([448, 464, 463.9, 480, 1e9, 2**-10, 1.5 * 2**-9, 2**-9, 2**-6, 0.0, -0.0, 1.0, -1.5, 17.0, 18.0],
                 dtype=np.float32)
    exp = [0x7E, 0x7E, 0x7E, 0x7F, 0x7F, 0x00, 0x02, 0x01, 0x08, 0x00, 0x80, 0x38, 0xBC, 0x58, 0x59]
    assert O.f32_to_e4m3fn(x).tolist() == exp
    assert O.f32_to_e4m3fn(np.array([19.0], np.float32))[0] == 0x5A  # 19 is a tie between 18 and 20 -> even mantissa (20)


def test_e4m3fn_decode_matches_torch_and_roundtrips():
    b = np.arange(256, dtype=np.uint8)
    t = torch.from_numpy(b).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(t, nan=-7.0), np.nan_to_num(O.E4M3FN_TABLE, nan=-7.0))
    finite = ~np.isnan(O.E4M3FN_TABLE)
    assert np.array_equal(O.f32_to_e4m3fn(O.E4M3FN_TABLE[finite]), b[finite])


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(0)
    y = (rng.standard_normal(200000) * rng.choice([1e-20, 1.0, 1e20], 200000)).astype(np.float32)
    assert np.array_equal(O.to_bf16(y), torch.from_numpy(y).bfloat16().float().numpy())
    assert np.array_equal(O.bf16_from_bits(O.bf16_bits(O.to_bf16(y))), O.to_bf16(y))


# ---------------------------------------------------------------- group quant
def test_eps_is_clamped_in_the_input_dtype():
    assert O.clamp_eps(1e-10, "bf16") == torch.tensor([0.0], dtype=torch.bfloat16).clamp(min=1e-10).float().item()
    assert O.clamp_eps(1e-10, "f32") == np.float32(1e-10)


def test_group_quant_closed_form_amax_448():
    """python/sglang/test/srt/quant/test_fp8_kernel.py:24-45: a group whose amax is exactly 448 has scale 1
    and quantises to the fp8 encoding of its own values."""
    rng = np.random.default_rng(1)
    vals = O.E4M3FN_TABLE[rng.integers(0, 0x7F, (16, 512))] * rng.choice([-1, 1], (16, 512)).astype(np.float32)
    vals = vals.reshape(-1, 128)
    vals[:, 0] = 448.0
    vals = vals.reshape(16, 512)
    q, s = O.per_token_group_quant_fp8(vals, 128, in_dtype="f32")
    assert (s == 1.0).all()
    assert np.array_equal(O.e4m3fn_to_f32(q), vals)


def test_group_quant_against_torch_library_ops():
    """Same steps with torch CPU tensor ops (abs/max/clamp/div/to(float8)) on bf16 data."""
    x = O.make_activation(96, 2048, 3)
    xt = torch.from_numpy(x).bfloat16()
    g = xt.reshape(-1, 128)
    amax = g.abs().max(dim=-1, keepdim=True)[0].clamp(min=1e-10).to(torch.float32)
    xs = amax / 448.0
    xq = (g / xs).clamp(min=-448.0, max=448.0).to(torch.float8_e4m3fn)
    q, s = O.per_token_group_quant_fp8(x, 128)
    assert np.array_equal(q.reshape(-1, 128), xq.view(torch.uint8).numpy())
    assert np.array_equal(s.reshape(-1, 1), xs.numpy())


def test_scale_table_every_bf16_amax():
    bits = np.arange(1, 0x7F80, dtype=np.uint32)
    amax = (bits << 16).view(np.float32)
    x = np.zeros((amax.size, 128), dtype=np.float32)
    x[:, 5] = amax
    _, s = O.per_token_group_quant_fp8(x, 128)
    expect = (torch.from_numpy(amax).bfloat16().clamp(min=1e-10).float() / 448.0).numpy()
    assert np.array_equal(s[:, 0], expect)


def test_ue8m0_bit_form_equals_pow2_ceil_log2_for_every_bf16_amax():
    bits = np.arange(0x0080, 0x7F80, dtype=np.uint32)  # positive normal bf16
    amax = np.maximum((bits << 16).view(np.float32), np.float32(1e-10))
    s = (amax / np.float32(448)).astype(np.float32)
    s = s[(s > 1e-30) & (s < 1e30)]
    via_log = torch.pow(2.0, torch.ceil(torch.log2(torch.from_numpy(s).double()))).float().numpy()
    assert np.array_equal(O.ceil_to_ue8m0(s), via_log)
    assert (O.ceil_to_ue8m0(s) >= s).all() and (O.ceil_to_ue8m0(s) < 2 * s).all()


def test_ue8m0_pack_roundtrip_and_layout():
    rng = np.random.default_rng(2)
    s = (2.0 ** rng.integers(-30, 10, (7, 6))).astype(np.float32)
    w = O.pack_ue8m0_scales(s)
    assert w.shape == (7, 2) and w.dtype == np.int32
    by = w.view(np.uint8).reshape(7, 8)
    assert np.array_equal(by[:, :6], O.ue8m0_byte(s)) and (by[:, 6:] == 0).all()
    assert np.array_equal(O.unpack_ue8m0_scales(w, 6), s)
    assert O.ue8m0_byte(np.array([1.0], np.float32))[0] == 127


def test_ue8m0_quant_divides_by_power_of_two():
    x = O.make_activation(8, 512, 4)
    q, s = O.per_token_group_quant_fp8(x, 128, scale_ue8m0=True)
    m, e = np.frexp(s)
    assert (m == 0.5).all()
    _, s_plain = O.per_token_group_quant_fp8(x, 128)
    assert (s >= s_plain).all() and (s < 2 * s_plain).all()


# ---------------------------------------------------------------- per-token / per-tensor
def test_per_token_and_tensor_quant_against_torch_ops():
    x = O.make_activation(33, 1024, 5)
    x[4] = 0
    q, s = O.per_token_quant_fp8(x)
    xt = torch.from_numpy(x)
    st = xt.abs().amax(dim=-1, keepdim=True) / 448.0
    inv = torch.where(st == 0, torch.zeros_like(st), 1.0 / st)
    qt = (xt * inv).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, qt) and np.array_equal(s, st.numpy())
    assert s[4, 0] == 0 and (q[4] == 0).all()
    q2, s2 = O.per_tensor_quant_fp8(x)
    s2t = xt.abs().max() / 448.0
    q2t = (xt * (1.0 / s2t)).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert s2[0] == s2t.item() and np.array_equal(q2, q2t)


def test_block_quant_weight_roundtrip_error():
    w = O.make_weight(384, 640, 1)
    q, s = O.block_quant_weight(w)
    assert s.shape == (3, 5)
    deq = O.e4m3fn_to_f32(q).reshape(3, 128, 5, 128) * s[:, None, :, None]
    err = np.abs(deq.reshape(384, 640) - w)
    assert err.max() <= np.abs(w).max() * 2**-4  # 3 mantissa bits
    blk = np.abs(O.e4m3fn_to_f32(q)).reshape(3, 128, 5, 128).max(axis=(1, 3))
    assert (blk == 448).all()  # every block uses the full range


# ---------------------------------------------------------------- matmuls
def _brute(Aq, Bq, As, Bs):
    A, B = O.e4m3fn_to_f32(Aq).astype(np.float64), O.e4m3fn_to_f32(Bq).astype(np.float64)
    M, K = A.shape
    N = B.shape[0]
    C = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            for k in range(K):
                C[m, n] += A[m, k] * B[n, k] * As[m, k // 128] * Bs[n // 128, k // 128]
    return C


def test_block_matmul_vs_brute_force_triple_loop():
    rng = np.random.default_rng(6)
    Aq = O.f32_to_e4m3fn(rng.standard_normal((5, 256)).astype(np.float32) * 20)
    Bq = O.f32_to_e4m3fn(rng.standard_normal((130, 256)).astype(np.float32) * 20)
    As = rng.uniform(0.5, 2, (5, 2)).astype(np.float32)
    Bs = rng.uniform(0.5, 2, (2, 2)).astype(np.float32)
    ref = _brute(Aq, Bq, As, Bs)
    got = O.w8a8_block_fp8_matmul(Aq, Bq, As, Bs, out_dtype="f32", acc=np.float64)
    np.testing.assert_allclose(got, ref, rtol=1e-6, atol=1e-6 * np.abs(ref).max())
    got32 = O.w8a8_block_fp8_matmul(Aq, Bq, As, Bs, out_dtype="f32", acc=np.float32)
    np.testing.assert_allclose(got32, ref, rtol=0, atol=1e-5 * np.abs(ref).max())


def test_block_matmul_dequantise_then_matmul_and_linearity():
    """sgl-kernel/tests/test_fp8_blockwise_gemm.py:19-59: broadcast the scales, multiply in high precision."""
    xq, xs = O.per_token_group_quant_fp8(O.make_activation(40, 1024, 7), 128)
    wq, ws = O.block_quant_weight(O.make_weight(384, 1024, 7))
    a = O.e4m3fn_to_f32(xq).astype(np.float64) * np.repeat(xs, 128, axis=1)
    b = O.e4m3fn_to_f32(wq).astype(np.float64) * np.repeat(np.repeat(ws, 128, axis=0), 128, axis=1)
    ref = a @ b.T
    got = O.w8a8_block_fp8_matmul(xq, wq, xs, ws, out_dtype="f32", acc=np.float64)
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6 * np.abs(ref).max())
    got4 = O.w8a8_block_fp8_matmul(xq, wq, (xs * 4).astype(np.float32), ws, out_dtype="f32", acc=np.float64)
    np.testing.assert_array_equal(got4, 4 * got)


def test_scaled_mm_vs_torch_restatement():
    """sgl-kernel/tests/test_fp8_gemm.py:6-14."""
    rng = np.random.default_rng(8)
    aq = O.f32_to_e4m3fn(rng.standard_normal((9, 512)).astype(np.float32) * 10)
    bq = O.f32_to_e4m3fn(rng.standard_normal((64, 512)).astype(np.float32) * 10)
    sa = rng.uniform(0.1, 1, 9).astype(np.float32)
    sb = rng.uniform(0.1, 1, 64).astype(np.float32)
    bias = O.to_bf16(rng.standard_normal(64).astype(np.float32))
    A = torch.from_numpy(aq).view(torch.float8_e4m3fn).to(torch.float32)
    B = torch.from_numpy(bq).view(torch.float8_e4m3fn).to(torch.float32)
    o = torch.matmul(A, B.t()) * torch.from_numpy(sa).view(-1, 1) * torch.from_numpy(sb).view(1, -1)
    o = (o + torch.from_numpy(bias)).to(torch.bfloat16).float().numpy()
    got = O.fp8_scaled_mm(aq, bq, sa, sb, "bf16", bias)
    assert np.abs(got - o).max() <= 2**-7 * np.abs(o).max()  # one bf16 ulp from summation order


# ---------------------------------------------------------------- C restatement == numpy restatement
def test_c_oracle_matches_numpy_oracle():
    lib = c_oracle.load()
    x = O.make_activation(70, 1536, 9)
    x[3, :128] = 0
    eps = float(O.clamp_eps(1e-10, "bf16"))
    for ue in (False, True):
        q, s = O.per_token_group_quant_fp8(x, 128, scale_ue8m0=ue)
        qc, sc = c_oracle.group_quant_bf16(lib, O.bf16_bits(x), 128, eps, ue)
        assert np.array_equal(q, qc) and np.array_equal(s.view(np.uint32), sc.view(np.uint32))
    q, s = O.per_token_group_quant_fp8(x, 128)
    wq, ws = O.block_quant_weight(O.make_weight(640, 1536, 9))
    ref = O.w8a8_block_fp8_matmul(q, wq, s, ws, out_dtype="f32", acc=np.float64)
    c = O.bf16_from_bits(c_oracle.block_gemm(lib, q, wq, s, ws))
    assert np.abs(c - ref).max() <= 2**-7 * np.abs(ref).max()
    sa = np.random.default_rng(1).uniform(0.1, 1, 70).astype(np.float32)
    sb = np.random.default_rng(2).uniform(0.1, 1, 640).astype(np.float32)
    ref2 = O.fp8_scaled_mm(q, wq, sa, sb, "f32")
    c2 = O.bf16_from_bits(c_oracle.scaled_mm(lib, q, wq, sa, sb))
    assert np.abs(c2 - ref2).max() <= 2**-7 * np.abs(ref2).max()


def test_w8a16_cpu_twin_restatement():
    """The W8A16 algorithm of the reference's CPU kernel (sgl-kernel/csrc/cpu/gemm_fp8.cpp:46-100, 356-424), restated in
    numpy and in C.  Pins: (1) on weights whose block scale is 1 and activations that are exact e4m3 values it IS the
    W8A8 block matmul with unit scales (no rounding anywhere: integers); (2) the weight dequantisation is the torch
    expression bf16(w8.to(bf16).float() * scale); (3) C == numpy to float-accumulation noise; (4) on realistic data it
    stays within 2e-2 of the W8A8 result (the activations are not quantised: that is the whole difference)."""
    import torch

    lib = c_oracle.load()
    rng = np.random.default_rng(5)
    M, N, K = 9, 256, 384
    # (1) exact case: small integers, unit scales
    a_int = rng.integers(-3, 4, (M, K)).astype(np.float32)
    aq = O.f32_to_e4m3fn(a_int)
    bq = O.f32_to_e4m3fn(rng.integers(-2, 3, (N, K)).astype(np.float32))
    ones_a = np.ones((M, K // 128), np.float32)
    ones_b = np.ones((N // 128, K // 128), np.float32)
    w8a8 = O.w8a8_block_fp8_matmul(aq, bq, ones_a, ones_b)
    twin = O.w8a16_block_fp8_matmul_cpu_twin(a_int, bq, ones_b)
    assert np.array_equal(w8a8, twin)
    assert np.array_equal(O.bf16_from_bits(c_oracle.w8a16_block_gemm(lib, O.bf16_bits(a_int), bq, ones_b)), twin)
    # (2) the dequantised weight against torch's own conversions
    wq, ws = O.block_quant_weight(O.make_weight(N, K, 3))
    wt = torch.from_numpy(wq).view(torch.float8_e4m3fn).to(torch.bfloat16).float()
    st = torch.from_numpy(np.repeat(np.repeat(ws, 128, axis=0), 128, axis=1))
    w_ref = (wt * st).to(torch.bfloat16).float().numpy()
    x = O.make_activation(M, K, 4)
    eye = np.eye(K, dtype=np.float32)[:M]  # rows of the identity pick weight columns out
    picked = O.w8a16_block_fp8_matmul_cpu_twin(eye, wq, ws)
    assert np.array_equal(picked, w_ref[:, :M].T)
    # (3) C against numpy, with bias
    bias = rng.normal(size=N).astype(np.float32)
    ref = O.w8a16_block_fp8_matmul_cpu_twin(x, wq, ws, bias, acc=np.float64)
    c = O.bf16_from_bits(c_oracle.w8a16_block_gemm(lib, O.bf16_bits(x), wq, ws, bias))
    assert np.abs(c - ref).max() <= 2**-7 * np.abs(ref).max()
    # (4) next to the W8A8 path on the same data
    q, s = O.per_token_group_quant_fp8(x, 128)
    w8 = O.w8a8_block_fp8_matmul(q, wq, s, ws, acc=np.float64)
    no_bias = O.w8a16_block_fp8_matmul_cpu_twin(x, wq, ws, acc=np.float64)
    assert np.abs(no_bias - w8).max() <= 2e-2 * np.abs(w8).max()


def test_moe_sum_rounding_orders():
    """moe_sum (sgl-kernel/csrc/moe/moe_sum.cu): element-type accumulation for 2-4 experts per token against torch's
    bf16 adds, float accumulation otherwise against torch.sum."""
    import torch

    rng = np.random.default_rng(4)
    for topk in (2, 3, 4, 8):
        x = O.to_bf16(rng.standard_normal((19, topk, 64)).astype(np.float32) * 3)
        xt = torch.from_numpy(x).to(torch.bfloat16)
        if topk <= 4:
            ref = torch.zeros((19, 64), dtype=torch.bfloat16)
            for k in range(topk):
                ref = ref + xt[:, k]
        else:
            ref = torch.sum(xt, dim=1)
        assert np.array_equal(O.moe_sum(x), ref.float().numpy())
    # the two orders differ: the pin above is not vacuous
    x = O.to_bf16(rng.standard_normal((200, 3, 64)).astype(np.float32) * 3)
    assert not np.array_equal(O.moe_sum(x), O.to_bf16(x.sum(axis=1)))


# ---------------------------------------------------------------- MoE helpers
@pytest.mark.parametrize("E,topk,block", [(8, 2, 16), (64, 6, 64), (256, 8, 64), (257, 8, 128)])
def test_moe_align_invariants(E, topk, block):
    """sgl-kernel/tests/test_moe_align.py:210-254: counts, padding, ownership."""
    rng = np.random.default_rng(E)
    T = 97
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    ids[rng.random(ids.shape) < 0.05] = -1
    sorted_ids, expert_ids, npad = O.moe_align_block_size(ids, block, E)
    numel = ids.size
    counts = np.bincount(ids.reshape(-1) + 1, minlength=E + 1)
    assert npad == sum((c + block - 1) // block * block for c in counts)
    assert sorted_ids.size == numel + (E + 1) * (block - 1)
    used = expert_ids[: npad // block]
    assert (np.diff(used) >= 0).all()
    for b, e in enumerate(used):
        blk = sorted_ids[b * block : (b + 1) * block]
        real = blk[blk < numel]
        assert (ids.reshape(-1)[real] == e).all()
        assert (blk[len(real):] == numel).all()
    real_all = sorted_ids[:npad][sorted_ids[:npad] < numel]
    assert np.array_equal(np.sort(real_all), np.arange(numel))
    assert (sorted_ids[npad:] == numel).all()


def test_silu_and_mul_and_sum_reduce_against_torch_bf16():
    rng = np.random.default_rng(10)
    x = O.to_bf16(rng.standard_normal((37, 512)).astype(np.float32) * 3)
    xt = torch.from_numpy(x).bfloat16()
    d = 256
    ref = (torch.nn.functional.silu(xt[..., :d].float()).to(torch.bfloat16) * xt[..., d:]).float().numpy()
    assert np.array_equal(O.silu_and_mul(x), ref)
    y = O.to_bf16(rng.standard_normal((19, 8, 128)).astype(np.float32))
    acc = torch.zeros(19, 128)
    for k in range(8):
        acc = acc + torch.from_numpy(y[:, k])
    ref2 = (acc * 2.5).to(torch.bfloat16).float().numpy()
    assert np.array_equal(O.moe_sum_reduce(y, 2.5), ref2)


def test_gelu_and_mul_against_torch_and_the_identities_of_the_erf_form():
    """gelu_and_mul on every finite bf16 gate value: against torch's library gelu (erf form) with the same two roundings
    and against what the definition fixes: gelu(v) - gelu(-v) = v (the two normal probabilities sum to one), gelu(v) = v
    for v >= 6 and -0 <= gelu(v) for v <= -6 in bf16, gelu(0) = 0.  The tanh approximation and x * sigmoid(1.702 x),
    the forms a mistaken restatement would take, fail the first check.
    Where the two may differ: torch's float32 erf and a correctly rounded one can differ in the last float32 bit, which
    shows where the product sits on a bf16 tie and, magnified, in 1 + erf for v < -4 (the sum cancels: an error of
    2^-24 in it is |v| 2^-25 in a result of 1e-5 and less); above 1.7e38 torch's order of the products overflows where
    the reference's, v * (0.5 * (1 + erf)), does not (activation.cu:66)."""
    bits = np.arange(1 << 16, dtype=np.uint32)
    g = (bits << 16).view(np.float32)
    g = g[np.isfinite(g)]
    one = np.ones_like(g)
    got = O.gelu_and_mul(np.stack([g, one], axis=-1).reshape(-1, 2))[:, 0]
    ref = torch.nn.functional.gelu(torch.from_numpy(g)).bfloat16().float().numpy()
    huge = np.abs(g) > 1.7e38
    assert np.array_equal(got[huge & (g > 0)], g[huge & (g > 0)]) and (got[huge & (g < 0)] == 0).all()
    got, ref, g = got[~huge], ref[~huge], g[~huge]
    assert (got == ref).mean() > 0.9995, (got == ref).mean()
    assert (np.abs(got - ref) <= np.maximum(np.abs(ref) * 2.0**-7, np.abs(g) * 2.0**-22)).all()
    tanh_form = torch.nn.functional.gelu(torch.from_numpy(g), approximate="tanh").bfloat16().float().numpy()
    quick = (torch.from_numpy(g) * torch.sigmoid(1.702 * torch.from_numpy(g))).bfloat16().float().numpy()
    mid = (np.abs(g) > 0.25) & (np.abs(g) < 3)     # beyond, every form is v / 2, v or next to 0 in bf16
    assert (got[mid] == ref[mid]).all()
    assert (got[mid] == tanh_form[mid]).mean() < 0.9 and (got[mid] == quick[mid]).mean() < 0.5
    big = g >= 6
    assert np.array_equal(got[big], g[big])
    assert (got[g <= -6] <= 0).all() and (got[g <= -6] > -1e-7).all()
    assert got[g == 0].tolist() == [0.0, 0.0]
    # gelu(v) - gelu(-v) = v: both sides in bf16, so within an ulp of each term
    pos = g[(g > 2.0**-100) & (g < 6)]
    both = O.gelu_and_mul(np.stack([np.concatenate([pos, -pos]), np.ones(2 * pos.size, np.float32)], axis=-1))[:, 0]
    diff = both[: pos.size] - both[pos.size:]
    assert (np.abs(diff - pos) <= 2.0**-7 * pos).all()
    # the second factor and its rounding
    rng = np.random.default_rng(12)
    x = O.to_bf16(rng.standard_normal((37, 512)).astype(np.float32) * 3)
    xt = torch.from_numpy(x).bfloat16()
    ref2 = (torch.nn.functional.gelu(xt[..., :256].float()).to(torch.bfloat16) * xt[..., 256:]).float().numpy()
    got2 = O.gelu_and_mul(x)
    gate, up = x[:, :256], x[:, 256:]
    assert np.array_equal(got2[gate > -3], ref2[gate > -3])
    assert (np.abs(got2 - ref2) <= 2.0**-6 * np.abs(ref2) + np.abs(gate * up) * 2.0**-21).all()
    assert not np.allclose(got2, O.silu_and_mul(x), rtol=2e-2)


def test_activation_only_against_torch_on_every_bf16_value():
    """activation_only (the ungated experts' activation) against the tensor library's own ops on bf16 tensors, every finite
    bf16 value: silu and relu2 bit for bit; gelu as in the gated test (last-bit differences of erf show on bf16 ties and,
    magnified by the cancellation in 1 + erf, below -3; above 1.7e38 torch's product order overflows)."""
    bits = np.arange(1 << 16, dtype=np.uint32)
    g = (bits << 16).view(np.float32)
    g = g[np.isfinite(g)]
    t = torch.from_numpy(g).bfloat16()
    silu = torch.nn.functional.silu(t).float().numpy()
    assert np.array_equal(O.activation_only(g, "silu"), silu)
    relu2 = torch.square(torch.nn.functional.relu(t)).float().numpy()
    got = O.activation_only(g, "relu2")
    assert np.array_equal(got, relu2) and (got[g < 0] == 0).all() and np.isinf(got[g > 2e19]).all()
    gelu = torch.nn.functional.gelu(t).float().numpy()
    got = O.activation_only(g, "gelu")
    ok = (np.abs(g) < 1.7e38) & ((np.abs(g) > 2.0**-100) | (g == 0))   # torch's bf16 kernel flushes subnormal results
    assert np.array_equal(got[ok & (g > -3)], gelu[ok & (g > -3)])
    tiny = (np.abs(g) <= 2.0**-100) & (g != 0)
    assert np.array_equal(got[tiny], O.to_bf16((g[tiny] * np.float32(0.5)).astype(np.float32)))   # gelu(v) = v / 2 there
    assert (np.abs(got[ok] - gelu[ok]) <= np.maximum(np.abs(gelu[ok]) * 2.0**-7, np.abs(g[ok]) * 2.0**-22)).all()
    # the gated forms with a second factor of one are the same functions
    one = np.ones_like(g)
    assert np.array_equal(O.silu_and_mul(np.stack([g, one], -1))[:, 0], O.activation_only(g, "silu"))
    assert np.array_equal(O.gelu_and_mul(np.stack([g, one], -1))[:, 0], O.activation_only(g, "gelu"))
    with pytest.raises(ValueError):
        O.activation_only(g, "tanh")


def test_grouped_topk_properties():
    """python/sglang/srt/layers/moe/topk.py:665-738 with the DeepSeek-V3 tuple (256 experts, 8 groups, top-4 groups, top-8)."""
    rng = np.random.default_rng(11)
    logits = rng.standard_normal((50, 256)).astype(np.float32)
    bias = (rng.standard_normal(256) * 0.1).astype(np.float32)
    w, ids = O.biased_grouped_topk(logits, bias, 8, 4, 8)
    assert w.shape == (50, 8) and ids.shape == (50, 8)
    np.testing.assert_allclose(w.sum(-1), 1.0, rtol=1e-5)
    for t in range(50):
        assert len(set(ids[t].tolist())) == 8
        assert len(set((ids[t] // 32).tolist())) <= 4
    # torch restatement of the same selection
    sc = torch.sigmoid(torch.from_numpy(logits))
    scb = sc + torch.from_numpy(bias)
    gs = scb.view(50, 8, 32).topk(2, dim=-1)[0].sum(-1)
    gi = gs.topk(4, dim=-1)[1]
    gm = torch.zeros_like(gs).scatter_(1, gi, 1)
    sm = gm.unsqueeze(-1).expand(50, 8, 32).reshape(50, 256)
    ti = scb.masked_fill(~sm.bool(), float("-inf")).topk(8, dim=-1)[1]
    assert np.array_equal(np.sort(ids, axis=1), np.sort(ti.numpy(), axis=1))


@pytest.mark.parametrize("params", [(128, 4, 2, 4), (256, 8, 4, 8), (512, 16, 8, 16)])
@pytest.mark.parametrize("shared", [0, 1, 2])
@pytest.mark.parametrize("scale_out", [False, True])
def test_moe_fused_gate_oracle_matches_grouped_topk(params, shared, scale_out):
    """The check of the reference's own test (sgl-kernel/tests/test_moe_fused_gate.py:25-101): on float32 inputs
    the fused gate must pick the same expert sets as biased_grouped_topk (here: a torch restatement built from
    library sigmoid / topk / scatter calls) and give the same weights to 1e-2."""
    E, G, tg, topk = params
    rows = 33
    g = torch.Generator().manual_seed(E + shared)
    x = torch.rand((rows, E), generator=g)
    bias = torch.rand((E,), generator=g)
    w, ids = O.moe_fused_gate(x.numpy(), bias.numpy(), G, tg, topk + shared, shared, 2.5, scale_out)
    sc = torch.sigmoid(x)
    scb = sc + bias
    gs = scb.view(rows, G, E // G).topk(2, dim=-1)[0].sum(-1)
    gi = gs.topk(tg, dim=-1)[1]
    gm = torch.zeros_like(gs).scatter_(1, gi, 1)
    sm = gm.unsqueeze(-1).expand(rows, G, E // G).reshape(rows, E)
    ti = scb.masked_fill(~sm.bool(), float("-inf")).topk(topk, dim=-1)[1]
    tw = sc.gather(1, ti)
    routed_sum = tw.sum(-1, keepdim=True)  # topk.py:726-731: the shared entries stay out of the normaliser
    if shared:
        tw = torch.cat([tw] + [routed_sum / 2.5] * shared, dim=1)
        assert np.array_equal(ids[:, topk:], np.tile(np.arange(E, E + shared, dtype=np.int32), (rows, 1)))
    tw = tw / routed_sum
    if scale_out:
        tw = tw * 2.5
    assert np.array_equal(np.sort(ids[:, :topk], axis=1), np.sort(ti.numpy(), axis=1))
    np.testing.assert_allclose(np.sort(w, axis=1), np.sort(tw.numpy(), axis=1), rtol=1e-2, atol=1e-3)
    # routed weights sum to 1, every shared expert carries 1 / routed_scaling_factor (times the factor if applied)
    np.testing.assert_allclose(w.sum(-1), (1.0 + shared / 2.5) * (2.5 if scale_out else 1.0), rtol=1e-5)


def test_moe_fused_gate_oracle_tie_rules():
    """Equal choices: the lower expert wins a place; equal group weights: the higher group is dropped first."""
    x = np.zeros((1, 16), np.float32)
    bias = np.zeros((16,), np.float32)
    w, ids = O.moe_fused_gate(x, bias, 4, 2, 3)
    assert ids[0].tolist() == [0, 1, 2]          # groups 3 and 2 dropped, then experts 0, 1, 2
    np.testing.assert_allclose(w[0], 1.0 / 3.0, rtol=1e-6)


def _bf16_bits_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def _golden():
    import os
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "w8a8_vectors.npz"))


@pytest.mark.parametrize("case", ["a", "b", "c"])
def test_oracle_against_golden_vectors(case):
    """tests/golden/w8a8_vectors.npz was written by torch library ops alone (tests/golden/make_vectors.py)."""
    G = _golden()
    x = _bf16_bits_to_f32(G[case + "_x_bf16_bits"])
    q, s = O.per_token_group_quant_fp8(x, 128)
    assert np.array_equal(q, G[case + "_q"]) and np.array_equal(s, G[case + "_s"])
    y = O.w8a8_block_fp8_matmul(G[case + "_q"], G[case + "_wq"], G[case + "_s"], G[case + "_ws"], out_dtype="f32", acc=np.float64)
    np.testing.assert_allclose(y, G[case + "_y"], rtol=1e-6, atol=1e-30)
    if case == "a":
        wq, ws = O.block_quant_weight(_bf16_bits_to_f32(G["a_w_bf16_bits"]))
        assert np.array_equal(wq, G["a_wq"]) and np.array_equal(ws, G["a_ws"])


# ---------------------------------------------------------------- composites: linear with bias, fused MoE, bf16 gate
def _t_group_quant(x_bf16):
    """Per-token-group quant as a chain of torch library ops on a bf16 tensor (the arithmetic of
    python/sglang/test/test_block_fp8.py:23-48, written against the library, not against the oracle)."""
    g = x_bf16.reshape(-1, 128)
    amax = g.abs().amax(dim=-1, keepdim=True).clamp(min=1e-10).to(torch.float32)
    s = amax / 448.0
    q = torch.clamp(g / s, -448.0, 448.0).to(torch.float8_e4m3fn)
    return q.reshape(x_bf16.shape), s.reshape(x_bf16.shape[0], -1)


def _t_block_matmul_f64(q, s, wq, ws):
    """Dequantise with broadcast scales and multiply in float64 (sgl-kernel/tests/test_fp8_blockwise_gemm.py:19-59)."""
    a = q.to(torch.float64) * s.to(torch.float64).repeat_interleave(128, dim=1)
    b = wq.to(torch.float64) * ws.to(torch.float64).repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
    return a @ b.t()


def test_block_fp8_linear_bias_branch_and_nd_input():
    """python/sglang/srt/layers/quantization/fp8_utils.py:306-326: the bias is added to the bf16 GEMM result with a
    bf16 tensor add (one more rounding), and leading dimensions are flattened and restored."""
    x = O.make_activation(12, 512, 21).reshape(3, 4, 512)
    wq, ws = O.block_quant_weight(O.make_weight(256, 512, 21))
    bias = O.to_bf16(np.random.default_rng(21).standard_normal(256).astype(np.float32))
    plain = O.block_fp8_linear(x, wq, ws)
    got = O.block_fp8_linear(x, wq, ws, bias)
    assert plain.shape == got.shape == (3, 4, 256)
    ref = (torch.from_numpy(plain).bfloat16() + torch.from_numpy(bias).bfloat16()).float().numpy()
    assert np.array_equal(got, ref)
    assert not np.array_equal(got, plain + bias)  # the second rounding is visible on this data
    # the flattened problem gives the same rows
    assert np.array_equal(O.block_fp8_linear(x.reshape(12, 512), wq, ws, bias), got.reshape(12, 256))
    # and the un-biased result is the torch-ops pipeline's, up to float32-vs-float64 summation at bf16 ties
    q, s = _t_group_quant(torch.from_numpy(x.reshape(12, 512)).bfloat16())
    y = _t_block_matmul_f64(q, s, torch.from_numpy(wq).view(torch.float8_e4m3fn), torch.from_numpy(ws))
    y = y.to(torch.float32).bfloat16().float().numpy()
    assert (y == plain.reshape(12, 256)).mean() > 0.995
    assert np.abs(y - plain.reshape(12, 256)).max() <= 2.0**-7 * np.abs(y).max()


@pytest.mark.parametrize("T,E,H,I,topk,rsf,activation", [(20, 4, 256, 128, 2, 2.5, "silu"), (33, 8, 384, 256, 3, 1.0, "silu"),
                                                         (20, 4, 256, 128, 2, 2.5, "gelu"), (20, 4, 256, 128, 2, 2.5, "relu2")])
def test_fused_moe_composite_against_torch_ops_pipeline(T, E, H, I, topk, rsf, activation):
    """fused_moe_block_fp8 against the same layer spelled with torch library ops, expert by expert as
    torch_w8a8_block_fp8_moe does (python/sglang/test/test_block_fp8.py:418-447), with the roundings of the fused
    path (fused_moe.py:498-639): GEMM1 -> bf16, silu -> bf16 -> times up -> bf16, requant, GEMM2 times the routed
    weight in float32 -> bf16, float32 sum over the top-k in ascending k times routed_scaling_factor -> bf16.
    The GEMMs run in float64 here and in float32 tile sums in the oracle, so a result that sits within a float32 ulp
    of a bf16 tie may round the other way; everything else must agree bit for bit."""
    rng = np.random.default_rng(T + E)
    x = O.make_activation(T, H, T)
    gated = activation != "relu2"     # relu2: experts without a gate projection (fused_moe.py:566-572), w13 is [E, I, H]
    n1 = 2 * I if gated else I
    kw = dict(activation=activation, is_gated=gated)
    w13q = np.empty((E, n1, H), np.uint8); w13s = np.empty((E, n1 // 128, H // 128), np.float32)
    w2q = np.empty((E, H, I), np.uint8); w2s = np.empty((E, H // 128, I // 128), np.float32)
    for e in range(E):
        w13q[e], w13s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((n1, H)).astype(np.float32) * 0.05))
        w2q[e], w2s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((H, I)).astype(np.float32) * 0.05))
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    ids[rng.random(ids.shape) < 0.1] = -1          # experts on another rank contribute nothing
    tw = rng.uniform(0.1, 1.0, (T, topk)).astype(np.float32)
    got = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, rsf, **kw)
    got_in = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, rsf, apply_router_weight_on_input=True, **kw)
    act_fn = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu2": None}[activation]

    xt = torch.from_numpy(x).bfloat16()
    xq, xs = _t_group_quant(xt)
    t_ids, t_w = torch.from_numpy(ids), torch.from_numpy(tw)

    def torch_pipeline(weight_on_input):
        per_slot = torch.zeros((T, topk, H), dtype=torch.bfloat16)
        for e in range(E):
            tok, slot = torch.nonzero(t_ids == e, as_tuple=True)
            if tok.numel() == 0:
                continue
            W1, S1 = torch.from_numpy(w13q[e]).view(torch.float8_e4m3fn), torch.from_numpy(w13s[e])
            W2, S2 = torch.from_numpy(w2q[e]).view(torch.float8_e4m3fn), torch.from_numpy(w2s[e])
            wk = t_w[tok, slot].unsqueeze(1)
            h1 = _t_block_matmul_f64(xq[tok].float(), xs[tok], W1, S1).to(torch.float32)
            h1 = (h1 * wk if weight_on_input else h1).bfloat16()
            act = act_fn(h1[:, :I].float()).bfloat16() * h1[:, I:] if gated else torch.square(torch.relu(h1))
            aq, a_s = _t_group_quant(act)
            h2 = _t_block_matmul_f64(aq.float(), a_s, W2, S2).to(torch.float32)
            per_slot[tok, slot] = (h2 if weight_on_input else h2 * wk).bfloat16()
        acc = torch.zeros((T, H), dtype=torch.float32)
        for k in range(topk):
            acc = acc + per_slot[:, k].float()
        return (acc * rsf).bfloat16().float().numpy()

    ref = torch_pipeline(False)
    assert got.shape == ref.shape == (T, H)
    assert (got == ref).mean() > 0.99, (got == ref).mean()
    assert np.abs(got - ref).max() <= 2.0**-6 * np.abs(ref).max()
    # the routed weight on the result of GEMM 1 instead (fused_moe.py:533,597): another function of the same inputs
    ref_in = torch_pipeline(True)
    assert (got_in == ref_in).mean() > 0.99, (got_in == ref_in).mean()
    assert np.abs(got_in - ref_in).max() <= 2.0**-6 * np.abs(ref_in).max()
    assert not np.allclose(got_in, got, rtol=1e-2)
    # rows whose every expert is absent are exactly zero
    dead = (ids == -1).all(axis=1)
    assert (got[dead] == 0).all()
    # what a plausible mistake would change: no routed weight, weight applied after the sum, no scaling factor
    assert not np.allclose(got, O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, np.ones_like(tw), ids, rsf, **kw), rtol=1e-2)
    if rsf != 1.0:
        assert not np.allclose(got, O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, 1.0, **kw), rtol=1e-2)
    if activation != "silu":
        other = dict(kw, activation="silu")
        assert not np.allclose(got, O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, rsf, **other), rtol=1e-2)


def _t_fused_gate_bf16(x, bias, G, topk_group, topk):
    """The gate of sgl-kernel/csrc/moe/moe_fused_gate.cu:52-257 with bf16 tensors and torch library ops: every
    intermediate (sigmoid, score + bias, the sum of a group's two best) is a bf16 tensor; the weakest group is
    dropped repeatedly (ties: the higher group), the best expert taken repeatedly (ties: the lower expert;
    torch.argmax returns the first maximum)."""
    rows, E = x.shape
    score = torch.sigmoid(x)                                # bf16 in, bf16 out
    choice = (score + bias).reshape(rows, G, E // G).clone()
    for _ in range(G - topk_group):
        top2 = choice.float().topk(2, dim=-1)[0].bfloat16()
        sums = (top2[..., 0] + top2[..., 1]).float()
        sums = torch.where(torch.isinf(sums), torch.full_like(sums, float("inf")), sums)
        worst = (G - 1) - torch.argmin(sums.flip(-1), dim=-1)   # last minimum = highest group among equals
        choice[torch.arange(rows), worst] = float("inf")
    flat = choice.float().reshape(rows, E)
    flat = torch.where(flat == float("inf"), torch.full_like(flat, float("-inf")), flat)
    ids = torch.empty((rows, topk), dtype=torch.int64)
    for k in range(topk):
        ids[:, k] = torch.argmax(flat, dim=-1)
        flat[torch.arange(rows), ids[:, k]] = float("-inf")
    w = score.float().gather(1, ids)
    return (w / w.sum(-1, keepdim=True)).numpy(), ids.numpy().astype(np.int32)


@pytest.mark.parametrize("E,G,tg,topk", [(256, 8, 4, 8), (128, 4, 2, 4)])
def test_moe_fused_gate_bf16_branch_against_torch_bf16_ops(E, G, tg, topk):
    """in_dtype="bf16": the oracle's rounding points against bf16 tensor arithmetic.  bf16 scores tie often, so
    the tie rules are exercised on every row."""
    g = torch.Generator().manual_seed(E)
    x = torch.randn((200, E), generator=g).bfloat16()
    bias = (torch.randn((E,), generator=g) * 0.1).bfloat16()
    w, ids = O.moe_fused_gate(x.float().numpy(), bias.float().numpy(), G, tg, topk, in_dtype="bf16")
    w_ref, ids_ref = _t_fused_gate_bf16(x, bias, G, tg, topk)
    # torch's bf16 sigmoid and numpy's float32 exp can differ in the last float32 bit, which moves a bf16 score only
    # at a tie: allow a handful of rows to differ, as sets they must still agree on all but those
    same = (ids == ids_ref).all(axis=1)
    assert same.mean() >= 0.98, same.mean()
    np.testing.assert_allclose(w[same], w_ref[same], rtol=1e-6, atol=1e-7)
    # the bf16 rounding matters: the float32 gate picks other experts on some rows of the same data
    _, ids32 = O.moe_fused_gate(x.float().numpy(), bias.float().numpy(), G, tg, topk, in_dtype="f32")
    assert (ids32 != ids).any()


def test_per_tensor_quant_mla_against_torch_ops_and_closed_form():
    """per_tensor_quant_mla_fp8 (fp8_kernel.py:1172-1266) restated with torch ops on a transposed bf16 view: per-row
    max(absmax, eps) / 448, the maximum of those, x * (1 / s) clamped and converted by torch's e4m3fn cast."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(24, 6, 128, generator=g) * 3).to(torch.bfloat16).transpose(0, 1)  # [H=6, S=24, D=128], strided
    rows = x.float().abs().amax(-1).clamp(min=1e-12) / 448.0
    s = rows.max()
    q = (x.float() * (1.0 / s)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    oq, os_ = O.per_tensor_quant_mla_fp8(x.float().numpy())
    assert os_.shape == (1,) and os_[0] == np.float32(s.item())
    assert np.array_equal(oq, q.view(torch.uint8).numpy())
    # closed forms: the element of largest magnitude lands on +-448; an all-zero tensor gets eps / 448 and zero bytes
    y = np.zeros((2, 3, 16), np.float32)
    y[1, 2, 5] = -7.0
    y[0, 0, 0] = 3.5
    q2, s2 = O.per_tensor_quant_mla_fp8(y)
    assert s2[0] == np.float32(7.0) / np.float32(448.0)
    assert O.e4m3fn_to_f32(q2)[1, 2, 5] == -448.0 and O.e4m3fn_to_f32(q2)[0, 0, 0] == 224.0
    q3, s3 = O.per_tensor_quant_mla_fp8(np.zeros((1, 2, 8), np.float32))
    assert s3[0] == np.float32(1e-12) / np.float32(448.0) and not q3.any()


def test_bmm_fp8_against_torch_bmm_and_brute_force():
    """bmm_fp8 the way sgl-kernel/tests/test_bmm_fp8.py checks it: torch.bmm of the de-quantised operands (float64 here),
    times both scales; plus a triple loop on a tiny case, which a transposed operand or a dropped scale would fail."""
    rng = np.random.default_rng(5)
    b, m, n, k = 3, 5, 7, 16
    aq = rng.integers(0, 0x70, (b, m, k), dtype=np.uint8) | (rng.integers(0, 2, (b, m, k), dtype=np.uint8) << 7)
    bq = rng.integers(0, 0x70, (b, n, k), dtype=np.uint8) | (rng.integers(0, 2, (b, n, k), dtype=np.uint8) << 7)
    sa, sb = np.float32(0.0123), np.float32(0.25)
    got = O.bmm_fp8(aq, bq, sa, sb, "f32")
    A = torch.from_numpy(aq).view(torch.float8_e4m3fn).double()
    B = torch.from_numpy(bq).view(torch.float8_e4m3fn).double().transpose(1, 2)  # [b, k, n] column-major, as the op takes it
    ref = (torch.bmm(A, B) * float(sa) * float(sb)).numpy()
    assert np.allclose(got, ref, rtol=1e-6, atol=0)
    brute = np.zeros((b, m, n))
    a_f, b_f = O.e4m3fn_to_f32(aq).astype(np.float64), O.e4m3fn_to_f32(bq).astype(np.float64)
    for i in range(b):
        for r in range(m):
            for c in range(n):
                brute[i, r, c] = sum(a_f[i, r, t] * b_f[i, c, t] for t in range(k)) * float(sa) * float(sb)
    assert np.allclose(got, brute, rtol=1e-6, atol=0)
    assert np.array_equal(O.bmm_fp8(aq, bq, sa, sb, "bf16"), O.to_bf16(got))


def test_prepare_moe_input_against_stable_argsort_and_bincount():
    """The expert-major sort restated with numpy library routines: bincount for the row counts, a stable argsort for
    the order; c_map must invert a_map's placement, and ids outside [0, E) take no row."""
    rng = np.random.default_rng(4)
    m, topk, E, n, k = 37, 4, 9, 256, 384
    ids = rng.integers(0, E, (m, topk)).astype(np.int32)
    ids[5, 2] = -1
    ids[6, 0] = E
    off, bso, ps1, ps2, a_map, c_map = O.prepare_moe_input(ids, E, n, k)
    flat = ids.reshape(-1)
    valid = (flat >= 0) & (flat < E)
    counts = np.bincount(flat[valid], minlength=E)
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(counts)]))
    assert np.array_equal(bso, np.concatenate([[0], np.cumsum((counts + 127) // 128 * 128)]))
    assert np.array_equal(ps1, np.stack([counts, np.full(E, 2 * n), np.full(E, k)], 1))
    assert np.array_equal(ps2, np.stack([counts, np.full(E, k), np.full(E, n)], 1))
    order = np.argsort(np.where(valid, flat, E), kind="stable")[: valid.sum()]  # slots by expert, ties in slot order
    assert np.array_equal(a_map[: valid.sum()], order // topk)
    assert np.array_equal(c_map[order], np.arange(valid.sum()))


def test_apply_shuffle_mul_sum_against_the_torch_expression():
    """The reference documents the op as (c2[c_map].view(m, topk, k) * topk_weights.view(m, topk, 1)).sum(dim=1)
    (prepare_moe_input.cu:369-386), computed in float32 and rounded once: in float64 here, one bf16 ulp of slack."""
    g = torch.Generator().manual_seed(8)
    m, topk, k = 13, 6, 40
    c2 = torch.randn(m * topk, k, generator=g).to(torch.bfloat16)
    w = torch.rand(m, topk, generator=g).to(torch.bfloat16)
    c_map = torch.randperm(m * topk, generator=g)
    ref = (c2.double()[c_map].view(m, topk, k) * w.double().view(m, topk, 1)).sum(dim=1)
    got = O.apply_shuffle_mul_sum(c2.float().numpy(), c_map.view(m, topk).numpy(), w.float().numpy(), "bf16")
    assert np.array_equal(got, O.to_bf16(got))
    err = np.abs(got - ref.numpy())
    assert (err <= np.abs(ref.numpy()) * 2.0 ** -8 + 1e-30).all()
    # no factors: a plain gather-sum, exact in float32 for small integers
    ints = torch.randint(-8, 8, (m * topk, k), generator=g).float()
    got2 = O.apply_shuffle_mul_sum(ints.numpy(), c_map.view(m, topk).numpy(), None, "f32")
    assert np.array_equal(got2, ints[c_map].view(m, topk, k).sum(1).numpy())


def test_grouped_mm_and_cutlass_composite():
    """The grouped GEMM against torch.mm of the de-quantised operands per expert (the check of sgl-kernel/tests/
    test_fp8_blockwise_moe.py:66-91), and the expert-major fused experts against the Triton-ordered composite: the
    same mathematics with the routed weight applied at a different rounding point."""
    rng = np.random.default_rng(6)
    E, N, K = 3, 256, 384
    sizes = [5, 0, 9]
    rows = sum(sizes)
    aq = rng.integers(0, 0x60, (rows, K), dtype=np.uint8) | (rng.integers(0, 2, (rows, K), dtype=np.uint8) << 7)
    bq = rng.integers(0, 0x60, (E, N, K), dtype=np.uint8) | (rng.integers(0, 2, (E, N, K), dtype=np.uint8) << 7)
    a_s = rng.uniform(0.5, 2.0, (rows, K // 128)).astype(np.float32) * 1e-2
    b_s = rng.uniform(0.5, 2.0, (E, N // 128, K // 128)).astype(np.float32) * 1e-2
    off = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    ps = np.array([[c, N, K] for c in sizes], dtype=np.int32)
    got = O.fp8_blockwise_scaled_grouped_mm(aq, bq, a_s, b_s, off, ps, "f32", acc=np.float64)
    A = torch.from_numpy(aq).view(torch.float8_e4m3fn).double() * torch.from_numpy(a_s).double().repeat_interleave(128, 1)
    for e in range(E):
        B = torch.from_numpy(bq[e]).view(torch.float8_e4m3fn).double() * \
            torch.from_numpy(b_s[e]).double().repeat_interleave(128, 0).repeat_interleave(128, 1)
        ref = torch.mm(A[off[e]:off[e + 1]], B.t()).numpy()
        assert np.allclose(got[off[e]:off[e + 1]], ref, rtol=1e-5, atol=1e-7)

    T, E, H, I, topk = 24, 6, 256, 128, 2
    x = O.make_activation(T, H, 3)
    w13q = np.empty((E, 2 * I, H), np.uint8); w13s = np.empty((E, 2 * I // 128, H // 128), np.float32)
    w2q = np.empty((E, H, I), np.uint8); w2s = np.empty((E, H // 128, I // 128), np.float32)
    for e in range(E):
        w13q[e], w13s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((2 * I, H)).astype(np.float32) * 0.05))
        w2q[e], w2s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((H, I)).astype(np.float32) * 0.05))
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    tw = O.to_bf16(rng.uniform(0.1, 1.0, (T, topk)).astype(np.float32))
    a = O.cutlass_fused_experts_fp8(x, w13q, w13s, w2q, w2s, tw, ids)
    b = O.fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, tw, ids, 1.0)
    assert np.abs(a - b).max() <= 2e-2 * np.abs(b).max()
