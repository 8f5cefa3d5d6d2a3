"""GPU parity of the quantisation kernels against the CPU oracle: bytes and scales bit-exact."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import bf16_tensor, u8

pytestmark = pytest.mark.gpu


def _layouts():
    # (column_major, tma_aligned, ue8m0)
    return [(False, False, False), (True, False, False), (True, True, False), (True, True, True)]


def _run_group_quant(x_np, dev, group, layout, dtype=torch.bfloat16, eps=1e-10):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    cm, al, ue = layout
    x = torch.from_numpy(x_np).to(dtype).to(dev)
    q, s = sglang_per_token_group_quant_fp8(x, group, eps=eps, column_major_scales=cm, scale_tma_aligned=al, scale_ue8m0=ue)
    torch.cuda.synchronize()
    return q, s


def _check(x_np, dev, group, layout, in_dtype="bf16", dtype=torch.bfloat16, eps=1e-10):
    cm, al, ue = layout
    q, s = _run_group_quant(x_np, dev, group, layout, dtype, eps)
    q_ref, s_ref = O.per_token_group_quant_fp8(x_np, group, eps=eps, in_dtype=in_dtype, scale_ue8m0=ue)
    M, K = x_np.shape
    assert q.shape == (M, K) and q.dtype == torch.float8_e4m3fn
    np.testing.assert_array_equal(u8(q), q_ref)
    G = K // group
    if ue:
        assert s.dtype == torch.int32 and s.shape == (M, (G + 3) // 4)
        assert s.stride(0) == 1 and s.stride(1) == (M + 3) // 4 * 4
        np.testing.assert_array_equal(s.cpu().numpy(), O.pack_ue8m0_scales(s_ref))
    else:
        assert s.dtype == torch.float32 and s.shape == (M, G)
        if cm:
            assert s.stride(0) == 1 and s.stride(1) == ((M + 3) // 4 * 4 if al else M)
        else:
            assert s.is_contiguous()
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))


@pytest.mark.parametrize("layout", _layouts())
@pytest.mark.parametrize("M", [1, 3, 31, 32, 33, 64, 257, 512])
def test_group_quant_config_shapes_small(dev, M, layout):
    x = O.make_activation(M, 7168, seed=M)
    _check(x, dev, 128, layout)


@pytest.mark.parametrize("layout", _layouts())
@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4])
def test_group_quant_sweep_4096(dev, seed, layout):
    x = O.make_activation(4096, 7168, seed=seed)
    _check(x, dev, 128, layout)


@pytest.mark.parametrize("layout", [(False, False, False), (True, False, False), (True, True, True)])
@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("M", [1, 64, 512])
def test_group_quant_sweep_small_sizes_every_seed(dev, M, seed, layout):
    """The bandwidth sweep's sizes below 4096 rows with each of its five seeds and three scale layouts (row-major
    float, column-major float, packed UE8M0)."""
    _check(O.make_activation(M, 7168, seed=seed), dev, 128, layout)


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4])
def test_group_quant_16384_every_layout(dev, seed):
    """The largest size of the bandwidth sweep (bf16 [16384, 7168]) with each of its five seeds, in all four scale
    layouts.  At this size the expected bytes and scales come from the C restatement of the oracle (OpenMP), which
    tests/test_oracle.py holds bit for bit against the numpy one."""
    from oracle import c_oracle

    M, K, G = 16384, 7168, 56
    x = O.make_activation(M, K, seed=seed)
    lib = c_oracle.load()
    eps = float(O.clamp_eps(1e-10, "bf16"))
    refs = {ue: c_oracle.group_quant_bf16(lib, O.bf16_bits(x), 128, eps, ue) for ue in (False, True)}
    for layout in _layouts():
        cm, al, ue = layout
        q_ref, s_ref = refs[ue]
        q, s = _run_group_quant(x, dev, 128, layout)
        assert torch.equal(q.view(torch.uint8).cpu(), torch.from_numpy(q_ref)), layout
        if ue:
            assert s.dtype == torch.int32 and s.shape == (M, G // 4) and s.stride() == (1, M)
            np.testing.assert_array_equal(s.cpu().numpy(), O.pack_ue8m0_scales(s_ref))
        else:
            assert s.shape == (M, G) and (s.stride() == (1, M) if cm else s.is_contiguous())
            np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))


@pytest.mark.parametrize("group", [16, 32, 64, 128, 256, 512])
@pytest.mark.parametrize("K", [512, 1536, 4096])
def test_group_sizes(dev, group, K):
    x = O.make_activation(83, K, seed=group + K)
    _check(x, dev, group, (False, False, False))
    _check(x, dev, group, (True, False, False))


@pytest.mark.parametrize("K", [128, 256, 384, 640, 2304])
def test_ragged_group_counts(dev, K):
    # K/128 not a multiple of 4: the last wave strip is partly empty, packed words have zero bytes
    x = O.make_activation(45, K, seed=K)
    for layout in _layouts():
        _check(x, dev, 128, layout)


def test_every_bf16_amax(dev):
    """Scale table over every positive finite bf16 amax (32 639 values) and the eps floor."""
    bits = np.arange(1, 0x7F80, dtype=np.uint32)
    amax = (bits << 16).view(np.float32)
    M = amax.size
    rng = np.random.default_rng(5)
    x = (rng.uniform(-1, 1, (M, 128)).astype(np.float32) * amax[:, None]).astype(np.float32)
    x = O.to_bf16(x)
    x[:, 7] = amax  # the group amax is exactly the table value
    x = np.clip(x, -amax[:, None], amax[:, None])
    for layout in _layouts():
        _check(x, dev, 128, layout)


@pytest.mark.parametrize("name,dtype", [("bf16", torch.bfloat16), ("f16", torch.float16)])
def test_exact_scale_groups_are_full_of_ties(dev, name, dtype):
    """When the amax mantissa is a multiple of 7, amax/448 is exact and x/scale lands exactly on fp8 rounding
    ties for many x (0.5 % of real activations): every such amax, against every mantissa of x over a range
    of exponents, must follow round-half-to-even exactly as the float32 divide + cast does."""
    if name == "bf16":
        mant_bits, to_dt = 7, O.to_bf16
    else:
        mant_bits, to_dt = 10, lambda v: v.astype(np.float16).astype(np.float32)
    specials = [m for m in range(1 << mant_bits, 2 << mant_bits) if m % 7 == 0]
    rows = []
    for m in specials:
        amax = np.float32(m) / np.float32(1 << mant_bits)  # in [1, 2)
        xm = np.arange(1 << mant_bits, 2 << mant_bits, dtype=np.float32) / np.float32(1 << mant_bits)
        xm = xm[:: max(1, xm.size // 128)][:128]
        for e in range(0, 9):  # x = mantissa * 2^-e, below amax
            g = (xm * np.float32(2.0 ** -e)).astype(np.float32)
            g = np.where(g > amax, g / 2, g)
            g[::2] *= -1
            g[5] = amax
            rows.append(to_dt(g))
    x = np.stack(rows).astype(np.float32)
    vals = O.e4m3fn_to_f32(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)
    mids = (vals[:-1] + vals[1:]) / 2
    y = np.abs(x.astype(np.float64)) / (np.abs(x).max(-1, keepdims=True).astype(np.float64) / 448.0)
    ties = int(np.isin(y, mids).sum())  # exact half-way cases in this input
    assert ties > 300
    for layout in _layouts():
        _check(x, dev, 128, layout, in_dtype=name, dtype=dtype)


def test_structural_ties_for_every_bf16_amax_mantissa(dev):
    """x = amax * t * 2^i / 448 (whenever that is a bf16 number) makes 448 x / amax exactly the rounding boundary
    t * 2^i of the cast, for every amax mantissa - including those whose scale amax/448 is inexact, where the
    reference's result depends on how the scale was rounded (boundaries 21 * 2^i and, among fp8 subnormals,
    7 * 2^-10).  Both signs, three amax exponents."""
    rows = []
    for ma in range(128, 256):
        for ea in (-3, 0, 5):
            amax = np.float32(ma) * np.float32(2.0 ** (ea - 7))
            vals = np.array([np.float64(amax) * t * 2.0**i / 448.0 for i in range(-18, 1) for t in range(1, 32, 2)])
            vb = O.to_bf16(vals.astype(np.float32))
            vb = vb[(vb.astype(np.float64) == vals) & (np.abs(vb) <= amax)][:127]
            g = np.zeros(128, np.float32)
            g[0] = amax
            g[1 : 1 + vb.size] = vb * np.where(np.arange(vb.size) % 2 == 0, 1, -1)
            rows.append(g)
    x = np.stack(rows)
    for layout in _layouts():
        _check(x, dev, 128, layout)


def test_zero_groups_and_closed_form(dev):
    # all-zero groups: q = 0, scale = bf16(eps)/448; amax = 448 -> scale 1, bytes = encode(x)
    x = np.zeros((8, 256), dtype=np.float32)
    x[1, :128] = O.to_bf16(np.linspace(-448, 448, 128).astype(np.float32))
    x[1, 0] = 448.0
    x[2, 128:] = -0.0
    q, s = _run_group_quant(x, dev, 128, (False, False, False))
    s = s.cpu().numpy()
    assert s[1, 0] == 1.0
    np.testing.assert_array_equal(u8(q)[1, :128], O.f32_to_e4m3fn(x[1, :128]))
    assert s[0, 0] == np.float32(O.clamp_eps(1e-10, "bf16")) / np.float32(448)
    assert (u8(q)[0] == 0).all() and (u8(q)[2, 128:] == 0x80).all()
    for layout in _layouts():
        _check(x, dev, 128, layout)


@pytest.mark.parametrize("dtype,name", [(torch.float16, "f16"), (torch.float32, "f32")])
def test_other_input_dtypes(dev, dtype, name):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((130, 1024)).astype(np.float32) * 3
    if name == "f16":
        x = x.astype(np.float16).astype(np.float32)
    x[5, :128] = 0
    for layout in _layouts():
        _check(x, dev, 128, layout, in_dtype=name, dtype=dtype)


def test_every_f16_amax(dev):
    bits = np.arange(1, 0x7C00, dtype=np.uint16)
    amax = bits.view(np.float16).astype(np.float32)
    x = np.zeros((amax.size, 128), dtype=np.float32)
    x[:, 3] = -amax
    x[:, 9] = (amax.astype(np.float16) * np.float16(0.37)).astype(np.float32)
    _check(x, dev, 128, (False, False, False), in_dtype="f16", dtype=torch.float16)


def test_quant_leaves_neighbours_untouched(dev):
    """Poisoned output buffers: only the declared elements are written (padded column-major rows too)."""
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_8bit

    M, K = 45, 640
    x = bf16_tensor(O.make_activation(M, K, 3), dev)
    qbuf = torch.full((M + 2, K), 0x55, dtype=torch.uint8, device=dev)
    sbuf = torch.full((K // 128 + 2, 48), -7.0, dtype=torch.float32, device=dev)
    q = qbuf[1 : M + 1].view(torch.float8_e4m3fn)
    s = sbuf[1 : 1 + K // 128].t()[:M]
    sgl_per_token_group_quant_8bit(x, q, s, 128, 1e-10, -448.0, 448.0)
    torch.cuda.synchronize()
    assert (qbuf[0] == 0x55).all() and (qbuf[-1] == 0x55).all()
    assert (sbuf[0] == -7).all() and (sbuf[-1] == -7).all() and (sbuf[:, M:] == -7).all()
    q_ref, s_ref = O.per_token_group_quant_fp8(x.float().cpu().numpy(), 128)
    np.testing.assert_array_equal(u8(q), q_ref)
    np.testing.assert_array_equal(s.cpu().numpy(), s_ref)


def test_empty_and_errors(dev):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_8bit

    q, s = sglang_per_token_group_quant_fp8(torch.empty((0, 256), dtype=torch.bfloat16, device=dev), 128)
    assert q.shape == (0, 256) and s.shape == (0, 2)
    x = torch.zeros((4, 256), dtype=torch.bfloat16, device=dev)
    qo = torch.empty((4, 256), dtype=torch.float8_e4m3fn, device=dev)
    with pytest.raises(RuntimeError):
        sgl_per_token_group_quant_8bit(x, qo, torch.empty((4, 2), device=dev), 96, 1e-10, -448.0, 448.0)
    with pytest.raises(RuntimeError):
        sgl_per_token_group_quant_8bit(x, qo, torch.empty((8,), device=dev), 128, 1e-10, -448.0, 448.0)
    with pytest.raises(RuntimeError):
        sgl_per_token_group_quant_8bit(x, qo, torch.empty((4, 2), device=dev), 128, 1e-10, -224.0, 224.0)
    with pytest.raises(RuntimeError):
        sgl_per_token_group_quant_8bit(x.t(), qo, torch.empty((4, 2), device=dev), 128, 1e-10, -448.0, 448.0)
    with pytest.raises(AssertionError):
        sglang_per_token_group_quant_fp8(x, 100)


@pytest.mark.parametrize("M,K", [(1, 4096), (7, 4096), (512, 14336), (2048, 4096), (33, 24576)])
def test_per_token_quant(dev, M, K):
    from sglang_amd.fp8_kernel import sglang_per_token_quant_fp8

    x = O.make_activation(M, K, seed=M + K)
    if M > 3:
        x[3] = 0
    q, s = sglang_per_token_quant_fp8(bf16_tensor(x, dev))
    torch.cuda.synchronize()
    q_ref, s_ref = O.per_token_quant_fp8(x)
    assert s.shape == (M, 1)
    np.testing.assert_array_equal(s.cpu().numpy(), s_ref)
    np.testing.assert_array_equal(u8(q), q_ref)


@pytest.mark.parametrize("numel", [8, 1000, 4096 * 7168 + 5])
def test_per_tensor_quant(dev, numel):
    from sglang_amd.fp8_kernel import scaled_fp8_quant

    rng = np.random.default_rng(numel)
    cols = 8 if numel % 8 == 0 else 1
    x = O.to_bf16(rng.standard_normal(numel).astype(np.float32) * 4).reshape(-1, cols)
    xt = bf16_tensor(x, dev)
    q, s = scaled_fp8_quant(xt)
    torch.cuda.synchronize()
    q_ref, s_ref = O.per_tensor_quant_fp8(x)
    np.testing.assert_array_equal(s.cpu().numpy(), s_ref)
    np.testing.assert_array_equal(u8(q), q_ref)
    st = torch.tensor([0.05], dtype=torch.float32, device=dev)
    q2, s2 = scaled_fp8_quant(xt, st)
    q2_ref, _ = O.per_tensor_quant_fp8(x, 0.05)
    np.testing.assert_array_equal(u8(q2), q2_ref)


@pytest.mark.parametrize("shape", [(5, 7, 64), (300, 2048), (1, 8)])
def test_static_quant_fp8(dev, shape):
    """static_quant_fp8 (reference: fp8_kernel.py:639-692): bytes of the oracle's static per-tensor quant, the scale handed
    back as given or once per row."""
    from sglang_amd.fp8_kernel import static_quant_fp8

    rng = np.random.default_rng(sum(shape))
    x = O.to_bf16(rng.standard_normal(shape).astype(np.float32) * 6)
    st = torch.tensor([0.037], dtype=torch.float32, device=dev)
    q, s = static_quant_fp8(bf16_tensor(x, dev), st)
    q_ref, _ = O.per_tensor_quant_fp8(x.reshape(-1, shape[-1]), 0.037)
    np.testing.assert_array_equal(u8(q).reshape(-1, shape[-1]), q_ref)
    assert s is st
    q2, s2 = static_quant_fp8(bf16_tensor(x, dev), st, repeat_scale=True)
    np.testing.assert_array_equal(u8(q2).reshape(-1, shape[-1]), q_ref)
    rows = int(np.prod(shape[:-1]))
    assert s2.shape == (rows, 1) and bool((s2 == st).all())


def test_group_quant_8bit_entry_points(dev):
    """sglang_per_token_group_quant_8bit / per_token_group_quant_8bit (reference: fp8_kernel.py:404-434, 535-574) are the
    FP8 group quant under the 8-bit names; the int8 destination is refused."""
    from sglang_amd.fp8_kernel import per_token_group_quant_8bit, sglang_per_token_group_quant_8bit, sglang_per_token_group_quant_fp8

    x = bf16_tensor(O.make_activation(33, 512, 2), dev)
    q0, s0 = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
    for fn in (sglang_per_token_group_quant_8bit, per_token_group_quant_8bit):
        q, s = fn(x, 128, torch.float8_e4m3fn, column_major_scales=True)
        assert torch.equal(q.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(s, s0) and s.stride() == s0.stride()
        with pytest.raises(RuntimeError, match="float8_e4m3fn"):
            fn(x, 128, torch.int8)


@pytest.mark.parametrize("layout", _layouts())
@pytest.mark.parametrize("M,K", [(1, 128), (37, 2048), (512, 2048), (4096, 2048)])
def test_silu_mul_group_quant_equals_the_two_step_pipeline(dev, M, K, layout):
    """fuse_silu_and_mul (reference: per_token_group_quant_8bit_v2.cu:336-341): the bytes and scales must equal
    silu_and_mul followed by the group quant, bit for bit - against this library's two kernels, and against
    the oracle's quant applied to the 16-bit values that silu_and_mul produced (the silu itself is compared
    with the oracle, to one bf16 ulp because of expf, in the MoE tests)."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import silu_and_mul

    cm, al, ue = layout
    kw = dict(column_major_scales=cm, scale_tma_aligned=al, scale_ue8m0=ue)
    x = torch.from_numpy(O.make_activation(M, 2 * K, seed=M + K)).to(dev).to(torch.bfloat16)
    q, s = sglang_per_token_group_quant_fp8(x, 128, fuse_silu_and_mul=True, **kw)
    mid = torch.empty((M, K), device=dev, dtype=torch.bfloat16)
    silu_and_mul(x, mid)
    q2, s2 = sglang_per_token_group_quant_fp8(mid, 128, **kw)
    torch.cuda.synchronize()
    assert q.shape == (M, K) and s.shape == s2.shape and s.stride() == s2.stride()
    np.testing.assert_array_equal(u8(q), u8(q2))
    if kw.get("scale_ue8m0"):
        assert torch.equal(s, s2)
    else:
        assert torch.equal(s.contiguous().view(torch.int32), s2.contiguous().view(torch.int32))
    q_ref, s_ref = O.per_token_group_quant_fp8(mid.float().cpu().numpy(), 128, scale_ue8m0=bool(kw.get("scale_ue8m0")))
    np.testing.assert_array_equal(u8(q), q_ref)


def test_silu_mul_group_quant_other_dtypes_and_errors(dev):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import silu_and_mul

    for dt in (torch.float16, torch.float32):
        x = (torch.randn((65, 512), device=dev) * 3).to(dt)
        q, s = sglang_per_token_group_quant_fp8(x, 128, fuse_silu_and_mul=True)
        mid = torch.empty((65, 256), device=dev, dtype=dt)
        silu_and_mul(x, mid)
        q2, s2 = sglang_per_token_group_quant_fp8(mid, 128)
        np.testing.assert_array_equal(u8(q), u8(q2))
        assert torch.equal(s, s2)
    x = torch.randn((4, 512), device=dev, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="group_size 128"):
        sglang_per_token_group_quant_fp8(x, 64, fuse_silu_and_mul=True)
    with pytest.raises(RuntimeError, match="masked_m"):
        sglang_per_token_group_quant_fp8(x, 128, fuse_silu_and_mul=True, masked_m=torch.zeros(1, device=dev, dtype=torch.int32))


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("layout", _layouts())
def test_masked_group_quant(dev, layout, fuse):
    """Masked expert layout (reference: per_token_group_quant_8bit_v2.cu with masked_m, ep_moe/kernels.py:364-429):
    rows below masked_m[e] must equal the unmasked op on the same rows bit for bit, rows at or past it must be
    left untouched (output and scales)."""
    from sglang_amd.fp8_kernel import create_per_token_group_quant_fp8_output_scale, fp8_max, fp8_min, sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_8bit

    cm, al, ue = layout
    E, m_max, K = 5, 40, 512
    masked = [0, 40, 7, 33, 1]
    width = 2 * K if fuse else K
    x = torch.from_numpy(O.make_activation(E * m_max, width, seed=11)).to(dev).to(torch.bfloat16).view(E, m_max, width)
    mm = torch.tensor(masked, device=dev, dtype=torch.int32)
    q = torch.full((E, m_max, K), 0x55, device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn)
    G = K // 128
    if ue:
        s = create_per_token_group_quant_fp8_output_scale((E, m_max, K), dev, 128, cm, al, ue)
    elif cm:  # per-expert column-major (tokens contiguous), optionally padded to 4 tokens
        pad = (m_max + 3) // 4 * 4 if al else m_max
        s = torch.empty((E, G, pad), device=dev, dtype=torch.float32).transpose(-1, -2)[:, :m_max, :]
    else:
        s = torch.empty((E, m_max, G), device=dev, dtype=torch.float32)
    s.fill_(7 if ue else 7.0)
    sgl_per_token_group_quant_8bit(x, q, s, 128, 1e-10, fp8_min, fp8_max, ue, fuse, mm)
    torch.cuda.synchronize()
    qn, sn = u8(q).reshape(E, m_max, K), s.cpu().numpy()
    for e in range(E):
        m = masked[e]
        if m:
            q2, s2 = sglang_per_token_group_quant_fp8(x[e, :m].contiguous(), 128, fuse_silu_and_mul=fuse, column_major_scales=cm,
                                                      scale_tma_aligned=al, scale_ue8m0=ue)
            np.testing.assert_array_equal(qn[e, :m], u8(q2).reshape(m, K))
            np.testing.assert_array_equal(sn[e, :m].view(np.uint32), s2.cpu().numpy().view(np.uint32))
        assert np.all(qn[e, m:] == 0x55)
        if not ue:
            assert np.all(sn[e, m:] == 7.0)


def test_silu_and_mul_masked_post_quant_fwd(dev):
    from sglang_amd.ep_moe_kernels import silu_and_mul_masked_post_quant_fwd
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    E, m_max, K = 3, 130, 256
    masked = torch.tensor([130, 0, 65], device=dev, dtype=torch.int32)
    x = (torch.randn((E, m_max, 2 * K), device=dev) * 2).to(torch.bfloat16)
    out = torch.zeros((E, m_max, K), device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn)
    sc = torch.zeros((E, m_max, K // 128), device=dev, dtype=torch.float32)
    silu_and_mul_masked_post_quant_fwd(x, out, sc, 128, masked)
    for e, m in enumerate(masked.tolist()):
        if m:
            q2, s2 = sglang_per_token_group_quant_fp8(x[e, :m].contiguous(), 128, fuse_silu_and_mul=True)
            np.testing.assert_array_equal(u8(out).reshape(E, m_max, K)[e, :m], u8(q2).reshape(m, K))
            assert torch.equal(sc[e, :m], s2)
        assert torch.all(sc[e, m:] == 0)


def test_silu_and_mul_masked_post_quant_fwd_ue8m0_scales_as_floats(dev):
    """scale_ue8m0=True (reference: ep_moe/kernels.py:348-350): the scale is 2^ceil(log2(amax/448)) stored as float32;
    bytes and scales equal the oracle's fused activation quant with UE8M0 scales, rows past masked_m keep their values."""
    from sglang_amd.ep_moe_kernels import silu_and_mul_masked_post_quant_fwd, tma_align_input_scale

    rng = np.random.default_rng(31)
    E, m_max, K = 3, 70, 384
    masked = np.array([70, 0, 33], dtype=np.int32)
    x = O.to_bf16(rng.standard_normal((E, m_max, 2 * K)).astype(np.float32) * 2)
    out = torch.full((E, m_max, K), 0x55, device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn)
    sc = torch.full((E, m_max, K // 128), 7.0, device=dev, dtype=torch.float32)
    silu_and_mul_masked_post_quant_fwd(bf16_tensor(x, dev), out, sc, 128, torch.from_numpy(masked).to(dev), scale_ue8m0=True)
    qn, sn = u8(out).reshape(E, m_max, K), sc.cpu().numpy()
    for e, m in enumerate(masked.tolist()):
        if m:
            q_ref, s_ref = O.silu_mul_per_token_group_quant_fp8(x[e, :m], 128, scale_ue8m0=True)
            np.testing.assert_array_equal(qn[e, :m], q_ref)
            np.testing.assert_array_equal(sn[e, :m], s_ref)
        assert np.all(qn[e, m:] == 0x55) and np.all(sn[e, m:] == 7.0)
    # the column-major copy of a scale matrix
    s2 = torch.from_numpy(rng.standard_normal((37, 5)).astype(np.float32)).to(dev)
    al = tma_align_input_scale(s2)
    assert al.shape == s2.shape and al.stride() == (1, 40) and torch.equal(al, s2)
