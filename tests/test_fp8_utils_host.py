"""Host-side weight transforms of fp8_utils (plain tensor code, runs on the CPU): checked against the numpy oracle
and against what the mathematics fixes (power-of-two scales, exact round trips)."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O


def _fp8(a_u8):
    return torch.from_numpy(np.ascontiguousarray(a_u8)).view(torch.float8_e4m3fn)


def test_block_quant_dequant_and_tensor_requant():
    from sglang_amd.fp8_utils import block_quant_dequant, block_quant_to_tensor_quant, channel_quant_to_tensor_quant

    w = O.make_weight(300, 520, seed=3)                        # not multiples of 128: ragged edge tiles
    wq, ws = O.block_quant_weight(w)
    deq = block_quant_dequant(_fp8(wq), torch.from_numpy(ws), [128, 128], torch.float32).numpy()
    ref = O.e4m3fn_to_f32(wq) * np.repeat(np.repeat(ws, 128, 0), 128, 1)[:300, :520]
    np.testing.assert_array_equal(deq, ref.astype(np.float32))
    q, s = block_quant_to_tensor_quant(_fp8(wq), torch.from_numpy(ws), [128, 128])
    assert q.dtype == torch.float8_e4m3fn and s.numel() == 1
    amax = np.abs(ref).max()
    np.testing.assert_allclose(float(s), amax / 448.0, rtol=1e-6)
    np.testing.assert_allclose(q.float().numpy() * float(s), ref, atol=float(s) * 16 + 1e-12)  # half an e4m3 ulp at 448
    xs = torch.rand((300, 1)) * 0.01 + 1e-3
    q2, s2 = channel_quant_to_tensor_quant(_fp8(wq), xs)
    ref2 = O.e4m3fn_to_f32(wq) * xs.numpy()
    np.testing.assert_allclose(float(s2), np.abs(ref2).max() / 448.0, rtol=1e-6)


def test_per_block_cast_and_ue8m0_requant():
    from sglang_amd.fp8_utils import per_block_cast_to_fp8, requant_weight_ue8m0

    w = torch.from_numpy(O.make_weight(256, 384, seed=5)).to(torch.bfloat16)
    q, sc = per_block_cast_to_fp8(w)
    assert q.shape == w.shape and sc.shape == (2, 3)
    m, e = np.frexp(sc.numpy())
    assert np.all(m == 0.5)                                      # powers of two
    blocks = w.float().view(2, 128, 3, 128).abs().amax(dim=(1, 3)).clamp(1e-4)
    assert torch.all(sc >= blocks / 448.0) and torch.all(sc < blocks / 448.0 * 2)   # the smallest power of two that fits
    ref_q = O.f32_to_e4m3fn((w.float() / sc.repeat_interleave(128, 0).repeat_interleave(128, 1)).numpy())
    np.testing.assert_array_equal(q.view(torch.uint8).numpy(), ref_q)
    # requant of a float-scale checkpoint: scales become powers of two, values stay within one e4m3 step of the
    # bf16 dequantisation
    wq, ws = O.block_quant_weight(O.make_weight(256, 256, seed=7))
    q2, s2 = requant_weight_ue8m0(_fp8(wq), torch.from_numpy(ws), [128, 128])
    assert np.all(np.frexp(s2.numpy())[0] == 0.5)
    deq = O.e4m3fn_to_f32(wq) * np.repeat(np.repeat(ws, 128, 0), 128, 1)
    back = q2.float().numpy() * np.repeat(np.repeat(s2.numpy(), 128, 0), 128, 1)
    step = np.repeat(np.repeat(s2.numpy(), 128, 0), 128, 1) * 32  # largest e4m3 spacing (between 416 and 448) in scaled units
    assert np.all(np.abs(back - deq) <= step * 0.5 + np.abs(deq) * 2 ** -8)
    # batched weights [E, n, k]
    q3, s3 = requant_weight_ue8m0(_fp8(np.stack([wq, wq])), torch.from_numpy(np.stack([ws, ws])), [128, 128])
    assert q3.shape == (2, 256, 256) and s3.shape == (2, 2, 2) and torch.equal(q3[0], q2) and torch.equal(s3[1], s2)


def test_input_to_float8():
    from sglang_amd.fp8_utils import input_to_float8

    x = torch.randn(64, 96) * 3
    q, s = input_to_float8(x)
    assert q.dtype == torch.float8_e4m3fn
    np.testing.assert_allclose(float(s), float(x.abs().max()) / 448.0, rtol=1e-6)
    assert float(q.float().abs().max()) == 448.0
    q0, s0 = input_to_float8(torch.zeros(4, 4))
    assert float(s0) == pytest.approx(1e-12 / 448.0) and torch.all(q0.float() == 0)


def test_ue8m0_unpack_and_marking():
    """Packed UE8M0 words -> float32 powers of two, for activations ([M, ceil(G/4)]) and for weights in the per-row
    layout the reference hands to DeepGEMM ([N, ceil(G/4)], the 128 rows of a block alike); mark_ue8m0 accepts powers
    of two only."""
    from sglang_amd.sgl_kernel import is_ue8m0, mark_ue8m0, unpack_ue8m0_scales, unpack_ue8m0_weight_scales

    rng = np.random.default_rng(5)
    s = (2.0 ** rng.integers(-30, 10, (7, 6))).astype(np.float32)
    packed = torch.from_numpy(O.pack_ue8m0_scales(s))
    np.testing.assert_array_equal(unpack_ue8m0_scales(packed, 6).numpy(), s)
    s3 = (2.0 ** rng.integers(-20, 5, (3, 5, 9))).astype(np.float32)   # a leading group dimension, ragged word count
    p3 = torch.from_numpy(np.stack([O.pack_ue8m0_scales(x) for x in s3]))
    np.testing.assert_array_equal(unpack_ue8m0_scales(p3, 9).numpy(), s3)
    # weights: [N/128, K/128] block scales repeated over the 128 rows of a block, then packed per row
    ws = (2.0 ** rng.integers(-14, -6, (3, 10))).astype(np.float32)
    per_row = torch.from_numpy(O.pack_ue8m0_scales(np.repeat(ws, 128, axis=0)))
    assert per_row.shape == (384, 3)
    np.testing.assert_array_equal(unpack_ue8m0_weight_scales(per_row, 10 * 128).numpy(), ws)
    t = torch.from_numpy(ws.copy())
    assert not is_ue8m0(t)
    assert mark_ue8m0(t) is t and is_ue8m0(t)
    with pytest.raises(RuntimeError, match="powers of two"):
        mark_ue8m0(torch.tensor([[1.0, 3.0]]))
    with pytest.raises(RuntimeError, match="powers of two"):
        mark_ue8m0(torch.tensor([[1.0, 0.0]]))
    # the mark belongs to the memory: other tensor objects over it see it, other memory does not, and it ends with
    # the marked object
    assert is_ue8m0(t.data) and is_ue8m0(torch.nn.Parameter(t, requires_grad=False)) and is_ue8m0(t.view(3, 10))
    assert not is_ue8m0(t.clone()) and not is_ue8m0(t[1:]) and not is_ue8m0(t.t())
    other = t.data
    del t
    assert not is_ue8m0(other)


def test_requant_weight_ue8m0_inplace_marks_the_parameter():
    """After the in-place requantisation of a float-scale checkpoint the scale parameter - the object a layer passes to
    the GEMM - and its .data are known to hold powers of two, so the hardware-scaled route can be taken."""
    from sglang_amd.fp8_utils import requant_weight_ue8m0_inplace
    from sglang_amd.sgl_kernel import is_ue8m0

    rng = np.random.default_rng(9)
    wq, ws = O.block_quant_weight(O.make_weight(256, 384, 1))
    ws = (ws * rng.uniform(0.6, 1.7, ws.shape)).astype(np.float32)
    weight = torch.nn.Parameter(torch.from_numpy(wq).view(torch.float8_e4m3fn), requires_grad=False)
    scale = torch.nn.Parameter(torch.from_numpy(ws), requires_grad=False)
    assert not is_ue8m0(scale)
    requant_weight_ue8m0_inplace(weight, scale, [128, 128])
    assert is_ue8m0(scale) and is_ue8m0(scale.data)
    bits = scale.data.view(torch.int32)
    assert bool(((bits & 0x7FFFFF) == 0).all())


def test_cast_to_e8m0_with_rounding_up_host():
    """deep_gemm_moe_runner.cast_to_e8m0_with_rounding_up on CPU tensors (reference: moe_runner/deep_gemm.py:48-58):
    equal to the oracle's ceil-to-power-of-two + word packing on ordinary scales, and the reference's corner cases."""
    import numpy as np
    import torch

    from oracle import fp8_oracle as O
    from sglang_amd.deep_gemm_moe_runner import cast_to_e8m0_with_rounding_up

    rng = np.random.default_rng(8)
    s = (rng.uniform(1.0, 2.0, (2, 5, 7)) * 2.0 ** rng.integers(-20, 10, (2, 5, 7))).astype(np.float32)
    s[0, 0, :3] = [1.0, 0.25, 3.0]
    got = cast_to_e8m0_with_rounding_up(torch.from_numpy(s)).numpy()
    ref = np.stack([O.pack_ue8m0_scales(O.ceil_to_ue8m0(x)) for x in s])
    assert got.shape == (2, 5, 2) and np.array_equal(got, ref)
    edge = np.array([[3.0e38, 1e-45, 8e-39, 0.0]], dtype=np.float32)
    b = cast_to_e8m0_with_rounding_up(torch.from_numpy(edge)).numpy().view(np.uint8).reshape(-1)
    assert list(b[:4]) == [0xFE, 0, 1, 0]


def test_transform_scale_ue8m0_round_trip():
    """transform_scale_ue8m0 / inverse_transform_scale_ue8m0 (reference: fp8_utils.py:505-565): words equal to the
    oracle's packing of the row-repeated scales, mn-major storage padded to 4 rows, exact round trip, 2-D and 3-D."""
    import numpy as np
    import torch

    from oracle import fp8_oracle as O
    from sglang_amd.fp8_utils import inverse_transform_scale_ue8m0, transform_scale_ue8m0

    rng = np.random.default_rng(12)
    for shape, mn in (((3, 6), 384), ((2, 2, 5), 256)):
        sf = (2.0 ** rng.integers(-14, 3, shape)).astype(np.float32)
        packed = transform_scale_ue8m0(torch.from_numpy(sf), mn)
        kb4 = (shape[-1] + 3) // 4
        assert packed.shape == shape[:-2] + (mn, kb4) and packed.dtype == torch.int32
        assert packed.stride(-2) == 1 and packed.stride(-1) == (mn + 3) // 4 * 4
        rep = np.repeat(sf, 128, axis=-2)
        ref = O.pack_ue8m0_scales(rep) if sf.ndim == 2 else np.stack([O.pack_ue8m0_scales(x) for x in rep])
        assert np.array_equal(packed.numpy(), ref)
        back = inverse_transform_scale_ue8m0(packed, mn)
        assert np.array_equal(back.numpy()[..., : shape[-1]], sf)
