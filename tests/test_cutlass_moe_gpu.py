"""GPU parity of the expert-major ("CUTLASS") MoE entry points against the oracle.

prepare_moe_input, shuffle_rows: integers and bytes, bit for bit (the order of the rows inside one expert is left
open by the reference's atomic counters: checked as a set).  apply_shuffle_mul_sum: bit for bit for 16-bit types.
fp8_blockwise_scaled_grouped_mm and cutlass_fused_experts_fp8: max relative error <= 1e-2 on bf16 / fp16 output, and the
1 - cosine-like `calc_diff` < 1e-3 that the reference's own tests use (sgl-kernel/tests/test_fp8_blockwise_moe.py:24-29,
python/sglang/test/test_cutlass_moe.py:15-19)."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import bf16_tensor, fp8_tensor

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _codes(rng, shape):
    return rng.integers(0, 0x60, shape, dtype=np.uint8) | (rng.integers(0, 2, shape, dtype=np.uint8) << 7)


def _rel(c, ref):
    return float(np.abs(c.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


def _calc_diff(x, y):
    x, y = x.astype(np.float64), y.astype(np.float64)
    return 1 - 2 * (x * y).sum() / max((x * x + y * y).sum(), 1e-300)


def _prepare(dev, ids, E, n, k, with_bs=False):
    from sglang_amd.sgl_kernel import prepare_moe_input

    t = torch.from_numpy(ids).to(dev)
    off = torch.full((E + 1,), -7, device=dev, dtype=torch.int32)
    bso = torch.full((E + 1,), -7, device=dev, dtype=torch.int32) if with_bs else None
    ps1 = torch.full((E, 3), -7, device=dev, dtype=torch.int32)
    ps2 = torch.full((E, 3), -7, device=dev, dtype=torch.int32)
    a_map = torch.full((ids.size,), -7, device=dev, dtype=torch.int32)
    c_map = torch.full((ids.size,), -7, device=dev, dtype=torch.int32)
    prepare_moe_input(t, off, ps1, ps2, a_map, c_map, E, n, k, bso)
    torch.cuda.synchronize()
    return off, bso, ps1, ps2, a_map, c_map


@pytest.mark.parametrize("m,topk,E", [(1, 8, 256), (37, 4, 9), (512, 8, 256), (4096, 8, 256), (33, 1, 4096), (16500, 8, 64)])
def test_prepare_moe_input(dev, m, topk, E):
    rng = np.random.default_rng(m + E)
    ids = np.stack([rng.permutation(E)[:topk] if E >= topk else rng.integers(0, E, topk) for _ in range(m)]).astype(np.int32)
    if m > 8:
        ids[5, 0] = -1
        ids[6, topk - 1] = E  # outside [0, E): takes no row
    n, k = 2048, 7168
    off, bso, ps1, ps2, a_map, c_map = _prepare(dev, ids, E, n, k, with_bs=True)
    o_off, o_bso, o_ps1, o_ps2, o_a, o_c = O.prepare_moe_input(ids, E, n, k)
    assert np.array_equal(off.cpu().numpy(), o_off) and np.array_equal(bso.cpu().numpy(), o_bso)
    assert np.array_equal(ps1.cpu().numpy(), o_ps1) and np.array_equal(ps2.cpu().numpy(), o_ps2)
    a_map, c_map = a_map.cpu().numpy(), c_map.cpu().numpy()
    flat = ids.reshape(-1)
    valid = (flat >= 0) & (flat < E)
    total = int(valid.sum())
    # every slot sits in a row of its own expert, the row points back at the slot's token, rows are used once
    assert (c_map[~valid] == -7).all() and (a_map[total:] == -7).all()
    rows = c_map[valid]
    assert np.array_equal(np.sort(rows), np.arange(total))
    assert ((rows >= o_off[flat[valid]]) & (rows < o_off[flat[valid] + 1])).all()
    assert np.array_equal(a_map[rows], np.nonzero(valid)[0] // topk)
    for e in (0, E // 2, E - 1):  # as a multiset the rows of an expert are the oracle's
        assert np.array_equal(np.sort(a_map[o_off[e]:o_off[e + 1]]), np.sort(o_a[o_off[e]:o_off[e + 1]]))


@pytest.mark.parametrize("dtype,cols", [(torch.float8_e4m3fn, 7168), (torch.float32, 56), (torch.bfloat16, 2048), (torch.uint8, 37),
                                        (torch.float32, 1), (torch.float16, 6)])
def test_shuffle_rows(dev, dtype, cols):
    from sglang_amd.sgl_kernel import shuffle_rows

    rng = np.random.default_rng(cols)
    src, dst = 50, 331
    raw = torch.from_numpy(rng.integers(0, 255, (src, cols * torch.empty((), dtype=dtype).element_size()), dtype=np.uint8)).to(dev)
    x = raw.view(dtype)
    mp = torch.from_numpy(rng.integers(0, src, dst).astype(np.int32)).to(dev)
    out = shuffle_rows(x, mp, (dst, cols))
    assert out.dtype == dtype and tuple(out.shape) == (dst, cols)
    assert np.array_equal(out.view(torch.uint8).cpu().numpy(), O.shuffle_rows(raw.cpu().numpy(), mp.cpu().numpy()))


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("m,topk,k,with_factors", [(13, 6, 40, True), (300, 8, 7168, True), (1, 1, 8, False), (64, 8, 2048, False)])
def test_apply_shuffle_mul_sum(dev, dtype, name, m, topk, k, with_factors):
    from sglang_amd.sgl_kernel import apply_shuffle_mul_sum

    g = torch.Generator().manual_seed(m * topk)
    c2 = torch.randn(m * topk, k, generator=g).to(dtype)
    w = torch.rand(m, topk, generator=g).to(dtype) if with_factors else None
    c_map = torch.randperm(m * topk, generator=g).to(torch.int32)
    out = torch.empty((m, k), device=dev, dtype=dtype)
    apply_shuffle_mul_sum(c2.to(dev), out, c_map.to(dev), None if w is None else w.to(dev).reshape(-1))
    ref = O.apply_shuffle_mul_sum(c2.float().numpy(), c_map.view(m, topk).numpy(), None if w is None else w.float().numpy(), name)
    assert np.array_equal(out.float().cpu().numpy(), ref)


def test_apply_shuffle_mul_sum_without_permutation_is_the_identity_map(dev):
    from sglang_amd.sgl_kernel import apply_shuffle_mul_sum

    g = torch.Generator().manual_seed(5)
    m, topk, k = 77, 8, 512
    c2 = torch.randn(m * topk, k, generator=g).to(torch.bfloat16)
    w = torch.rand(m, topk, generator=g).to(torch.bfloat16)
    out = torch.empty((m, k), device=dev, dtype=torch.bfloat16)
    apply_shuffle_mul_sum(c2.to(dev), out, None, w.to(dev).reshape(-1))
    ref = O.apply_shuffle_mul_sum(c2.float().numpy(), np.arange(m * topk, dtype=np.int32).reshape(m, topk), w.float().numpy(), "bf16")
    assert np.array_equal(out.float().cpu().numpy(), ref)
    with pytest.raises(RuntimeError, match="without a permutation"):
        apply_shuffle_mul_sum(c2[:-1].to(dev), out, None, None)


@pytest.mark.parametrize("m,topk,E,block", [(1, 8, 256, 16), (37, 4, 9, 32), (512, 8, 256, 64), (700, 8, 8, 256), (4096, 8, 256, 128)])
def test_moe_slot_blocks(dev, m, topk, E, block):
    """The slot table built from prepare_moe_input's outputs: integer invariants of the reference's aligner
    (python/sglang/srt/layers/moe/fused_moe_triton/moe_align_block_size.py:17-82) - every expert's slots, as a set, in
    blocks of its own, padded with the slot count - without the leading bucket for ids outside [0, E)."""
    from sglang_amd.sgl_kernel import moe_slot_blocks

    rng = np.random.default_rng(m * 7 + E)
    ids = np.stack([rng.permutation(E)[:topk] if E >= topk else rng.integers(0, E, topk) for _ in range(m)]).astype(np.int32)
    if m > 8:
        ids[3, 0] = -1
        ids[4, topk - 1] = E
    off, _, ps1, _, _, c_map = _prepare(dev, ids, E, 256, 512)
    sorted_ids, expert_ids, post_pad = moe_slot_blocks(torch.from_numpy(ids).to(dev), off, ps1, c_map, block)
    torch.cuda.synchronize()
    sorted_ids, expert_ids, used = sorted_ids.cpu().numpy(), expert_ids.cpu().numpy(), int(post_pad.cpu()[0])
    flat = ids.reshape(-1)
    counts = np.bincount(flat[(flat >= 0) & (flat < E)], minlength=E)
    assert used == int(((counts + block - 1) // block * block).sum())
    pos = 0
    for e in range(E):
        nblk = (counts[e] + block - 1) // block
        assert (expert_ids[pos // block:pos // block + nblk] == e).all()
        seg = sorted_ids[pos:pos + nblk * block]
        assert np.array_equal(np.sort(seg[:counts[e]]), np.nonzero(flat == e)[0])
        assert (seg[counts[e]:] == flat.size).all()
        pos += nblk * block
    assert pos == used


def test_apply_shuffle_mul_sum_errors(dev):
    from sglang_amd.sgl_kernel import apply_shuffle_mul_sum

    x = torch.zeros((8, 16), device=dev, dtype=torch.bfloat16)
    out = torch.zeros((4, 16), device=dev, dtype=torch.bfloat16)
    perm = torch.zeros((8,), device=dev, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="factors must match output dtype"):
        apply_shuffle_mul_sum(x, out, perm, torch.zeros((8,), device=dev, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="m \\* topk"):
        apply_shuffle_mul_sum(x, out, perm[:7], None)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        apply_shuffle_mul_sum(x[:, :12].contiguous(), out[:, :12].contiguous(), perm, None)


def _grouped_case(rng, E, sizes, N, K):
    rows = int(sum(sizes))
    aq, bq = _codes(rng, (rows, K)), _codes(rng, (E, N, K))
    a_s = rng.uniform(0.5, 2.0, (rows, K // 128)).astype(np.float32) * 1e-2
    b_s = rng.uniform(0.5, 2.0, (E, N // 128, K // 128)).astype(np.float32) * 1e-2
    off = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    ps = np.array([[c, N, K] for c in sizes], dtype=np.int32)
    return rows, aq, bq, a_s, b_s, off, ps


@pytest.mark.parametrize("E,max_rows,N,K", [(8, 256, 512, 1024), (16, 256, 384, 512), (32, 64, 256, 256), (64, 12, 256, 384),
                                            (128, 3, 128, 128), (4, 700, 768, 640)])
@pytest.mark.parametrize("out_dtype,name", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
def test_fp8_blockwise_scaled_grouped_mm(dev, E, max_rows, N, K, out_dtype, name):
    """The reference test's construction (random rows per expert in [1, max], one expert left empty), through every
    block size of the grouped kernel."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    rng = np.random.default_rng(E * 31 + N)
    sizes = rng.integers(1, max_rows + 1, E)
    sizes[E // 2] = 0
    rows, aq, bq, a_s, b_s, off, ps = _grouped_case(rng, E, sizes, N, K)
    dummy = torch.empty((E,), device=dev, dtype=torch.int64)
    layout = torch.zeros((E, 5), device=dev, dtype=torch.int32)
    out = torch.full((rows, N), 3.0, device=dev, dtype=out_dtype)
    b = fp8_tensor(bq, dev).transpose(1, 2)
    sb = torch.from_numpy(b_s).to(dev).transpose(1, 2)
    fp8_blockwise_scaled_grouped_mm(out, dummy, dummy, dummy, dummy, dummy, fp8_tensor(aq, dev), b, torch.from_numpy(a_s).to(dev), sb,
                                    dummy, dummy, dummy, layout, layout, torch.from_numpy(ps).to(dev),
                                    torch.from_numpy(off).to(dev)[:-1].contiguous(), torch.empty((16,), device=dev, dtype=torch.uint8))
    torch.cuda.synchronize()
    ref = O.fp8_blockwise_scaled_grouped_mm(aq, bq, a_s, b_s, off, ps, "f32", acc=np.float64)
    got = out.float().cpu().numpy()
    assert _rel(got, ref) <= REL_TOL, _rel(got, ref)
    for e in range(E):
        if sizes[e]:
            assert _calc_diff(got[off[e]:off[e + 1]], ref[off[e]:off[e + 1]]) < 1e-3


def test_grouped_mm_leaves_unowned_rows_untouched_and_takes_untransposed_scales(dev):
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    rng = np.random.default_rng(12)
    E, N, K = 4, 256, 384  # N/128 != K/128: the shape alone says the scales are the un-transposed checkpoint tensor
    sizes = np.array([10, 0, 20, 5])
    rows, aq, bq, a_s, b_s, off, ps = _grouped_case(rng, E, sizes, N, K)
    ps[2, 0] = 12  # expert 2 uses only 12 of its 20 rows
    dummy = torch.empty((E,), device=dev, dtype=torch.int64)
    out = torch.full((rows, N), 3.0, device=dev, dtype=torch.bfloat16)
    fp8_blockwise_scaled_grouped_mm(out, dummy, dummy, dummy, dummy, dummy, fp8_tensor(aq, dev), fp8_tensor(bq, dev).transpose(1, 2),
                                    torch.from_numpy(a_s).to(dev), torch.from_numpy(b_s).to(dev), dummy, dummy, dummy, dummy, dummy,
                                    torch.from_numpy(ps).to(dev), torch.from_numpy(off[:-1].copy()).to(dev), dummy)
    got = out.float().cpu().numpy()
    ref = O.fp8_blockwise_scaled_grouped_mm(aq, bq, a_s, b_s, off, ps, "f32", acc=np.float64)
    owned = np.zeros(rows, bool)
    for e in range(E):
        owned[off[e]:off[e] + ps[e, 0]] = True
    assert _rel(got[owned], ref[owned]) <= REL_TOL
    assert (got[~owned] == 3.0).all()
    with pytest.raises(RuntimeError, match="column-major"):
        fp8_blockwise_scaled_grouped_mm(out, dummy, dummy, dummy, dummy, dummy, fp8_tensor(aq, dev),
                                        fp8_tensor(bq, dev).transpose(1, 2).contiguous(), torch.from_numpy(a_s).to(dev),
                                        torch.from_numpy(b_s).to(dev), dummy, dummy, dummy, dummy, dummy,
                                        torch.from_numpy(ps).to(dev), torch.from_numpy(off[:-1].copy()).to(dev), dummy)


def test_grouped_mm_reads_square_scales_in_the_ops_own_layout(dev):
    """N/128 == K/128: scales_b is [E, K/128, N/128] whatever its strides - the transposed view the reference passes and a
    contiguous tensor of the same logical content give the same result (a contiguous square tensor is never taken for
    the un-transposed checkpoint layout)."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    rng = np.random.default_rng(13)
    E, N, K = 3, 256, 256
    sizes = np.array([7, 40, 3])
    rows, aq, bq, a_s, b_s, off, ps = _grouped_case(rng, E, sizes, N, K)
    b_s = (b_s * rng.uniform(0.5, 2.0, b_s.shape)).astype(np.float32)  # make the block scales visibly non-symmetric
    dummy = torch.empty((E,), device=dev, dtype=torch.int64)
    ref = O.fp8_blockwise_scaled_grouped_mm(aq, bq, a_s, b_s, off, ps, "f32", acc=np.float64)
    view = torch.from_numpy(b_s).to(dev).transpose(1, 2)                      # [E, K/128, N/128], stride(1) == 1
    dense = torch.from_numpy(np.ascontiguousarray(b_s.transpose(0, 2, 1))).to(dev)  # same values, contiguous
    for scales in (view, dense):
        out = torch.empty((rows, N), device=dev, dtype=torch.bfloat16)
        fp8_blockwise_scaled_grouped_mm(out, dummy, dummy, dummy, dummy, dummy, fp8_tensor(aq, dev), fp8_tensor(bq, dev).transpose(1, 2),
                                        torch.from_numpy(a_s).to(dev), scales, dummy, dummy, dummy, dummy, dummy,
                                        torch.from_numpy(ps).to(dev), torch.from_numpy(off[:-1].copy()).to(dev), dummy)
        assert _rel(out.float().cpu().numpy(), ref) <= REL_TOL


def _experts(rng, E, H, I, std=0.05):
    w13q = np.empty((E, 2 * I, H), np.uint8); w13s = np.empty((E, 2 * I // 128, H // 128), np.float32)
    w2q = np.empty((E, H, I), np.uint8); w2s = np.empty((E, H // 128, I // 128), np.float32)
    for e in range(E):
        w13q[e], w13s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((2 * I, H)).astype(np.float32) * std))
        w2q[e], w2s[e] = O.block_quant_weight(O.to_bf16(rng.standard_normal((H, I)).astype(np.float32) * std))
    return w13q, w13s, w2q, w2s


@pytest.mark.parametrize("T,E,H,I,topk", [(1, 8, 256, 128, 2), (33, 8, 512, 256, 2), (96, 16, 1024, 512, 4), (700, 8, 512, 256, 8)])
def test_cutlass_fused_experts_fp8(dev, T, E, H, I, topk):
    """The call of Fp8MoEMethod.apply (fp8.py:1080-1103): transposed weights and scales, pre-allocated index buffers and
    output; against the oracle's expert-major composite, and close to the Triton-ordered fused_experts_impl of this
    library on the same inputs (as python/sglang/test/test_cutlass_moe.py compares the two paths)."""
    from sglang_amd.cutlass_moe import cutlass_fused_experts_fp8
    from sglang_amd.fused_moe import fused_experts_impl

    rng = np.random.default_rng(T + E)
    x = O.make_activation(T, H, T)
    w13q, w13s, w2q, w2s = _experts(rng, E, H, I)
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    tw = O.to_bf16(rng.uniform(0.1, 1.0, (T, topk)).astype(np.float32))
    i64 = lambda: torch.empty((E,), device=dev, dtype=torch.int64)  # noqa: E731
    w1, w2 = fp8_tensor(w13q, dev), fp8_tensor(w2q, dev)
    s1, s2 = torch.from_numpy(w13s).to(dev), torch.from_numpy(w2s).to(dev)
    xt, twt, idt = bf16_tensor(x, dev), bf16_tensor(tw, dev), torch.from_numpy(ids).to(dev)
    out = torch.empty((T, H), device=dev, dtype=torch.bfloat16)
    ret = cutlass_fused_experts_fp8(
        xt, w1.transpose(1, 2), w2.transpose(1, 2), s1.transpose(1, 2), s2.transpose(1, 2), twt, idt,
        torch.full((E,), H, device=dev, dtype=torch.int64), torch.full((E,), 2 * I, device=dev, dtype=torch.int64),
        torch.full((E,), I, device=dev, dtype=torch.int64), torch.full((E,), H, device=dev, dtype=torch.int64),
        torch.empty((1024,), device=dev, dtype=torch.uint8), i64(), i64(), i64(), i64(), i64(),
        torch.empty((E + 1,), device=dev, dtype=torch.int32), torch.empty((E, 3), device=dev, dtype=torch.int32),
        torch.empty((E, 3), device=dev, dtype=torch.int32), use_fp8_blockscale=True, output=out)
    torch.cuda.synchronize()
    assert ret is out
    got = out.float().cpu().numpy()
    ref = O.cutlass_fused_experts_fp8(x, w13q, w13s, w2q, w2s, tw, ids)
    assert _rel(got, ref) <= REL_TOL, _rel(got, ref)
    triton_order = fused_experts_impl(xt, w1, w2, twt.float(), idt, use_fp8_w8a8=True, w1_scale=s1, w2_scale=s2, block_shape=[128, 128])
    assert _calc_diff(got, triton_order.float().cpu().numpy()) < 1e-3
