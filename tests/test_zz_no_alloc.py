"""fp8k_block_gemm_noalloc (the block GEMM whose scratch is a fixed device array inside the library) against
fp8k_block_gemm with a caller-owned workspace, both called through the C ABI: the same kernels on the same plan, so
the outputs must agree bit for bit.  Two calls in a row share the built-in buffer, the second with a smaller input
(what the first call left in the buffer must not leak into it); shapes cover float partials of a K cut, the
column-major scale copy, and a shape that needs no scratch at all.  Sizes beyond the built-in buffer are refused.
"""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from tests.conftest import fp8_tensor

pytestmark = pytest.mark.gpu


def _entry():
    from sglang_amd._lib import lib

    return lib, lib.fp8k_block_gemm_noalloc


def _problem(M, N, K, seed, dev):
    rng = np.random.default_rng(seed)
    xq = rng.integers(0, 0x68, (M, K), dtype=np.uint8) | (rng.integers(0, 2, (M, K), dtype=np.uint8) << 7)
    wq = rng.integers(0, 0x68, (N, K), dtype=np.uint8) | (rng.integers(0, 2, (N, K), dtype=np.uint8) << 7)
    xs = (rng.uniform(0.5, 2.0, (M, K // 128)) * 1e-2).astype(np.float32)
    ws = (rng.uniform(0.5, 2.0, (N // 128, K // 128)) * 1e-3).astype(np.float32)
    return xq, wq, xs, ws, fp8_tensor(xq, dev), fp8_tensor(wq, dev), torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev)


def _both(lib, fn, A, B, As, Bs, M, N, K, dev):
    from sglang_amd._lib import check, stream_ptr

    st = stream_ptr(dev)
    need = lib.fp8k_block_gemm_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    C_ref = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    check(lib.fp8k_block_gemm(A.data_ptr(), B.data_ptr(), As.data_ptr(), Bs.data_ptr(), C_ref.data_ptr(), M, N, K, K, K,
                              As.stride(0), As.stride(1), Bs.stride(0), Bs.stride(1), N, 2, ws.data_ptr(), need, st))
    check(fn(A.data_ptr(), B.data_ptr(), As.data_ptr(), Bs.data_ptr(), C.data_ptr(), M, N, K, K, K,
             As.stride(0), As.stride(1), Bs.stride(0), Bs.stride(1), N, 2, st))
    torch.cuda.synchronize()
    return C, C_ref, need


# (first call, second smaller call): K-cut partials of the direct, streaming, 128x128 and 256x256 families, the scale copy
PAIRS = [((16, 7168, 16384), (5, 7168, 2304)), ((128, 7168, 16384), (40, 4608, 7168)), ((512, 1024, 4096), (300, 512, 1024)),
         ((4096, 4608, 7168), (1024, 4608, 7168)), ((1000, 2304, 512), (33, 256, 128))]


@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_block_gemm_equals_workspace_form_on_two_calls_in_a_row(dev, first, second):
    lib, fn = _entry()
    used_scratch = False
    for i, (M, N, K) in enumerate((first, second)):
        print("noalloc case", first, second, "call", i, flush=True)
        xq, wq, xs, ws, A, B, As, Bs = _problem(M, N, K, M + N + K, dev)
        C, C_ref, need = _both(lib, fn, A, B, As, Bs, M, N, K, dev)
        used_scratch |= need > 0
        assert bool(torch.isfinite(C).all())
        assert torch.equal(C, C_ref), (M, N, K)
        # and against the oracle on a sample, <= 1e-2 max relative error
        rows = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(M).integers(0, M, 4)]))
        cols = np.unique(np.concatenate([np.arange(0, min(N, 130)), np.random.default_rng(N).integers(0, N, 200)]))
        ref = O.w8a8_block_fp8_matmul(xq[rows], wq, xs[rows], ws, out_dtype="f32", acc=np.float64)[:, cols]
        got = C[torch.from_numpy(rows).to(dev)][:, torch.from_numpy(cols).to(dev)].float().cpu().numpy()
        assert np.abs(got - ref).max() / np.abs(ref).max() <= 1e-2
    assert used_scratch


def test_noalloc_block_gemm_refuses_sizes_beyond_its_buffer(dev):
    lib, fn = _entry()
    M, N, K = 200000, 7168, 18432      # the column-major scale copy alone is 115 MB
    assert lib.fp8k_block_gemm_workspace_bytes(M, N, K) > (80 << 20)
    p = torch.zeros(256, dtype=torch.uint8, device=dev).data_ptr()
    rc = fn(p, p, p, p, p, M, N, K, K, K, K // 128, 1, K // 128, 1, N, 2, None)
    assert rc == 4
    msg = lib.fp8k_last_error().decode()
    assert "needs" in msg and "built-in" in msg and "fp8k_block_gemm" in msg


def test_noalloc_block_gemm_replayed_from_a_hip_graph(dev):
    """Two calls recorded into one HIP graph after a warm-up call outside the capture (the address look-up is not a
    stream operation), replayed three times with eager work and synchronisations in between: every replay must give the
    workspace form's bits.  Both shapes use the built-in scratch (K-cut partials, scale copy)."""
    from sglang_amd._lib import check, stream_ptr

    lib, fn = _entry()
    shapes = [(128, 7168, 16384), (1024, 4608, 7168)]
    probs = [_problem(M, N, K, 7 + M, dev) for (M, N, K) in shapes]
    refs = []
    for (M, N, K), pr in zip(shapes, probs):
        C, C_ref, need = _both(lib, fn, *pr[4:], M, N, K, dev)  # also the warm-up call on this device
        assert need > 0 and torch.equal(C, C_ref)
        refs.append(C_ref)
    outs = [torch.empty_like(r) for r in refs]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        st = stream_ptr(dev)
        for (M, N, K), pr, C in zip(shapes, probs, outs):
            A, B, As, Bs = pr[4:]
            check(fn(A.data_ptr(), B.data_ptr(), As.data_ptr(), Bs.data_ptr(), C.data_ptr(), M, N, K, K, K,
                     As.stride(0), As.stride(1), Bs.stride(0), Bs.stride(1), N, 2, st))
    for replay in range(3):
        for C in outs:
            C.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for C, r in zip(outs, refs):
            assert torch.equal(C, r), replay
        # eager work that uses the same built-in buffer between the replays
        M, N, K = shapes[0]
        C, C_ref, _ = _both(lib, fn, *probs[0][4:], M, N, K, dev)
        assert torch.equal(C, C_ref)
