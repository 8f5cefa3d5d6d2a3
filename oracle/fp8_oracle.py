"""CPU oracle for the W8A8 FP8 linear path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the arithmetic of the reference functions on the
path.  Only tests, the smoke check and the CPU-baseline leg of the bench may
import it; the product package never does.

Every function names the reference lines it follows (paths relative to the
reference checkout).  None of them was produced by running the reference: they
are pinned by closed forms, exhaustive tables and library routines
(tests/test_oracle_*.py):

* e4m3fn encode/decode      - exhaustive against torch's CPU ``.to(float8_e4m3fn)``
                              and the OCP table (448 max, 0x7F NaN, 2^-9 subnormals)
* group quant               - closed form of test/srt/quant/test_fp8_kernel.py:24-45
                              (amax == 448 -> scale 1, bytes == input), exhaustive
                              scale table over every positive finite bf16 amax
* UE8M0                     - exact bit form vs 2**ceil(log2(s)) for every bf16 amax
* block / scaled matmul     - dequantise-then-matmul in float64, brute-force triple
                              loop on tiny shapes, exactness on integer data
* moe_align_block_size      - integer invariants (bincount, padding, ownership)
* silu_and_mul / sum_reduce - torch CPU bf16 arithmetic

All tensors are numpy arrays.  bf16 / fp16 tensors are carried as float32 arrays
whose values are representable in the narrow type (``to_bf16`` rounds).
"""
from __future__ import annotations

import numpy as np

FP8_MAX = 448.0
FP8_MIN = -448.0

# --------------------------------------------------------------------------
# number formats
# --------------------------------------------------------------------------


def to_bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bf16 (ties to even); result kept as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    b = x.view(np.uint32).astype(np.uint64)
    nan = np.isnan(x)
    r = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).copy()
    out[nan] = np.nan
    return out.reshape(x.shape)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """uint16 bit patterns of a float32 array that holds bf16-representable values."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b).astype(np.uint32) << 16).view(np.float32)


def f32_to_e4m3fn(x: np.ndarray) -> np.ndarray:
    """OCP FP8 e4m3fn encode, round-to-nearest-even, no saturation.

    |x| that rounds above 448 and NaN become 0x7F | sign (the format has no Inf).
    Same contract as ``tensor.to(torch.float8_e4m3fn)`` which the reference's
    native quant ends with (python/sglang/test/test_block_fp8.py:44).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    a = (bits & 0x7FFFFFFF).astype(np.uint32)
    out = np.zeros(x.shape, dtype=np.uint8)

    normal = a >= np.uint32(0x3C800000)  # |x| >= 2^-6
    # normal: keep 3 mantissa bits, RNE on bit 20
    ar = a.astype(np.uint64) + 0x7FFFF + ((a >> 20) & 1)
    code = (ar >> 20).astype(np.int64) - (120 << 3)
    code = np.where(code > 0x7F, 0x7F, code)
    out = np.where(normal, code, 0).astype(np.uint8)
    # subnormal: multiples of 2^-9, RNE; 8 * 2^-9 is the smallest normal (code 0x08)
    mag = np.abs(np.nan_to_num(x, nan=0.0, posinf=0.0, neginf=0.0)).astype(np.float64)
    sub = np.rint(np.where(normal, 0.0, mag) * 512.0).astype(np.uint8)
    out = np.where(normal, out, sub).astype(np.uint8)
    out = np.where(np.isnan(x) | (a >= np.uint32(0x7F800000)), np.uint8(0x7F), out)
    return (out | sign).astype(np.uint8)


def _build_e4m3fn_table() -> np.ndarray:
    t = np.zeros(256, dtype=np.float32)
    for v in range(256):
        s, e, m = v >> 7, (v >> 3) & 15, v & 7
        if e == 0:
            r = m * 2.0**-9
        elif e == 15 and m == 7:
            r = float("nan")
        else:
            r = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[v] = -r if s else r
    return t


E4M3FN_TABLE = _build_e4m3fn_table()


def e4m3fn_to_f32(q: np.ndarray) -> np.ndarray:
    return E4M3FN_TABLE[np.asarray(q, dtype=np.uint8)]


# --------------------------------------------------------------------------
# a.1 / a.2 / a.3  per-token-group quant
# --------------------------------------------------------------------------


def clamp_eps(eps: float, in_dtype: str) -> np.float32:
    """eps as the reference's native path sees it.

    ``x_.abs().max(-1).clamp(min=eps)`` runs in the input dtype before the cast to
    float32 (python/sglang/test/test_block_fp8.py:42), so for a bf16 input the
    Python scalar 1e-10 is first rounded to bf16 (0x2EDC -> 1.00044e-10).  fp16
    cannot hold 1e-10 (it would clamp to 0 and make 0/0); for fp16 and fp32 the
    float32 eps of the device kernel is used instead
    (sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:42).
    """
    if in_dtype == "bf16":
        return np.float32(to_bf16(np.array([eps], dtype=np.float32))[0])
    return np.float32(eps)


def ceil_to_ue8m0(s: np.ndarray) -> np.ndarray:
    """Smallest power of two >= s, by exponent bits (s positive, normal float32).

    Equals ``2**ceil(log2(s))`` (python/sglang/srt/layers/quantization/fp8_utils.py:585-586,
    per_token_group_quant_8bit.cu:86-88) without going through log2.
    """
    b = np.ascontiguousarray(s, dtype=np.float32).view(np.uint32)
    e = (b >> 23) + ((b & 0x7FFFFF) != 0)
    return (e.astype(np.uint32) << 23).view(np.float32)


def ue8m0_byte(s_pow2: np.ndarray) -> np.ndarray:
    """Biased exponent byte of a power-of-two float32 (per_token_group_quant_8bit.cu:91-97)."""
    return (np.ascontiguousarray(s_pow2, dtype=np.float32).view(np.uint32) >> 23).astype(np.uint8)


def per_token_group_quant_fp8(x, group_size=128, eps=1e-10, in_dtype="bf16", scale_ue8m0=False):
    """Reference: native_per_token_group_quant_fp8, python/sglang/test/test_block_fp8.py:23-48.

    x: float32 array [..., K] holding values of `in_dtype`.  Returns
    (q uint8 [..., K], s float32 [..., K/group]) with s row-major.
    With scale_ue8m0 the scale is rounded up to a power of two before the divide
    (per_token_group_quant_8bit.cu:86-88,107).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.shape[-1] % group_size == 0
    g = x.reshape(-1, group_size)
    amax = np.maximum(np.abs(g).max(axis=-1, keepdims=True), clamp_eps(eps, in_dtype)).astype(np.float32)
    s = (amax / np.float32(FP8_MAX)).astype(np.float32)
    if scale_ue8m0:
        s = ceil_to_ue8m0(np.maximum(s, np.float32(1e-10)))
    with np.errstate(all="ignore"):
        y = (g / s).astype(np.float32)
    y = np.clip(y, np.float32(FP8_MIN), np.float32(FP8_MAX))
    q = f32_to_e4m3fn(y).reshape(x.shape)
    s = s.reshape(x.shape[:-1] + (x.shape[-1] // group_size,))
    return q, s


def pack_ue8m0_scales(s: np.ndarray) -> np.ndarray:
    """[M, G] power-of-two scales -> int32 words [M, ceil(G/4)] (logical view).

    Byte j%4 of word j//4 holds the exponent of group j; unused bytes are zero
    (per_token_group_quant_8bit.cu:54-61, per_token_group_quant_8bit_v2.cu:322-329).
    The device tensor stores this transposed (M contiguous, M padded to 4).
    """
    M, G = s.shape
    W = (G + 3) // 4
    by = np.zeros((M, W * 4), dtype=np.uint8)
    by[:, :G] = ue8m0_byte(s)
    return by.view("<u4").view(np.int32).reshape(M, W)


def unpack_ue8m0_scales(w: np.ndarray, G: int) -> np.ndarray:
    """Inverse of pack_ue8m0_scales; decode is (byte << 23) as float32 (fp8_utils.py:549-550)."""
    M = w.shape[0]
    by = np.ascontiguousarray(w, dtype=np.int32).view(np.uint8).reshape(M, -1)[:, :G]
    return (by.astype(np.uint32) << 23).view(np.float32)


# --------------------------------------------------------------------------
# a.6  per-token and per-tensor quant (reciprocal-multiply forms)
# --------------------------------------------------------------------------


def per_token_quant_fp8(x):
    """Reference: sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:44-70.

    scale = rowamax/448 (no eps); q = clamp(x * (1/scale)); an all-zero row gives
    scale 0 and scale_inv 0.  Returns (q uint8 [M,K], s float32 [M,1]).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    amax = np.abs(x).max(axis=-1, keepdims=True).astype(np.float32)
    s = (amax / np.float32(FP8_MAX)).astype(np.float32)
    with np.errstate(all="ignore"):
        inv = np.where(s == 0, np.float32(0), (np.float32(1.0) / s)).astype(np.float32)
    y = np.clip((x * inv).astype(np.float32), np.float32(FP8_MIN), np.float32(FP8_MAX))
    return f32_to_e4m3fn(y), s


def per_tensor_quant_fp8(x, static_scale=None):
    """Reference: sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:10-94.

    Dynamic: scale = absmax/448; both modes: q = clamp(x * (1/scale)).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    if static_scale is None:
        s = np.float32(np.abs(x).max() / np.float32(FP8_MAX)) if x.size else np.float32(0)
    else:
        s = np.float32(static_scale)
    with np.errstate(all="ignore"):
        inv = np.float32(1.0) / np.float32(s)
        y = np.clip((x * inv).astype(np.float32), np.float32(FP8_MIN), np.float32(FP8_MAX))
    return f32_to_e4m3fn(y), np.array([s], dtype=np.float32)


def per_tensor_quant_mla_fp8(x, eps=1e-12):
    """Reference: _per_tensor_quant_mla_fp8_stage1/2, python/sglang/srt/layers/quantization/fp8_kernel.py:1172-1266:
    every row contributes max(rowabsmax, eps) / 448 to an atomic maximum, then q = clamp(x * (1 / scale)) in float32.
    x float32 [H, S, D] (values of the input type) -> (q uint8 [H, S, D], scale float32 [1])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rowmax = np.maximum(np.abs(x).max(axis=-1), np.float32(eps)).astype(np.float32)
    s = np.float32((rowmax / np.float32(FP8_MAX)).astype(np.float32).max())
    inv = np.float32(1.0) / s
    y = np.clip((x * inv).astype(np.float32), np.float32(FP8_MIN), np.float32(FP8_MAX))
    return f32_to_e4m3fn(y), np.array([s], dtype=np.float32)


def bmm_fp8(Aq, Bq, a_scale, b_scale, out_dtype="bf16"):
    """Reference: sgl-kernel/python/sgl_kernel/gemm.py:66-82 with the check of sgl-kernel/tests/test_bmm_fp8.py:21-39
    (torch.bmm of the de-quantised operands).  Aq uint8 [b, m, k]; Bq uint8 [b, n, k] (the op's column-major [b, k, n]
    is this memory); one float32 scale per operand.  out[b] = (A[b] @ B[b]^T) * a_scale * b_scale."""
    A = e4m3fn_to_f32(Aq).astype(np.float64)
    B = e4m3fn_to_f32(Bq).astype(np.float64)
    C = np.einsum("bmk,bnk->bmn", A, B).astype(np.float32)
    C = C * np.float32(a_scale) * np.float32(b_scale)
    return _cast_out(C, out_dtype)


# --------------------------------------------------------------------------
# offline weight quant (test/srt/cpu/utils.py:39-87 semantics: amax/448 per block)
# --------------------------------------------------------------------------


def block_quant_weight(w, block_n=128, block_k=128):
    """w float32 [N,K] -> (q uint8 [N,K], s float32 [ceil(N/bn), ceil(K/bk)]); s = blockamax/448, 0 -> 1."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    nt, kt = (N + block_n - 1) // block_n, (K + block_k - 1) // block_k
    pad = np.zeros((nt * block_n, kt * block_k), dtype=np.float32)
    pad[:N, :K] = w
    blk = pad.reshape(nt, block_n, kt, block_k)
    amax = np.abs(blk).max(axis=(1, 3)).astype(np.float32)
    s = (amax / np.float32(FP8_MAX)).astype(np.float32)
    s = np.where(s == 0, np.float32(1), s)
    y = np.clip((blk / s[:, None, :, None]).astype(np.float32), np.float32(FP8_MIN), np.float32(FP8_MAX))
    q = f32_to_e4m3fn(y).reshape(nt * block_n, kt * block_k)[:N, :K]
    return np.ascontiguousarray(q), s


# --------------------------------------------------------------------------
# a.5  block-scaled matmul, a.6 scaled_mm
# --------------------------------------------------------------------------


def w8a8_block_fp8_matmul(Aq, Bq, As, Bs, block_size=(128, 128), out_dtype="bf16", acc=np.float32):
    """Reference: native_w8a8_block_fp8_matmul, python/sglang/test/test_block_fp8.py:273-325.

    Aq uint8 [M,K], Bq uint8 [N,K], As f32 [M, ceil(K/bk)], Bs f32 [ceil(N/bn), ceil(K/bk)].
    C = sum_i (A_i @ B_ji^T) * (As[:,i] * Bs[j,i]) accumulated tile by tile, then cast.
    `acc` float64 gives the mathematically tighter value used for tolerance checks.
    """
    bn, bk = block_size
    A = e4m3fn_to_f32(Aq).astype(acc)
    B = e4m3fn_to_f32(Bq).astype(acc)
    M, K = A.shape
    N = B.shape[0]
    nt, kt = (N + bn - 1) // bn, (K + bk - 1) // bk
    assert As.shape == (M, kt) and Bs.shape == (nt, kt)
    C = np.zeros((M, N), dtype=acc)
    for i in range(kt):
        a = A[:, i * bk : (i + 1) * bk]
        for j in range(nt):
            b = B[j * bn : (j + 1) * bn, i * bk : (i + 1) * bk]
            s = (As[:, i : i + 1].astype(acc) * acc(Bs[j, i])).astype(acc)
            C[:, j * bn : (j + 1) * bn] += (a @ b.T) * s
    return _cast_out(C, out_dtype)


def w8a16_block_fp8_matmul_cpu_twin(A, Bq, Bs, bias=None, block_size=(128, 128), acc=np.float32):
    """The ALGORITHM of the reference's CPU kernel fp8_scaled_mm_cpu for more than four rows
    (sgl-kernel/csrc/cpu/gemm_fp8.cpp:46-100, 256-298, 356-424).  W8A16 - NOT the W8A8 path of the rest of this
    file: a timing baseline and a sanity check, no bit oracle.  The bf16 activations A [M,K] are used unquantised;
    every weight element becomes bf16(float(w8) * Bs[n/bn, k/bk]); float accumulation over the whole K; + float
    bias; one rounding to bf16."""
    bn, bk = block_size
    A = to_bf16(np.asarray(A, dtype=np.float32))
    N, K = Bq.shape
    W = e4m3fn_to_f32(Bq)
    W = to_bf16(W * np.repeat(np.repeat(Bs, bn, axis=0)[:N], bk, axis=1)[:, :K])
    C = A.astype(acc) @ W.astype(acc).T
    if bias is not None:
        C = C + np.asarray(bias, dtype=np.float32).astype(acc)[None, :]
    return to_bf16(C.astype(np.float32))


def _cast_out(C, out_dtype):
    if out_dtype == "bf16":
        return to_bf16(C.astype(np.float32))
    if out_dtype == "f16":
        return C.astype(np.float32).astype(np.float16).astype(np.float32)
    return C.astype(np.float32)


def fp8_scaled_mm(Aq, Bq, sA, sB, out_dtype="bf16", bias=None):
    """Reference: torch_scaled_mm, sgl-kernel/tests/test_fp8_gemm.py:6-14; epilogue order
    sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:100-136.

    Aq uint8 [M,K]; Bq uint8 [N,K] (the op's mat_b is [K,N] column-major = this memory);
    sA f32 [M], sB f32 [N]; bias [N] added in float32 before the output cast.
    """
    A = e4m3fn_to_f32(Aq).astype(np.float64)
    B = e4m3fn_to_f32(Bq).astype(np.float64)
    C = (A @ B.T).astype(np.float32)
    C = C * np.asarray(sA, np.float32).reshape(-1, 1) * np.asarray(sB, np.float32).reshape(1, -1)
    if bias is not None:
        C = C + np.asarray(bias, np.float32).reshape(1, -1)
    return _cast_out(C, out_dtype)


def block_fp8_linear(x, Wq, Ws, bias=None, block_size=(128, 128)):
    """Reference: triton_w8a8_block_fp8_linear, python/sglang/srt/layers/quantization/fp8_utils.py:306-326.

    x bf16 values [..., K]; quant (a.1) -> block matmul (a.5) -> + bias in bf16 -> bf16.
    """
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    q, s = per_token_group_quant_fp8(x2, block_size[1])
    out = w8a8_block_fp8_matmul(q, Wq, s, Ws, block_size, "bf16")
    if bias is not None:
        out = to_bf16(out + np.asarray(bias, np.float32))
    return out.reshape(x.shape[:-1] + (Wq.shape[0],))


# --------------------------------------------------------------------------
# a.7  moe_align_block_size (integer)
# --------------------------------------------------------------------------


def moe_align_block_size(topk_ids, block_size, num_experts):
    """Reference: python/sglang/srt/layers/moe/fused_moe_triton/moe_align_block_size.py:17-82 and
    sgl-kernel/csrc/moe/moe_align_kernel.cu:56-228.

    topk_ids int [T, top_k] with values in [-1, num_experts).  The op is invoked with
    num_experts+1 buckets: bucket 0 collects id -1, bucket e+1 expert e.  Returns
    (sorted_ids int32[numel + (E+1)(B-1)], expert_ids int32[ceil(len/B)], num_post_pad int).
    Inside one expert the device order depends on atomics; the oracle uses ascending
    flat index, and tests compare per-expert sets.  expert_ids past num_post_pad/B are -2
    here (unspecified on device).
    """
    ids = np.asarray(topk_ids).reshape(-1).astype(np.int64)
    numel = ids.size
    E1 = num_experts + 1
    max_pad = numel + E1 * (block_size - 1)
    sorted_ids = np.full(max_pad, numel, dtype=np.int32)
    nblk = (max_pad + block_size - 1) // block_size
    expert_ids = np.full(nblk, -2, dtype=np.int32)
    pos = 0
    for b in range(E1):
        tok = np.nonzero(ids + 1 == b)[0]
        if tok.size == 0:
            continue
        padded = (tok.size + block_size - 1) // block_size * block_size
        sorted_ids[pos : pos + tok.size] = tok
        expert_ids[pos // block_size : (pos + padded) // block_size] = b - 1
        pos += padded
    return sorted_ids, expert_ids, pos


# --------------------------------------------------------------------------
# a.9 silu_and_mul, a.10 moe_sum_reduce, a.11 routing
# --------------------------------------------------------------------------


def silu_and_mul(x):
    """Reference: sgl-kernel/csrc/elementwise/activation.cu:56-60,85-105 (bf16: silu in f32, round
    to bf16, multiply, round to bf16).  x float32-of-bf16 [..., 2d] -> [..., d]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    d = x.shape[-1] // 2
    g, u = x[..., :d], x[..., d:]
    with np.errstate(over="ignore"):
        silu = to_bf16((g / (np.float32(1) + np.exp(-g).astype(np.float32))).astype(np.float32))
    return to_bf16((silu * u).astype(np.float32))


def gelu_and_mul(x):
    """Reference: sgl-kernel/csrc/elementwise/activation.cu:62-67,129-149 (bf16: v * (0.5 * (1 + erf(v / sqrt 2))) in
    f32 operation by operation, round to bf16, multiply, round to bf16).  x float32-of-bf16 [..., 2d] -> [..., d].
    erf is taken in float64 and rounded once (a correctly rounded erff; device libraries are within a few ulp of it)."""
    from scipy.special import erf

    x = np.ascontiguousarray(x, dtype=np.float32)
    d = x.shape[-1] // 2
    g, u = x[..., :d], x[..., d:]
    t = (g * np.float32(0.70710678118654752440)).astype(np.float32)
    cdf = (np.float32(0.5) * (np.float32(1) + erf(t.astype(np.float64)).astype(np.float32))).astype(np.float32)
    gelu = to_bf16((g * cdf).astype(np.float32))
    return to_bf16((gelu * u).astype(np.float32))


def activation_only(x, kind):
    """Reference: the ungated branch of fused_experts_impl, fused_moe.py:566-572 - F.silu, F.gelu (erf form),
    torch.square(F.relu(.)) on a 16-bit tensor: the function in float32, one rounding to bf16.
    x float32-of-bf16 -> same shape."""
    from scipy.special import erf

    x = np.ascontiguousarray(x, dtype=np.float32)
    if kind == "silu":
        with np.errstate(over="ignore"):
            y = x / (np.float32(1) + np.exp(-x).astype(np.float32))
    elif kind == "gelu":
        t = (x * np.float32(0.70710678118654752440)).astype(np.float32)
        y = x * (np.float32(0.5) * (np.float32(1) + erf(t.astype(np.float64)).astype(np.float32))).astype(np.float32)
    elif kind == "relu2":
        r = np.maximum(x, np.float32(0))
        with np.errstate(over="ignore"):
            y = r * r
    else:
        raise ValueError(kind)
    return to_bf16(y.astype(np.float32))


def silu_mul_per_token_group_quant_fp8(x, group_size=128, eps=1e-10, scale_ue8m0=False):
    """Reference: sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:336-341 (FUSE_SILU_AND_MUL: the value that
    is quantised is T(T(silu(gate))) * up in the input type T) - i.e. silu_and_mul followed by the group quant.
    x float32-of-bf16 [M, 2K] -> (q [M, K], scales)."""
    return per_token_group_quant_fp8(silu_and_mul(x), group_size, eps=eps, scale_ue8m0=scale_ue8m0)


def moe_sum_reduce(x, routed_scaling_factor=1.0):
    """Reference: sgl-kernel/csrc/moe/moe_sum_reduce.cu:56-113: out[t] = bf16(rsf * sum_k f32(x[t,k])),
    k ascending, float32 accumulation."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    acc = np.zeros((x.shape[0], x.shape[2]), dtype=np.float32)
    for k in range(x.shape[1]):
        acc = (acc + x[:, k, :]).astype(np.float32)
    return to_bf16((acc * np.float32(routed_scaling_factor)).astype(np.float32))


def moe_sum(x):
    """Reference: sgl-kernel/csrc/moe/moe_sum.cu:11-69.  x float32-of-bf16 [T, topk, H] -> [T, H]: for 2, 3 and 4
    experts per token the sum runs in the element type (a bf16 rounding after every addition, ascending k, starting from
    zero), otherwise at::sum_out (float accumulation, one rounding)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    topk = x.shape[1]
    if topk in (2, 3, 4):
        acc = np.zeros((x.shape[0], x.shape[2]), dtype=np.float32)
        for k in range(topk):
            acc = to_bf16(acc + x[:, k])
        return acc
    return to_bf16(x.astype(np.float64).sum(axis=1).astype(np.float32))


def biased_grouped_topk(logits, bias, num_expert_group, topk_group, topk, renormalize=True):
    """Reference: biased_grouped_topk_impl, python/sglang/srt/layers/moe/topk.py:665-738.

    sigmoid scores; group score = sum of the top-2 (score+bias) in each group; keep the best
    `topk_group` groups; top-k over the kept experts by (score+bias); weights are the un-biased
    scores, renormalised.  Returns (weights f32 [T,topk], ids int32 [T,topk])."""
    logits = np.asarray(logits, np.float32)
    T, E = logits.shape
    scores = (np.float32(1) / (np.float32(1) + np.exp(-logits))).astype(np.float32)
    sc = scores + (0 if bias is None else np.asarray(bias, np.float32)[None, :])
    grp = sc.reshape(T, num_expert_group, E // num_expert_group)
    top2 = -np.sort(-grp, axis=-1)[..., :2].sum(-1)
    gidx = np.argsort(-top2, axis=-1, kind="stable")[:, :topk_group]
    gmask = np.zeros((T, num_expert_group), dtype=bool)
    np.put_along_axis(gmask, gidx, True, axis=1)
    emask = np.repeat(gmask, E // num_expert_group, axis=1)
    masked = np.where(emask, sc, -np.inf)
    ids = np.argsort(-masked, axis=-1, kind="stable")[:, :topk]
    w = np.take_along_axis(scores, ids, axis=1)
    if renormalize:
        w = w / w.sum(-1, keepdims=True)
    return w.astype(np.float32), ids.astype(np.int32)


def moe_fused_gate(x, bias, num_expert_group, topk_group, topk, num_fused_shared_experts=0,
                   routed_scaling_factor=0.0, apply_routed_scaling_factor_on_output=False, in_dtype="f32"):
    """Reference: moe_fused_gate_impl, sgl-kernel/csrc/moe/moe_fused_gate.cu:52-257, followed step by step
    (pure-Python loops: small cases only).  Arithmetic happens in the input type T: T(sigmoid), T(score + bias),
    T(top1 + top2) per group; the weakest group is dropped repeatedly (ties: the higher group goes), then the best
    remaining expert is taken repeatedly (ties: the lower expert wins).  x [rows, E] and bias [E] hold values of
    `in_dtype` ("f32" or "bf16").  Returns (weights f32 [rows, topk], ids int32 [rows, topk])."""
    rnd = to_bf16 if in_dtype == "bf16" else (lambda a: np.asarray(a, np.float32))
    x = np.asarray(x, np.float32)
    bias = np.asarray(bias, np.float32)
    rows, E = x.shape
    vpt = E // num_expert_group
    take = topk - num_fused_shared_experts
    out_w = np.zeros((rows, topk), np.float32)
    out_i = np.zeros((rows, topk), np.int32)
    with np.errstate(over="ignore"):
        score = rnd((np.float32(1) / (np.float32(1) + np.exp(-x).astype(np.float32))).astype(np.float32))
    choice_all = rnd((score + bias[None, :]).astype(np.float32))
    for r in range(rows):
        choice = choice_all[r].copy().reshape(num_expert_group, vpt)
        for _ in range(num_expert_group - topk_group):
            srt = -np.sort(-choice, axis=1)
            sums = rnd((srt[:, 0] + srt[:, 1]).astype(np.float32)) if vpt > 1 else srt[:, 0]
            worst = max(g for g in range(num_expert_group) if sums[g] == sums.min())
            choice[worst, :] = np.inf
        flat = np.where(np.isinf(choice) & (choice > 0), -np.inf, choice).reshape(-1)
        wsum = np.float32(0)
        for k in range(take):
            e = int(np.argmax(flat))  # first maximum = lowest index
            out_i[r, k] = e
            out_w[r, k] = score[r, e]
            wsum = np.float32(wsum + score[r, e])
            flat[e] = -np.inf
        for i in range(num_fused_shared_experts):
            out_i[r, take + i] = E + i
            out_w[r, take + i] = np.float32(np.float64(wsum) / routed_scaling_factor)
        w = (out_w[r] / wsum).astype(np.float32)
        if apply_routed_scaling_factor_on_output:
            w = (w.astype(np.float64) * routed_scaling_factor).astype(np.float32)
        out_w[r] = w
    return out_w, out_i


# --------------------------------------------------------------------------
# a.8 + pipeline: block-FP8 fused MoE
# --------------------------------------------------------------------------


def fused_moe_block_fp8(x, w13q, w13s, w2q, w2s, topk_w, topk_ids, routed_scaling_factor=1.0, block=(128, 128),
                        apply_router_weight_on_input=False, activation="silu", is_gated=True):
    """Reference: fused_experts_impl, python/sglang/srt/layers/moe/fused_moe_triton/fused_moe.py:498-639
    (sequence) and torch_w8a8_block_fp8_moe, python/sglang/test/test_block_fp8.py:418-447 (math).

    x bf16 values [T,H]; w13q uint8 [E,2I,H]; w2q uint8 [E,H,I]; scales per 128x128 block.
    quant(x) -> GEMM1 -> silu_and_mul (gelu_and_mul with activation="gelu", fused_moe.py:547-565; with is_gated=False
    w13q is [E,I,H] and the activation - silu, gelu or relu2 - keeps the width, :566-572) -> quant ->
    GEMM2 * topk_weight (f32, then bf16) -> sum over k in f32 * routed_scaling_factor -> bf16.
    apply_router_weight_on_input (fused_moe.py:533,597; the kernel multiplies the float accumulator before the output
    cast, fused_moe_triton_kernels.py MUL_ROUTED_WEIGHT): the weight multiplies the result of GEMM 1 instead.
    """
    T, H = x.shape
    E, I2, _ = w13q.shape
    topk = topk_ids.shape[1]
    xq, xs = per_token_group_quant_fp8(x, block[1])
    inter = np.zeros((T, topk, H), dtype=np.float32)
    for e in range(E):
        t_idx, k_idx = np.nonzero(topk_ids == e)
        if t_idx.size == 0:
            continue
        wk = topk_w[t_idx, k_idx][:, None].astype(np.float32)
        if apply_router_weight_on_input:
            h1 = to_bf16((w8a8_block_fp8_matmul(xq[t_idx], w13q[e], xs[t_idx], w13s[e], block, "f32") * wk).astype(np.float32))
        else:
            h1 = w8a8_block_fp8_matmul(xq[t_idx], w13q[e], xs[t_idx], w13s[e], block, "bf16")
        act = {"silu": silu_and_mul, "gelu": gelu_and_mul}[activation](h1) if is_gated else activation_only(h1, activation)
        aq, as_ = per_token_group_quant_fp8(act, block[1])
        h2 = w8a8_block_fp8_matmul(aq, w2q[e], as_, w2s[e], block, "f32")
        inter[t_idx, k_idx] = to_bf16(h2 if apply_router_weight_on_input else (h2 * wk).astype(np.float32))
    return moe_sum_reduce(inter, routed_scaling_factor)


# --------------------------------------------------------------------------
# expert-major ("CUTLASS") form of the fused experts
# --------------------------------------------------------------------------


def prepare_moe_input(topk_ids, num_experts, n, k):
    """Reference: sgl-kernel/csrc/moe/prepare_moe_input.cu:12-141.  topk_ids int32 [m, topk] ->
    (expert_offsets [E+1], blockscale_offsets [E+1], problem_sizes1 [E,3], problem_sizes2 [E,3], a_map, c_map).
    The reference hands out the rows of an expert through an atomic counter, so their order inside the expert is not
    defined; this restatement takes the slots in ascending order (one of the orders the reference can produce)."""
    ids = np.asarray(topk_ids, dtype=np.int64)
    topk = ids.shape[1]
    flat = ids.reshape(-1)
    counts = np.array([(flat == e).sum() for e in range(num_experts)], dtype=np.int32)
    offsets = np.zeros(num_experts + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(counts)
    bs_offsets = np.zeros(num_experts + 1, dtype=np.int32)
    bs_offsets[1:] = np.cumsum((counts + 127) // 128 * 128)
    ps1 = np.stack([counts, np.full_like(counts, 2 * n), np.full_like(counts, k)], axis=1).astype(np.int32)
    ps2 = np.stack([counts, np.full_like(counts, k), np.full_like(counts, n)], axis=1).astype(np.int32)
    a_map = np.zeros(flat.size, dtype=np.int32)
    c_map = np.zeros(flat.size, dtype=np.int32)
    cursor = offsets[:-1].copy()
    for i, e in enumerate(flat):
        if 0 <= e < num_experts:
            a_map[cursor[e]] = i // topk
            c_map[i] = cursor[e]
            cursor[e] += 1
    return offsets, bs_offsets, ps1, ps2, a_map, c_map


def shuffle_rows(x, dst2src_map):
    """Reference: prepare_moe_input.cu:169-193: out[d] = x[dst2src_map[d]]."""
    return np.ascontiguousarray(np.asarray(x)[np.asarray(dst2src_map, dtype=np.int64)])


def apply_shuffle_mul_sum(x, permutation, factors, out_dtype="bf16"):
    """Reference: prepare_moe_input.cu:252-310: out[t] = T(sum_j f32(factors[t*topk+j]) * f32(x[perm[t*topk+j]])), float32
    accumulation in ascending j (the product of two 16-bit values is exact in float32, so a fused multiply-add and a
    multiply followed by an add give the same sum).  x float32 values of the element type [m*topk, k]; permutation
    [m, topk]; factors float32 values of the element type [m, topk] or None."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    perm = np.asarray(permutation, dtype=np.int64)
    m, topk = perm.shape
    acc = np.zeros((m, x.shape[1]), dtype=np.float32)
    for j in range(topk):
        f = np.float32(1.0) if factors is None else np.asarray(factors, dtype=np.float32)[:, j][:, None]
        acc = (acc + (f * x[perm[:, j]]).astype(np.float32)).astype(np.float32)
    return _cast_out(acc, out_dtype)


def fp8_blockwise_scaled_grouped_mm(Aq, Bq, As, Bs, expert_offsets, problem_sizes, out_dtype="bf16", acc=np.float32):
    """Reference: sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu with the check of sgl-kernel/tests/
    test_fp8_blockwise_moe.py:109-216: for every expert e, rows [expert_offsets[e], + problem_sizes[e, 0]) of A times
    that expert's weight, 1x128 scales on A and 128x128 scales on B.  Aq uint8 [rows, K]; Bq uint8 [E, N, K];
    As f32 [rows, K/128]; Bs f32 [E, N/128, K/128].  Rows that no expert owns stay zero."""
    E, N, _ = Bq.shape
    out = np.zeros((Aq.shape[0], N), dtype=np.float32)
    for e in range(E):
        r0, cnt = int(expert_offsets[e]), int(problem_sizes[e][0])
        if cnt:
            out[r0:r0 + cnt] = w8a8_block_fp8_matmul(Aq[r0:r0 + cnt], Bq[e], As[r0:r0 + cnt], Bs[e], (128, 128), out_dtype, acc=acc)
    return out


def cutlass_fused_experts_fp8(x, w13q, w13s, w2q, w2s, topk_w, topk_ids, out_dtype="bf16"):
    """Reference: cutlass_fused_experts_fp8, python/sglang/srt/layers/moe/cutlass_moe.py:119-247: prepare_moe_input ->
    group quant of x -> rows replicated into expert order -> grouped GEMM 1 (out dtype) -> silu_and_mul -> group quant
    -> grouped GEMM 2 (out dtype) -> apply_shuffle_mul_sum with topk_weights cast to the out dtype.
    x bf16 values [m, k]; w13q uint8 [E, 2n, k]; w2q uint8 [E, k, n]; topk_w float32 [m, topk]."""
    E = w13q.shape[0]
    n = w2q.shape[2]
    k = x.shape[1]
    offsets, _, ps1, ps2, a_map, c_map = prepare_moe_input(topk_ids, E, n, k)
    xq, xs = per_token_group_quant_fp8(x, 128)
    c1 = fp8_blockwise_scaled_grouped_mm(shuffle_rows(xq, a_map), w13q, shuffle_rows(xs, a_map), w13s, offsets, ps1, out_dtype)
    iq, is_ = per_token_group_quant_fp8(silu_and_mul(c1), 128)
    c2 = fp8_blockwise_scaled_grouped_mm(iq, w2q, is_, w2s, offsets, ps2, out_dtype)
    return apply_shuffle_mul_sum(c2, c_map.reshape(topk_ids.shape), _cast_out(np.asarray(topk_w, np.float32), out_dtype), out_dtype)


# --------------------------------------------------------------------------
# seeded synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------


def make_activation(M, K, seed, outlier_frac=1e-3, outlier_mul=50.0):
    """bf16 activations: N(0,1) with a fraction of entries scaled up (numpy Generator, PCG64)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K), dtype=np.float32)
    mask = rng.random((M, K), dtype=np.float32) < outlier_frac
    x = np.where(mask, x * np.float32(outlier_mul), x)
    return to_bf16(x)


def make_weight(N, K, seed, std=0.02):
    rng = np.random.default_rng(seed + 1000003)
    return to_bf16(rng.standard_normal((N, K), dtype=np.float32) * np.float32(std))
