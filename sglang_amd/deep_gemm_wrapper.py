"""The three block-FP8 GEMM entry points that SGLang's DeepGEMM runner calls, on this library's kernels.

Reference: python/sglang/srt/layers/deep_gemm_wrapper/entrypoint.py:26-88 (thin wrappers over the third-party
`deep_gemm` package, not vendored in the reference; its published layouts are restated here):

* gemm_nt_f8f8bf16            lhs (a [m,k] e4m3fn, a_s [m,k/128] f32), rhs (b [n,k], b_s [n/128,k/128]) -> out [m,n]
* grouped ... contig          lhs rows of all groups concatenated, `m_indices[i]` = group of row i, -1 = skip the row
* grouped ... masked          lhs [G,m_max,k]; only the first masked_m[g] rows of group g are computed

All three are the 128x128 block-scaled product `out = sum_kb (a_kb . b_kb^T) * a_s[:,kb] * b_s[nb,kb]` with float32
accumulation.  The grouped forms run on the grouped MoE GEMM: the group of every row becomes its "expert id"
(rows to skip get an id the aligner ignores, so they are neither computed nor written), moe_align_block_size
sorts the rows into per-group blocks, and each row is its own token slot (top_k = 1, no routed weight).
Scales are float32, or packed UE8M0 words (int32: [.., m, ceil(k/128/4)] for the activations, one row per weight row
[.., n, ceil(k/128/4)] for the weights, the layout the reference prepares for DeepGEMM on Blackwell, fp8_kernel.py:
1018-1043); the grouped kernels take float scales, so packed words are expanded to powers of two first.  When BOTH
tensors arrive packed every scale is a power of two, and 256-row blocks let the matrix cores apply them
(fp8k_moe_block_gemm_ue8m0) instead of the float promote.
"""
from typing import Tuple

import torch

from . import custom_ops as _ops
from .fp8_kernel import w8a8_block_fp8_matmul
from .fused_moe import SORT_SCALES_MIN_BLOCK, get_default_config, moe_align_block_size
from .sgl_kernel import unpack_ue8m0_scales, unpack_ue8m0_weight_scales

_IGNORED = -2  # moe_align_block_size drops ids below -1


def _check_pair(name: str, x: Tuple[torch.Tensor, torch.Tensor]) -> None:
    q, s = x
    if q.dtype != torch.float8_e4m3fn:
        raise RuntimeError("%s: data must be float8_e4m3fn" % name)
    if s.dtype not in (torch.float32, torch.int32):
        raise RuntimeError("%s: scales must be float32 or packed int32 UE8M0 words" % name)


def _float_scales(a, a_s, b, b_s):
    """Packed UE8M0 words -> float32 powers of two (activations per row, weights per 128-row block); the third
    result says whether both tensors came packed (then every scale is a power of two by construction)."""
    k = a.shape[-1]
    pow2 = a_s.dtype == torch.int32 and b_s.dtype == torch.int32
    if a_s.dtype == torch.int32:
        a_s = unpack_ue8m0_scales(a_s, (k + 127) // 128)
    if b_s.dtype == torch.int32:
        b_s = unpack_ue8m0_weight_scales(b_s, k)
    return a_s, b_s, pow2


def gemm_nt_f8f8bf16(lhs: Tuple[torch.Tensor, torch.Tensor], rhs: Tuple[torch.Tensor, torch.Tensor], out: torch.Tensor):
    """Reference: entrypoint.py:70-88 (deep_gemm.fp8_gemm_nt)."""
    _check_pair("lhs", lhs)
    _check_pair("rhs", rhs)
    a, a_s = lhs
    b, b_s = rhs
    res = w8a8_block_fp8_matmul(a, b, a_s, b_s, [128, 128], out.dtype)
    out.copy_(res)


def _grouped(a, a_s, b, b_s, out, row_group: torch.Tensor, rows_per_group: int, pow2: bool) -> None:
    G = b.shape[0]
    rows = a.shape[0]
    if rows == 0:
        return
    block_m = get_default_config(max(rows_per_group, 1) * G, G, 1)["BLOCK_SIZE_M"]
    sorted_ids, expert_ids, num_post_pad = moe_align_block_size(row_group, block_m, G)
    if block_m >= SORT_SCALES_MIN_BLOCK:
        # as in the fused-MoE layer: the activation scales first go into the order of the sorted rows; with both tensors
        # packed and 256-row blocks the matrix cores then apply the exponents themselves
        a_s = _ops.moe_sort_scales(a_s, sorted_ids, num_post_pad, 1, rows)
        _ops.moe_block_gemm(a, b, out, a_s, b_s, None, sorted_ids, expert_ids, num_post_pad, False, 1, block_m, rows,
                            True, pow2 and block_m == 256)
        return
    _ops.moe_block_gemm(a, b, out, a_s, b_s, None, sorted_ids, expert_ids, num_post_pad, False, 1, block_m, rows)


def grouped_gemm_nt_f8f8bf16_contig(
    lhs: Tuple[torch.Tensor, torch.Tensor], rhs: Tuple[torch.Tensor, torch.Tensor], out: torch.Tensor,
    m_indices: torch.Tensor,
):
    """Reference: entrypoint.py:52-67 (deep_gemm.m_grouped_fp8_gemm_nt_contiguous).  Rows with m_indices == -1
    are left untouched in `out`."""
    _check_pair("lhs", lhs)
    _check_pair("rhs", rhs)
    a, a_s = lhs
    b, b_s = rhs
    a_s, b_s, pow2 = _float_scales(a, a_s, b, b_s)
    if a.dim() != 2 or b.dim() != 3 or m_indices.numel() != a.shape[0]:
        raise RuntimeError("grouped_gemm_nt_f8f8bf16_contig: lhs [m,k], rhs [G,n,k], m_indices [m]")
    idx = m_indices.to(torch.int32)
    idx = torch.where(idx < 0, torch.full_like(idx, _IGNORED), idx)
    _grouped(a, a_s, b, b_s, out, idx, (a.shape[0] + b.shape[0] - 1) // b.shape[0], pow2)


def grouped_gemm_nt_f8f8bf16_masked(
    lhs: Tuple[torch.Tensor, torch.Tensor], rhs: Tuple[torch.Tensor, torch.Tensor], out: torch.Tensor,
    masked_m: torch.Tensor, expected_m: int,
):
    """Reference: entrypoint.py:26-49 (deep_gemm.fp8_m_grouped_gemm_nt_masked).  Rows at or past masked_m[g] are
    left untouched in `out`; `expected_m` (the typical rows per group) only picks the block size."""
    _check_pair("lhs", lhs)
    _check_pair("rhs", rhs)
    a, a_s = lhs
    b, b_s = rhs
    a_s, b_s, pow2 = _float_scales(a, a_s, b, b_s)
    if a.dim() != 3 or b.dim() != 3 or a.shape[0] != b.shape[0] or masked_m.numel() != a.shape[0]:
        raise RuntimeError("grouped_gemm_nt_f8f8bf16_masked: lhs [G,m_max,k], rhs [G,n,k], masked_m [G]")
    G, m_max, k = a.shape
    if not (a.is_contiguous() and out.is_contiguous()) or a_s.shape[:2] != (G, m_max):
        raise RuntimeError("grouped_gemm_nt_f8f8bf16_masked: lhs and out must be contiguous, scales [G,m_max,k/128]")
    dev = a.device
    row = torch.arange(m_max, device=dev, dtype=torch.int32)[None, :]
    grp = torch.arange(G, device=dev, dtype=torch.int32)[:, None]
    idx = torch.where(row < masked_m.to(torch.int32)[:, None], grp, torch.full_like(grp, _IGNORED)).reshape(-1)
    _grouped(a.view(G * m_max, k), a_s.reshape(G * m_max, -1), b, b_s, out.view(G * m_max, -1), idx, max(int(expected_m), 1), pow2)
