"""C-ABI checks that need no GPU: the library loads, exports every symbol the headers under include/ declare,
and rejects bad arguments with a status and a message before touching the device."""
import ctypes
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = sorted(glob.glob(os.path.join(ROOT, "include", "*.h")))


def _declared_symbols():
    syms = set()
    for header in HEADERS:
        text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
        syms.update(re.findall(r"\b(fp8k_[a-z0-9_]+)\s*\(", text))
    return sorted(syms)


def test_library_exports_every_declared_symbol():
    from sglang_amd import _lib

    syms = _declared_symbols()
    assert len(syms) >= 9
    for s in syms:
        assert hasattr(_lib.lib, s), "libfp8k.so does not export %s" % s
        assert s in _lib.SIGNATURES, "Python binding has no signature for %s" % s
    assert sorted(_lib.SIGNATURES) == syms
    assert _lib.lib.fp8k_abi_version() == _lib.ABI_VERSION


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    import importlib

    from sglang_amd import _lib

    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib._load()
    importlib.reload(_lib)


def test_invalid_arguments_are_rejected_on_the_host():
    from sglang_amd import _lib

    lib = _lib.lib
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p = (p + 255) // 256 * 256
    # K not divisible by the group size
    rc = lib.fp8k_group_quant(p, p, p, 4, 100, 128, 1e-10, -448.0, 448.0, _lib.BF16, 1, 1, 0, None)
    assert rc == 1 and b"group_size" in lib.fp8k_last_error()
    # fnuz range is refused: gfx950 is OCP e4m3fn
    rc = lib.fp8k_group_quant(p, p, p, 4, 128, 128, 1e-10, -224.0, 224.0, _lib.BF16, 1, 1, 0, None)
    assert rc == 1 and b"448" in lib.fp8k_last_error()
    rc = lib.fp8k_group_quant(p, p, p, 4, 128, 48, 1e-10, -448.0, 448.0, _lib.BF16, 1, 1, 0, None)
    assert rc == 1
    rc = lib.fp8k_group_quant(None, p, p, 4, 128, 128, 1e-10, -448.0, 448.0, _lib.BF16, 1, 1, 0, None)
    assert rc == 1 and b"null" in lib.fp8k_last_error()
    rc = lib.fp8k_group_quant(p, p, p, 4, 256, 64, 1e-10, -448.0, 448.0, _lib.BF16, 1, 1, 1, None)
    assert rc == 1 and b"UE8M0" in lib.fp8k_last_error()
    # empty input is a no-op
    assert lib.fp8k_group_quant(None, None, None, 0, 128, 128, 1e-10, -448.0, 448.0, _lib.BF16, 1, 1, 0, None) == 0
    assert lib.fp8k_last_error() == b""
    # GEMM: out dtype, alignment, workspace
    rc = lib.fp8k_block_gemm(p, p, p, p, p, 4, 256, 256, 256, 256, 2, 1, 2, 1, 256, _lib.F32, None, 0, None)
    assert rc == 1 and b"Half or BFloat16" in lib.fp8k_last_error()
    rc = lib.fp8k_block_gemm(p, p, p, p, p, 4, 256, 250, 250, 250, 2, 1, 2, 1, 256, _lib.BF16, None, 0, None)
    assert rc == 1 and b"16 bytes" in lib.fp8k_last_error()
    rc = lib.fp8k_block_gemm(p, p, p, p, p, 4, 250, 256, 256, 256, 2, 1, 2, 1, 250, _lib.BF16, None, 0, None)
    assert rc == 1
    need = lib.fp8k_block_gemm_workspace_bytes(16, 7168, 16384)
    assert need > 0
    rc = lib.fp8k_block_gemm(p, p, p, p, p, 16, 7168, 16384, 16384, 16384, 128, 1, 128, 1, 7168, _lib.BF16, None, 0, None)
    assert rc == 4 and b"workspace" in lib.fp8k_last_error()
    # no K cut at this shape: only the area for a column-major copy of the activation scales
    assert lib.fp8k_block_gemm_workspace_bytes(4096, 7168, 16384) == 4096 * 128 * 4
    assert lib.fp8k_scaled_mm_workspace_bytes(4096, 7168, 16384) == 0
    rc = lib.fp8k_token_quant(p, p, p, 4, 100, _lib.BF16, None)
    assert rc == 1 and b"divisible by 8" in lib.fp8k_last_error()
    rc = lib.fp8k_scaled_mm(p, p, p, p, p, p, 4, 256, 256, 256, 256, 256, _lib.BF16, 7, None, 0, None)
    assert rc == 1 and b"bias" in lib.fp8k_last_error()


def test_python_wrappers_reject_cpu_tensors():
    import torch

    from sglang_amd.sgl_kernel import fp8_scaled_mm, sgl_per_token_group_quant_8bit

    x = torch.zeros((4, 128), dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        sgl_per_token_group_quant_8bit(x, torch.empty((4, 128), dtype=torch.float8_e4m3fn), torch.empty((4, 1)), 128,
                                       1e-10, -448.0, 448.0)
    a = torch.zeros((4, 128), dtype=torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="GPU"):
        fp8_scaled_mm(a, a.t(), torch.ones(4), torch.ones(4), torch.bfloat16)


def test_scale_layout_factory_matches_reference_shapes():
    """python/sglang/srt/layers/quantization/fp8_kernel.py:437-478."""
    import torch

    from sglang_amd.fp8_kernel import create_per_token_group_quant_fp8_output_scale as mk

    s = mk((45, 7168), "cpu", 128, False, False, False)
    assert s.shape == (45, 56) and s.is_contiguous() and s.dtype == torch.float32
    s = mk((45, 7168), "cpu", 128, True, False, False)
    assert s.shape == (45, 56) and s.stride() == (1, 45)
    s = mk((45, 7168), "cpu", 128, True, True, False)
    assert s.shape == (45, 56) and s.stride() == (1, 48)
    s = mk((45, 7168), "cpu", 128, True, True, True)
    assert s.shape == (45, 14) and s.stride() == (1, 48) and s.dtype == torch.int32
    s = mk((45, 640), "cpu", 128, True, True, True)
    assert s.shape == (45, 2)
