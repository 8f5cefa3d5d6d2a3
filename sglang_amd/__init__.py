"""MI355X-native W8A8 FP8 linear path behind SGLang's operator signatures.

Modules:
  sgl_kernel  - the ops SGLang reaches through ``sgl_kernel`` (quant, GEMMs, MoE helpers)
  fp8_kernel  - ``sglang.srt.layers.quantization.fp8_kernel`` entry points
  fp8_utils   - ``sglang.srt.layers.quantization.fp8_utils`` entry points (linear apply)
  fused_moe   - block-FP8 fused-experts pipeline
"""
from . import _lib  # noqa: F401  (fails loudly when the HIP library is not built)

__all__ = ["sgl_kernel", "fp8_kernel", "fp8_utils", "fused_moe"]
