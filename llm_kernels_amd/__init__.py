"""llm_kernels_amd -- MI355X (gfx950) kernels behind the LLM_Kernels quantized-GEMM Python API.

Sub-packages mirror the reference's module paths:
    quantization.{fp8_kernel,int8_kernel,w4a8_kernel,bitpack,quant_utils}
    fast_dequant.simple_marlin.{utils,marlin}
    moe.{group_gemm_kernel,ep_moe}
Putting this directory on sys.path makes `import quantization.fp8_kernel` etc. resolve here.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
