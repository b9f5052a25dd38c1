"""Block quantisers of the communication payloads on MI355X (reference quant_communication/quant_utils.py).

int8_quant (:35), int8_dequant (:88), fp8_quant (:137), fp8_dequant (:186) keep their names, signatures and
quirks: int8 rounds half up (`floor(x / s + 0.5)`, :27), both quantisers store the scale as float16 (:53,
:152 -- the fp8 docstring says float32, the code float16), and the dequantisers multiply in the dtype of the
scale before casting to `output_dtype` (:80, :180).  Only the single-GPU payload kernels are here; the
collectives that would carry the payload are outside this library.
"""
from typing import Tuple

import torch

try:
    from .. import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib


def int8_quant(x: torch.Tensor, block_size: int = 32) -> Tuple[torch.Tensor, torch.Tensor]:
    """1 x block_size groups: s = max|x| / 127 (fp32), y = floor(x / s + 0.5) as int8, s stored as float16."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    _lib.require_gpu(x)
    y = torch.empty_like(x, dtype=torch.int8)
    s = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float16)
    _lib.call("llmk_act_quant_i8", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s),
              x.numel() // block_size, block_size, 1, _lib.stream(x), exc=AssertionError)
    return y, s


def _dequant(y, s, output_dtype, kind):
    assert y.is_contiguous() and s.is_contiguous(), 'Input tensors must be contiguous'
    assert y.size(-1) % s.size(-1) == 0, "Last dimension of y must be a multiple of last dimension of s"
    _lib.require_gpu(y, s)
    block_size = y.size(-1) // s.size(-1)
    x = torch.empty_like(y, dtype=output_dtype)
    _lib.call("llmk_comm_dequant", _lib.ptr(y), kind, _lib.ptr(s), _lib.dt(s.dtype), _lib.ptr(x), _lib.dt(output_dtype),
              s.numel(), block_size, _lib.stream(y), exc=AssertionError)
    return x


def int8_dequant(y: torch.Tensor, s: torch.Tensor, output_dtype: torch.dtype) -> torch.Tensor:
    """x = (y as s.dtype) * s, rounded in s.dtype, cast to output_dtype."""
    assert y.dtype == torch.int8, "Input y must be torch.int8"
    return _dequant(y, s, output_dtype, _lib.KIND_I8)


def fp8_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """1 x block_size groups: s = max|x| / 448 (fp32), y = (x / s) as float8_e4m3fn, s stored as float16."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    _lib.require_gpu(x)
    y = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    s = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float16)
    _lib.call("llmk_comm_quant_fp8", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s), _lib.dt(s.dtype),
              x.numel() // block_size, block_size, _lib.stream(x), exc=AssertionError)
    return y, s


def fp8_dequant(y: torch.Tensor, s: torch.Tensor, output_dtype: torch.dtype) -> torch.Tensor:
    """x = (y as s.dtype) * s, rounded in s.dtype, cast to output_dtype."""
    assert y.dtype == torch.float8_e4m3fn, "Input y must be torch.float8_e4m3fn"
    return _dequant(y, s, output_dtype, _lib.KIND_FP8)
