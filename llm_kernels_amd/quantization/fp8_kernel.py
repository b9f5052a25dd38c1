"""DeepSeek-V3 style blockwise FP8 (OCP e4m3) quantisation and GEMM on MI355X.

Same functions as the reference quantization/fp8_kernel.py: act_quant (:33), weight_dequant (:84),
fp8_gemm (:170); weight_quant is the 128x128 weight analogue the reference lacks.  The bodies
validate like the reference (AssertionError), allocate the outputs and call the HIP kernels.
"""
from typing import Tuple

import torch

try:
    from .. import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib


def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """1 x block_size groups: s = max|x| / 448 (fp32), y = (x / s) as float8_e4m3fn."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    _lib.require_gpu(x)
    y = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    s = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float32)
    _lib.call("llmk_act_quant_fp8", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s),
              x.numel() // block_size, block_size, _lib.stream(x))
    return y, s


def weight_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """block x block tiles of W [N, K]: s = blockmax / 448 (fp32), y = (x / s) as float8_e4m3fn."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.dim() == 2, 'Input tensors must have 2 dimensions'
    _lib.require_gpu(x)
    M, N = x.size()
    y = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    s = x.new_empty(((M + block_size - 1) // block_size, (N + block_size - 1) // block_size), dtype=torch.float32)
    _lib.call("llmk_weight_quant_fp8_block", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s),
              M, N, block_size, _lib.stream(x))
    return y, s


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """y = fp32(x) * s[block] in torch's default dtype."""
    assert x.is_contiguous() and s.is_contiguous(), 'Input tensors must be contiguous'
    assert x.dim() == 2 and s.dim() == 2, 'Input tensors must have 2 dimensions'
    _lib.require_gpu(x, s)
    M, N = x.size()
    y = torch.empty_like(x, dtype=torch.get_default_dtype())
    s32 = s if s.dtype == torch.float32 else s.float()     # held until the launch is queued; no copy for fp32 scales
    _lib.call("llmk_weight_dequant_fp8_block", _lib.ptr(x), _lib.ptr(s32), _lib.ptr(y), _lib.dt(y.dtype),
              M, N, block_size, _lib.stream(x))
    return y


def fp8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor):
    """c[..., n] = sum_kb (a_kb . b_kb[n]) * a_s[..., kb] * b_s[n // 128, kb], fp32 accumulate,
    returned in torch's default dtype.  a [..., K] e4m3fn, b [N, K] e4m3fn, K % 128 == 0."""
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    assert a_s.is_contiguous() and b_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    _lib.require_gpu(a, a_s, b, b_s)
    K = a.size(-1)
    M = a.numel() // K
    N = b.size(0)
    assert a_s.dtype == torch.float32 and b_s.dtype == torch.float32, 'fp8 scales must be float32'
    c = a.new_empty(*a.size()[:-1], N, dtype=torch.get_default_dtype())
    _lib.call("llmk_gemm_fp8_block", _lib.ptr(a), _lib.ptr(a_s), _lib.ptr(b), _lib.ptr(b_s), _lib.ptr(c),
              _lib.dt(c.dtype), M, N, K, *_lib.gemm_workspace(a.device, M, N, K), _lib.stream(a), exc=AssertionError)
    return c
