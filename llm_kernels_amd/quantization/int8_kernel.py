"""Blockwise W8A8 int8 quantisation and GEMM on MI355X.

Same functions as the reference quantization/int8_kernel.py: act_quant (:34), weight_quant (:91),
weight_dequant (:145), int8_gemm (:233).  act_quant_per_token / weight_quant_per_channel /
int8_gemm_per_token add the per-token x per-channel scheme with one full-K int32 accumulation.
"""
from typing import Tuple

import torch

try:
    from .. import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib


def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """1 x block_size groups: s = max|x| / 127 (fp32), y = round-half-away(x / s) int8, s stored fp16."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    _lib.require_gpu(x)
    y = torch.empty_like(x, dtype=torch.int8)
    s = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float16)
    _lib.call("llmk_act_quant_i8", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s),
              x.numel() // block_size, block_size, _lib.ROUND_HALF_AWAY, _lib.stream(x))
    return y, s


def weight_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """block x block tiles of W [N, K]: s = blockmax / 127, half-away rounding, fp16 scales."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.dim() == 2, 'Input tensors must have 2 dimensions'
    _lib.require_gpu(x)
    M, N = x.size()
    y = torch.empty_like(x, dtype=torch.int8)
    s = x.new_empty(((M + block_size - 1) // block_size, (N + block_size - 1) // block_size), dtype=torch.float16)
    _lib.call("llmk_weight_quant_i8_block", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s),
              M, N, block_size, 127.0, _lib.ROUND_HALF_AWAY, 0, _lib.stream(x))
    return y, s


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    assert x.is_contiguous() and s.is_contiguous(), 'Input tensors must be contiguous'
    assert x.dim() == 2 and s.dim() == 2, 'Input tensors must have 2 dimensions'
    _lib.require_gpu(x, s)
    M, N = x.size()
    y = torch.empty_like(x, dtype=torch.get_default_dtype())
    _lib.call("llmk_weight_dequant_i8_block", _lib.ptr(x), _lib.ptr(s), _lib.dt(s.dtype), _lib.ptr(y),
              _lib.dt(y.dtype), M, N, block_size, _lib.stream(x))
    return y


def int8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor):
    """c[..., n] = sum_kb fp32(int32 a_kb . b_kb[n]) * a_s[..., kb] * b_s[n // 128, kb]; default dtype out."""
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    assert a_s.is_contiguous() and b_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    _lib.require_gpu(a, a_s, b, b_s)
    K = a.size(-1)
    M = a.numel() // K
    N = b.size(0)
    assert a_s.dtype == b_s.dtype, 'activation and weight scales must share a dtype'
    c = a.new_empty(*a.size()[:-1], N, dtype=torch.get_default_dtype())
    _lib.call("llmk_gemm_i8_block", _lib.ptr(a), _lib.ptr(a_s), _lib.ptr(b), _lib.ptr(b_s), _lib.dt(a_s.dtype),
              _lib.ptr(c), _lib.dt(c.dtype), M, N, K, *_lib.gemm_workspace(a.device, M, N, K), _lib.stream(a),
              exc=AssertionError)
    return c


# ----------------------------------------------------------------------------- per-token x per-channel
def _rowwise_quant(x: torch.Tensor):
    """One scale per row of the last dimension: s = max|row| / 127 (fp32), y = round-half-away(x / s)."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    _lib.require_gpu(x)
    if x.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        x = x.float()
    cols = x.size(-1)
    rows = x.numel() // cols if cols else 0
    y = torch.empty_like(x, dtype=torch.int8)
    s = x.new_empty(x.size()[:-1], dtype=torch.float32)
    _lib.call("llmk_quant_i8_rowwise", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s), rows, cols, _lib.stream(x))
    return y, s


def act_quant_per_token(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token symmetric int8 with fp32 scales [..]."""
    return _rowwise_quant(x)


def weight_quant_per_channel(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-output-channel symmetric int8 of W [N, K] with fp32 scales [N]."""
    return _rowwise_quant(w)


def int8_gemm_per_token(a, a_s, b, b_s, return_int32: bool = False):
    """c[m, n] = int32(sum_k a[m,k] b[n,k]) * a_s[m] * b_s[n]; optionally also the raw int32 accumulators."""
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    _lib.require_gpu(a, a_s, b, b_s)
    K = a.size(-1)
    M = a.numel() // K
    N = b.size(0)
    a_s = a_s.reshape(-1).float().contiguous()
    b_s = b_s.reshape(-1).float().contiguous()
    assert a_s.numel() == M and b_s.numel() == N, 'need one scale per token and per output channel'
    c = a.new_empty(*a.size()[:-1], N, dtype=torch.get_default_dtype())
    acc = a.new_empty(*a.size()[:-1], N, dtype=torch.int32) if return_int32 else None
    # (only the K split of mid-size M uses scratch here)
    ws = _lib.gemm_workspace(a.device, M, N, K) if M <= 512 else (None, 0)
    _lib.call("llmk_gemm_i8_rowcol", _lib.ptr(a), _lib.ptr(a_s), _lib.ptr(b), _lib.ptr(b_s), _lib.ptr(c),
              _lib.dt(c.dtype), _lib.ptr(acc), M, N, K, *ws, _lib.stream(a), exc=AssertionError)
    return (c, acc) if return_int32 else c
