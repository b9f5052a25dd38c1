"""W4A8 (QServe-style two-level) weight quantisation and GEMM on MI355X.

Same functions as the reference quantization/w4a8_kernel.py: act_quant (:171), weight_quant (:265),
weight_dequant (:104), w4a8_gemm (:406).  Level 1: 128x128 blocks, s = absmax/119, clamp +-119;
level 2: per (row, 128-col group) asymmetric uint4 with int8 scale s4 and zero z4; eight rows are
packed per int32 word (nibble i of word [r, k] is row 8r + i).
"""
from typing import Tuple

import torch

try:
    from .. import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib
from .bitpack import pack_weights_over_rows

PACKING_BITS = 32
W_BITS = 4


def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """1 x block_size groups: s = max|x| / 127 (fp32), y = floor(x / s + 0.5) int8, s stored fp16."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    _lib.require_gpu(x)
    y = torch.empty_like(x, dtype=torch.int8)
    s = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float16)
    _lib.call("llmk_act_quant_i8", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s),
              x.numel() // block_size, block_size, _lib.ROUND_HALF_UP, _lib.stream(x))
    return y, s


def weight_quant(x: torch.Tensor, block_size: int = 128, group_size_int4: int = 128,
                 pack_direction: str = "row") -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """W [N, K] -> (packed int32 [N/8, K], s fp16 [N/128, K/128], s4 int8 [N, K/g], z4 int8 [N, K/g])."""
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.dim() == 2, 'Input tensors must have 2 dimensions'
    assert x.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    assert block_size % group_size_int4 == 0, 'block_size must be divisible by group_size_int4'
    _lib.require_gpu(x)
    M, N = x.size()
    y = torch.empty_like(x, dtype=torch.int8)
    s = x.new_empty(((M + block_size - 1) // block_size, (N + block_size - 1) // block_size), dtype=torch.float16)
    ng = (N + group_size_int4 - 1) // group_size_int4
    s4 = x.new_empty(M, ng, dtype=torch.int8)
    z4 = x.new_empty(M, ng, dtype=torch.int8)
    st = _lib.stream(x)
    _lib.call("llmk_weight_quant_i8_block", _lib.ptr(x), _lib.dt(x.dtype), _lib.ptr(y), _lib.ptr(s),
              M, N, block_size, 119.0, _lib.ROUND_HALF_UP, 1, st)
    _lib.call("llmk_weight_quant_w4a8_level2", _lib.ptr(y), _lib.ptr(s4), _lib.ptr(z4), M, N, group_size_int4, st)
    # offline path: the reference checks the nibble range on the host at this point (a device sync)
    assert y.min() >= 0 and y.max() <= 15, 'Quantized values must be in the range [0, 15]'
    assert pack_direction == "row", "Only row packing is supported"
    assert M % (PACKING_BITS // W_BITS) == 0, f'row nums must be divisible by {PACKING_BITS // W_BITS}'
    y_packed, _ = pack_weights_over_rows(y, W_BITS, PACKING_BITS, transpose=False)
    return y_packed, s, s4, z4


def weight_dequant(y: torch.Tensor, s: torch.Tensor, s4: torch.Tensor, z4: torch.Tensor,
                   block_size: int = 128, group_size_int4: int = 128, pack_direction: str = "row") -> torch.Tensor:
    """packed [N/8, K] -> fp16 [N, K]: ((q - z4) * s4 evaluated in int8) * s."""
    assert y.is_contiguous(), 'Input tensor must be contiguous'
    assert y.dim() == 2, 'Input tensors must have 2 dimensions'
    assert y.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    assert block_size % group_size_int4 == 0, 'block_size must be divisible by group_size_int4'
    assert pack_direction == "row", "Only row packing is supported for dequantization"
    _lib.require_gpu(y, s, s4, z4)
    Mp, K = y.size()
    N = Mp * (PACKING_BITS // W_BITS)
    out = torch.empty((N, K), dtype=torch.float16, device=y.device)
    s, s4, z4 = s.contiguous(), s4.contiguous(), z4.contiguous()      # named: alive until the launch is queued
    _lib.call("llmk_weight_dequant_w4a8", _lib.ptr(y), _lib.ptr(s), _lib.ptr(s4), _lib.ptr(z4), _lib.ptr(out),
              N, K, block_size, group_size_int4, _lib.stream(y))
    return out


def w4a8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor,
              b_s: torch.Tensor, b_s4: torch.Tensor, b_z4: torch.Tensor,
              GROUP_SIZE_INT4: int = 128, elements_per_sample: int = 8,
              pack_direction: str = "row") -> torch.Tensor:
    """c = a(int8) x dequant_int8(b)^T with per-128-K a_s * b_s scaling; default dtype out."""
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    assert a_s.is_contiguous() and b_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    assert b_s4.is_contiguous() and b_z4.is_contiguous(), 'Scaling factor and zero point tensors must be contiguous'
    assert pack_direction == "row", "Only row packing is supported for dequantization"
    assert elements_per_sample == PACKING_BITS // W_BITS, 'weights must be packed 8 nibbles per int32'
    _lib.require_gpu(a, a_s, b, b_s, b_s4, b_z4)
    K = a.size(-1)
    M = a.numel() // K
    N = b.size(0) * elements_per_sample
    assert a_s.dtype == b_s.dtype, 'activation and weight scales must share a dtype'
    c = a.new_empty(*a.size()[:-1], N, dtype=torch.get_default_dtype())
    # what this shape's kernels use: nothing for the fused decode kernel with K <= 4096, fp32 partial sums for its
    # K ranges or the K slices of the fused tile kernels, the expanded int8 weights + the int8 GEMM's scratch otherwise
    need = _lib.load().llmk_gemm_w4a8_workspace_bytes(M, N, K, GROUP_SIZE_INT4)
    ws = _lib.workspace(a.device, need) if need > 0 else None
    _lib.call("llmk_gemm_w4a8", _lib.ptr(a), _lib.ptr(a_s), _lib.ptr(b), _lib.ptr(b_s), _lib.dt(a_s.dtype),
              _lib.ptr(b_s4), _lib.ptr(b_z4), _lib.ptr(c), _lib.dt(c.dtype), M, N, K, GROUP_SIZE_INT4,
              _lib.ptr(ws), need if ws is not None else 0, _lib.stream(a), exc=AssertionError)
    return c
