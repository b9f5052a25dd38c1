"""Integer -> half converters and the one-tile MFMA GEMM on MI355X.

Library forms of the reference's standalone CUDA study programs: fast_dequant/fast_dtype_convert/
fast_uint4_to_fp16.cu (`value - 8`), fast_uint8_to_fp16.cu and fast_uint8_to_bf16.cu (`value - 128`), and
fast_dequant/simple_marlin/mma_fp16.cu (fp16 C = A x B with one matrix-core tile per wave).  The uint4
converter returns the values in natural order, like the reference's `uint4_to_fp16_simple_kernel` (:112-127).
"""
import torch

try:
    from .. import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib


def pack_uint4(values: torch.Tensor) -> torch.Tensor:
    """Host/device helper of the reference (`pack_uint4`, fast_uint4_to_fp16.cu:130-140): value i -> bits 4(i % 8)
    of word i // 8.  Returns int32 words (the tail word is zero padded)."""
    v = values.flatten().to(torch.int64) & 0xF
    pad = (-v.numel()) % 8
    if pad:
        v = torch.cat([v, v.new_zeros(pad)])
    w = (v.view(-1, 8) << (4 * torch.arange(8, device=v.device))).sum(dim=1)
    return torch.where(w >= 2 ** 31, w - 2 ** 32, w).to(torch.int32)      # same 32 bits, as int32


def uint4_to_fp16(packed: torch.Tensor, size: int) -> torch.Tensor:
    """out[i] = nibble_i - 8 as float16 for the first `size` nibbles of the int32 words."""
    _lib.require_gpu(packed)
    assert packed.is_contiguous() and packed.dtype in (torch.int32, torch.uint32)
    assert 0 <= size <= packed.numel() * 8
    out = torch.empty(size, dtype=torch.float16, device=packed.device)
    _lib.call("llmk_convert_u4_to_f16", _lib.ptr(packed), _lib.ptr(out), size, _lib.stream(packed))
    return out


def uint8_to_fp16(x: torch.Tensor) -> torch.Tensor:
    """out = x - 128 as float16 (same shape)."""
    _lib.require_gpu(x)
    assert x.is_contiguous() and x.dtype == torch.uint8
    out = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    _lib.call("llmk_convert_u8_to_f16", _lib.ptr(x), _lib.ptr(out), x.numel(), _lib.stream(x))
    return out


def uint8_to_bf16(x: torch.Tensor) -> torch.Tensor:
    """out = x - 128 as bfloat16 (same shape)."""
    _lib.require_gpu(x)
    assert x.is_contiguous() and x.dtype == torch.uint8
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    _lib.call("llmk_convert_u8_to_bf16", _lib.ptr(x), _lib.ptr(out), x.numel(), _lib.stream(x))
    return out


def mma_fp16(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """C [M, N] float16 = A [M, K] x B [K, N] (both float16, row-major), fp32 accumulation."""
    _lib.require_gpu(a, b)
    assert a.is_contiguous() and b.is_contiguous() and a.dtype == b.dtype == torch.float16
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0]
    c = torch.empty(a.shape[0], b.shape[1], dtype=torch.float16, device=a.device)
    _lib.call("llmk_gemm_f16_simple", _lib.ptr(a), _lib.ptr(b), _lib.ptr(c), a.shape[0], b.shape[1], a.shape[1],
              _lib.stream(a))
    return c
