"""CPU restatement of the converter study programs and of the communication payload quantisers.

TEST INFRASTRUCTURE ONLY: imported by tests/ (and nothing in the product).

Follows fast_dequant/fast_dtype_convert/fast_uint4_to_fp16.cu:112-140 (simple kernel and pack_uint4),
fast_uint8_to_fp16.cu:65-73, fast_uint8_to_bf16.cu:62-70, fast_dequant/simple_marlin/mma_fp16.cu (cpu_gemm_reference)
and quant_communication/quant_utils.py:9-205.  Pinned by the reference's own recipes (value i % 16 -> v - 8,
i % 256 -> v - 128, (i % 16) / 10 and (i % 8) / 10 GEMM operands), by hand vectors and by closed forms in
tests/test_oracle_convert.py.
"""
import numpy as np
import torch


def pack_uint4(values):
    """fast_uint4_to_fp16.cu:130-140: value i -> bits 4 (i % 8) of word i // 8."""
    v = np.asarray(values, dtype=np.uint64) & 0xF
    pad = (-len(v)) % 8
    v = np.concatenate([v, np.zeros(pad, dtype=np.uint64)])
    w = np.zeros(len(v) // 8, dtype=np.uint64)
    for j in range(8):
        w |= v[j::8] << np.uint64(4 * j)
    return w.astype(np.uint32)


def uint4_to_fp16(packed, size):
    """fast_uint4_to_fp16.cu:112-127: out[i] = float16(nibble_i - 8)."""
    w = np.asarray(packed, dtype=np.uint32)
    idx = np.arange(size)
    nib = (w[idx // 8] >> (4 * (idx % 8)).astype(np.uint32)) & 0xF
    return (nib.astype(np.float32) - 8.0).astype(np.float16)


def uint8_minus_128(x, dtype):
    """fast_uint8_to_fp16.cu:65-73 / fast_uint8_to_bf16.cu:62-70."""
    return (torch.as_tensor(x).to(torch.float32) - 128.0).to(dtype)


def gemm_f16(a, b):
    """mma_fp16.cu cpu_gemm_reference: fp32 accumulation of fp16 operands, fp16 result."""
    return (a.float() @ b.float()).to(torch.float16)


def int8_quant(x, block_size=32):
    """quant_utils.py:9-58: s = max|x| / 127 in fp32, y = floor(x / s + 0.5), s stored fp16."""
    xf = x.float().reshape(-1, block_size)
    s = xf.abs().amax(dim=1, keepdim=True) / 127.0
    y = torch.floor(xf / s + 0.5).to(torch.int8)
    return y.reshape(x.shape), s.to(torch.float16).reshape(*x.shape[:-1], x.shape[-1] // block_size)


def fp8_quant(x, block_size=128):
    """quant_utils.py:116-155: s = max|x| / 448 in fp32, y = x / s as e4m3fn, s stored fp16."""
    xf = x.float().reshape(-1, block_size)
    s = xf.abs().amax(dim=1, keepdim=True) / 448.0
    y = (xf / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return y.reshape(x.shape), s.to(torch.float16).reshape(*x.shape[:-1], x.shape[-1] // block_size)


def dequant(y, s, output_dtype):
    """quant_utils.py:61-113,158-205: x = (y as s.dtype) * s in s.dtype, then cast."""
    block = y.shape[-1] // s.shape[-1]
    yf = y.to(s.dtype).reshape(-1, block)
    return (yf * s.reshape(-1, 1)).to(output_dtype).reshape(y.shape)
