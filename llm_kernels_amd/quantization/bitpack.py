"""n-bit pack / unpack, same functions as the reference quantization/bitpack.py.

`pack_weights_over_rows/cols` and `unpack_over_rows/cols` (reference aliases, bitpack.py:376-379)
run HIP kernels through the C ABI; the `_torch` variants are plain torch expressions kept for
API parity (bitpack.py:9-67,152-161,296-305).  The `_triton` names are kept as aliases of the
HIP-backed functions so that existing call sites keep working.
"""
import torch

try:
    from .. import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib

_PACK_DTYPE = {8: torch.uint8, 16: torch.int16, 32: torch.int32, 64: torch.int64}
_OUT_BYTES = {torch.uint8: 1, torch.int8: 1, torch.int16: 2, torch.int32: 4, torch.int64: 8}


def _check(W_nbits, packing_bitwidth):
    assert packing_bitwidth in [8, 16, 32, 64], "Unsuported bitpacking width"
    assert W_nbits in [8, 4, 2, 1], "Unsuported nbits"
    return packing_bitwidth // W_nbits


# ----------------------------------------------------------------------------- torch variants
def pack_weights_over_rows_torch(W_q: torch.Tensor, W_nbits: int, packing_bitwidth: int, transpose: bool):
    e = _check(W_nbits, packing_bitwidth)
    acc_dtype = torch.int32 if packing_bitwidth <= 32 else torch.int64
    w = W_q.to(acc_dtype)
    rows = W_q.shape[0] // e
    out = torch.zeros((rows, W_q.shape[1]), dtype=acc_dtype, device=W_q.device)
    for i in range(e):
        out += w[i::e, :][:rows] << (i * W_nbits)
    out = out.to(_PACK_DTYPE[packing_bitwidth])
    return (out.t() if transpose else out), e


def pack_weights_over_cols_torch(W_q: torch.Tensor, W_nbits: int, packing_bitwidth: int, transpose: bool):
    e = _check(W_nbits, packing_bitwidth)
    acc_dtype = torch.int32 if packing_bitwidth <= 32 else torch.int64
    w = W_q.to(acc_dtype)
    cols = W_q.shape[1] // e
    out = torch.zeros((W_q.shape[0], cols), dtype=acc_dtype, device=W_q.device)
    for i in range(e):
        out += w[:, i::e][:, :cols] << (i * W_nbits)
    out = out.to(_PACK_DTYPE[packing_bitwidth])
    return (out.t() if transpose else out), e


def unpack_over_cols_torch(W_q_packed, W_nbits, num_output_cols, dtype=torch.uint8):
    rows, cols = W_q_packed.shape
    e = num_output_cols // cols
    shifts = torch.arange(e, device=W_q_packed.device, dtype=W_q_packed.dtype) * W_nbits
    mask = (1 << W_nbits) - 1
    return ((W_q_packed.unsqueeze(-1) >> shifts) & mask).to(dtype).view(rows, num_output_cols)


def unpack_over_rows_torch(W_q_packed, W_nbits, num_output_rows, dtype=torch.uint8):
    rows, cols = W_q_packed.shape
    e = num_output_rows // rows
    shifts = torch.arange(e, device=W_q_packed.device, dtype=W_q_packed.dtype) * W_nbits
    mask = (1 << W_nbits) - 1
    u = ((W_q_packed.unsqueeze(-1) >> shifts) & mask).to(dtype)
    return u.permute(0, 2, 1).reshape(num_output_rows, cols)


# ----------------------------------------------------------------------------- HIP variants
def _as_kernel_input(W_q):
    if W_q.dtype not in _OUT_BYTES:
        W_q = W_q.to(torch.uint8)
    return W_q.contiguous()


def pack_weights_over_rows_hip(W_q: torch.Tensor, W_nbits: int, packing_bitwidth: int, transpose: bool):
    e = _check(W_nbits, packing_bitwidth)
    _lib.require_gpu(W_q)
    rows_in, cols = W_q.shape
    rows = rows_in // e
    w = _as_kernel_input(W_q)
    out = torch.empty((rows, cols), dtype=_PACK_DTYPE[packing_bitwidth], device=W_q.device)
    _lib.call("llmk_pack_rows", _lib.ptr(w), _OUT_BYTES[w.dtype], _lib.ptr(out), rows, cols,
              W_nbits, packing_bitwidth, _lib.stream(W_q))
    return (out.t() if transpose else out), e


def pack_weights_over_cols_hip(W_q: torch.Tensor, W_nbits: int, packing_bitwidth: int, transpose: bool):
    e = _check(W_nbits, packing_bitwidth)
    _lib.require_gpu(W_q)
    rows, cols_in = W_q.shape
    cols = cols_in // e
    w = _as_kernel_input(W_q)
    if cols * e != cols_in:
        w = w[:, :cols * e].contiguous()
    out = torch.empty((rows, cols), dtype=_PACK_DTYPE[packing_bitwidth], device=W_q.device)
    _lib.call("llmk_pack_cols", _lib.ptr(w), _OUT_BYTES[w.dtype], _lib.ptr(out), rows, cols,
              W_nbits, packing_bitwidth, _lib.stream(W_q))
    return (out.t() if transpose else out), e


def _pack_bits_of(t):
    if t.dtype not in _OUT_BYTES:
        raise TypeError("packed tensor must be an 8/16/32/64-bit integer tensor, got %s" % t.dtype)
    return _OUT_BYTES[t.dtype] * 8


def unpack_over_rows_hip(W_q_packed, W_nbits, num_output_rows, dtype=torch.uint8):
    _lib.require_gpu(W_q_packed)
    rows, cols = W_q_packed.shape
    e = num_output_rows // rows
    if dtype not in _OUT_BYTES:
        raise TypeError("unsupported output dtype %s" % dtype)
    p = W_q_packed.contiguous()
    out = torch.empty((num_output_rows, cols), dtype=dtype, device=p.device)
    if rows * e != num_output_rows:
        raise ValueError("num_output_rows must be a multiple of the packed row count")
    _lib.call("llmk_unpack_rows", _lib.ptr(p), _pack_bits_of(p), _lib.ptr(out), _OUT_BYTES[dtype],
              rows, cols, W_nbits, e, _lib.stream(p))
    return out


def unpack_over_cols_hip(W_q_packed, W_nbits, num_output_cols, dtype=torch.uint8):
    _lib.require_gpu(W_q_packed)
    rows, cols = W_q_packed.shape
    e = num_output_cols // cols
    if dtype not in _OUT_BYTES:
        raise TypeError("unsupported output dtype %s" % dtype)
    if cols * e != num_output_cols:
        raise ValueError("num_output_cols must be a multiple of the packed column count")
    p = W_q_packed.contiguous()
    out = torch.empty((rows, num_output_cols), dtype=dtype, device=p.device)
    _lib.call("llmk_unpack_cols", _lib.ptr(p), _pack_bits_of(p), _lib.ptr(out), _OUT_BYTES[dtype],
              rows, cols, W_nbits, e, _lib.stream(p))
    return out


# names used by callers of the reference module
pack_weights_over_rows_triton = pack_weights_over_rows_hip
pack_weights_over_cols_triton = pack_weights_over_cols_hip
unpack_over_rows_triton = unpack_over_rows_hip
unpack_over_cols_triton = unpack_over_cols_hip

pack_weights_over_rows = pack_weights_over_rows_hip
pack_weights_over_cols = pack_weights_over_cols_hip
unpack_over_rows = unpack_over_rows_hip
unpack_over_cols = unpack_over_cols_hip
