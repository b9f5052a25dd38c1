"""n-bit pack / unpack restated with numpy unsigned arithmetic (test oracle).

Follows quantization/bitpack.py of the reference:
  pack over rows   bitpack.py:9-36 (torch) / :228-293 (Triton, the public alias :376)
  pack over cols   bitpack.py:38-67 / :84-149 (alias :377)
  unpack rows      bitpack.py:296-305 / :308-373 (alias :378)
  unpack cols      bitpack.py:152-161 / :163-226 (alias :379)
and quantization/quant_utils.py:5-64 (Int4QuantUtils).

The public aliases are the Triton variants: values are cast to the output
integer type, shifted left by i*nbits and OR-reduced *without masking*; the
64-bit case shifts in 64-bit (the torch variants shift in int32 and are wrong
for shifts >= 32 -- the oracle implements the mathematically intended form).
"""
import numpy as np

_UINT = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}
_SINT = {8: np.uint8, 16: np.int16, 32: np.int32, 64: np.int64}  # torch has no uint16/32/64 outputs


def _check(nbits, width):
    assert width in (8, 16, 32, 64), "Unsuported bitpacking width"
    assert nbits in (8, 4, 2, 1), "Unsuported nbits"
    return width // nbits


def pack_rows(w, nbits, width):
    """out[r, c] = OR_i (w[r*e + i, c] << (i*nbits)) truncated to `width` bits."""
    e = _check(nbits, width)
    w = np.asarray(w)
    rows, cols = w.shape
    ut = _UINT[width]
    wv = w.astype(np.int64).astype(np.uint64)
    out = np.zeros((rows // e, cols), dtype=np.uint64)
    for i in range(e):
        out |= (wv[i:rows // e * e:e, :] << np.uint64(i * nbits))
    out = (out & np.uint64((1 << width) - 1 if width < 64 else 0xFFFFFFFFFFFFFFFF)).astype(ut)
    return out.view(_SINT[width]), e


def pack_cols(w, nbits, width):
    """out[r, c] = OR_i (w[r, c*e + i] << (i*nbits)) truncated to `width` bits."""
    e = _check(nbits, width)
    w = np.asarray(w)
    rows, cols = w.shape
    ut = _UINT[width]
    wv = w.astype(np.int64).astype(np.uint64)
    out = np.zeros((rows, cols // e), dtype=np.uint64)
    for i in range(e):
        out |= (wv[:, i:cols // e * e:e] << np.uint64(i * nbits))
    out = (out & np.uint64((1 << width) - 1 if width < 64 else 0xFFFFFFFFFFFFFFFF)).astype(ut)
    return out.view(_SINT[width]), e


def _as_unsigned(p):
    p = np.asarray(p)
    bits = p.dtype.itemsize * 8
    return p.view(_UINT[bits]).astype(np.uint64), bits


def unpack_rows(packed, nbits, num_output_rows, dtype=np.uint8):
    """out[r*e + i, c] = (packed[r, c] >> (i*nbits)) & mask."""
    pu, _ = _as_unsigned(packed)
    rows, cols = pu.shape
    e = num_output_rows // rows
    mask = np.uint64((1 << nbits) - 1)
    out = np.zeros((rows * e, cols), dtype=np.uint64)
    for i in range(e):
        out[i::e, :] = (pu >> np.uint64(i * nbits)) & mask
    return out.astype(dtype)


def unpack_cols(packed, nbits, num_output_cols, dtype=np.uint8):
    """out[r, c*e + i] = (packed[r, c] >> (i*nbits)) & mask."""
    pu, _ = _as_unsigned(packed)
    rows, cols = pu.shape
    e = num_output_cols // cols
    mask = np.uint64((1 << nbits) - 1)
    out = np.zeros((rows, cols * e), dtype=np.uint64)
    for i in range(e):
        out[:, i::e] = (pu >> np.uint64(i * nbits)) & mask
    return out.astype(dtype)


def int4_pack(imatrix, storage_bits=32, q_bits=4, direction="row"):
    """Int4QuantUtils.pack (quant_utils.py:6-34): input masked with & 0x0F first."""
    m = (np.asarray(imatrix).astype(np.int64) & 0x0F).astype(np.uint8)
    if direction == "row":
        out, _ = pack_rows(m, q_bits, storage_bits)
    elif direction == "column":
        out, _ = pack_cols(m, q_bits, storage_bits)
    else:
        raise ValueError(direction)
    return out


def int4_unpack(qmatrix, storage_bits=32, q_bits=4, direction="row"):
    """Int4QuantUtils.unpack (quant_utils.py:37-64): returns int8 in 0..15."""
    q = np.asarray(qmatrix)
    e = storage_bits // q_bits
    if direction == "row":
        return unpack_rows(q, q_bits, q.shape[0] * e, dtype=np.int8)
    elif direction == "column":
        return unpack_cols(q, q_bits, q.shape[1] * e, dtype=np.int8)
    raise ValueError(direction)
