"""Int4QuantUtils: 4-bit pack / unpack into int16 / int32 words (reference quantization/quant_utils.py:5-64).

`direction="row"` packs consecutive rows into one word, `"column"` consecutive columns.  Tensors on a
HIP device go through the bit-pack kernels; the input is masked with 0x0F first, as in the reference.
"""
import torch

from . import bitpack


class Int4QuantUtils():

    @staticmethod
    def pack(imatrix: torch.Tensor, storage_bits: int = 32, q_bits: int = 4, direction: str = "row"):
        m = (imatrix.to(torch.int8) & 0x0F).to(torch.uint8)
        bits = 16 if storage_bits == 16 else 32
        if direction == "row":
            fn = bitpack.pack_weights_over_rows if m.is_cuda else bitpack.pack_weights_over_rows_torch
        elif direction == "column":
            fn = bitpack.pack_weights_over_cols if m.is_cuda else bitpack.pack_weights_over_cols_torch
        else:
            raise ValueError("direction must be 'row' or 'column'")
        q, _ = fn(m, q_bits, bits, False)
        return q

    @staticmethod
    def unpack(qmatrix: torch.Tensor, storage_bits: int = 32, q_bits: int = 4, direction: str = "row"):
        e = storage_bits // q_bits
        if direction == "row":
            fn = bitpack.unpack_over_rows if qmatrix.is_cuda else bitpack.unpack_over_rows_torch
            return fn(qmatrix, q_bits, qmatrix.shape[0] * e, torch.int8)
        elif direction == "column":
            fn = bitpack.unpack_over_cols if qmatrix.is_cuda else bitpack.unpack_over_cols_torch
            return fn(qmatrix, q_bits, qmatrix.shape[-1] * e, torch.int8)
        raise ValueError("direction must be 'row' or 'column'")
