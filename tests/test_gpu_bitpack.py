"""HIP pack/unpack vs the numpy oracle, bit-exact (through the C ABI via the Python mirror)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import bitpack_ref as bp
from llm_kernels_amd.quantization import bitpack, quant_utils
from helpers import announce

pytestmark = pytest.mark.gpu

_NP2T = {np.dtype(np.uint8): torch.uint8, np.dtype(np.int16): torch.int16, np.dtype(np.int32): torch.int32,
         np.dtype(np.int64): torch.int64}


@pytest.mark.parametrize("nbits,width", list(itertools.product([1, 2, 4, 8], [8, 16, 32, 64])))
def test_pack_unpack_all_widths(dev, nbits, width):
    announce("bitpack", nbits, width)
    rng = np.random.default_rng(nbits * 100 + width)
    e = width // nbits
    w = rng.integers(0, 2 ** nbits, size=(5 * e, 3 * e + 1 if False else 3 * e), dtype=np.uint8)
    wt = torch.from_numpy(w).to(dev)
    pr, er = bitpack.pack_weights_over_rows(wt, nbits, width, transpose=False)
    pc, ec = bitpack.pack_weights_over_cols(wt, nbits, width, transpose=False)
    opr, _ = bp.pack_rows(w, nbits, width)
    opc, _ = bp.pack_cols(w, nbits, width)
    assert er == ec == e
    assert pr.dtype == _NP2T[opr.dtype] and torch.equal(pr.cpu(), torch.from_numpy(opr))
    assert torch.equal(pc.cpu(), torch.from_numpy(opc))
    ur = bitpack.unpack_over_rows(pr, nbits, w.shape[0])
    uc = bitpack.unpack_over_cols(pc, nbits, w.shape[1])
    assert ur.dtype == torch.uint8 and torch.equal(ur.cpu(), torch.from_numpy(w))
    assert torch.equal(uc.cpu(), torch.from_numpy(w))
    # torch variants agree wherever they are defined correctly (shifts < 32)
    if width <= 32:
        tr, _ = bitpack.pack_weights_over_rows_torch(wt, nbits, width, False)
        assert torch.equal(tr, pr)
        assert torch.equal(bitpack.unpack_over_rows_torch(pr, nbits, w.shape[0]), ur)
        assert torch.equal(bitpack.unpack_over_cols_torch(pc, nbits, w.shape[1]), uc)


@pytest.mark.parametrize("nbits,width", list(itertools.product([1, 2, 4, 8], [8, 16, 32, 64])))
def test_pack_unpack_all_widths_16_byte_kernels(dev, nbits, width):
    """The same for shapes that the 16-bytes-per-thread kernels take (uint8 elements, 192 columns: a multiple of 16 and
    of every e), plus a partial unpack (fewer rows than the words hold) on those kernels."""
    announce("bitpack 16-byte kernels", nbits, width)
    rng = np.random.default_rng(nbits * 1000 + width)
    e = width // nbits
    w = rng.integers(0, 2 ** nbits, size=(3 * e, 192), dtype=np.uint8)
    wt = torch.from_numpy(w).to(dev)
    pr, _ = bitpack.pack_weights_over_rows(wt, nbits, width, transpose=False)
    pc, _ = bitpack.pack_weights_over_cols(wt, nbits, width, transpose=False)
    assert torch.equal(pr.cpu(), torch.from_numpy(bp.pack_rows(w, nbits, width)[0]))
    assert torch.equal(pc.cpu(), torch.from_numpy(bp.pack_cols(w, nbits, width)[0]))
    assert torch.equal(bitpack.unpack_over_rows(pr, nbits, w.shape[0]).cpu(), torch.from_numpy(w))
    assert torch.equal(bitpack.unpack_over_cols(pc, nbits, w.shape[1]).cpu(), torch.from_numpy(w))
    if e > 1:
        part = bitpack.unpack_over_rows(pr, nbits, 3 * (e // 2))      # e / 2 elements of every word
        ref = w.reshape(3, e, 192)[:, :e // 2, :].reshape(3 * (e // 2), 192)
        assert torch.equal(part.cpu(), torch.from_numpy(np.ascontiguousarray(ref)))


def test_reference_recipe_and_transpose(dev):
    announce("bitpack recipe 8x16")
    torch.manual_seed(0)
    W_q = torch.randint(0, 16, (8, 16), dtype=torch.uint8, device=dev)
    packed, e = bitpack.pack_weights_over_rows(W_q, 4, 32, transpose=False)
    unpacked = bitpack.unpack_over_rows(packed, 4, W_q.shape[0], dtype=torch.uint8)
    assert torch.equal(W_q, unpacked) and e == 8
    pt, _ = bitpack.pack_weights_over_rows(W_q, 4, 32, transpose=True)
    assert pt.shape == (16, 1) and torch.equal(pt.t(), packed)
    hand = torch.arange(1, 9, dtype=torch.uint8, device=dev).reshape(8, 1)
    hp, _ = bitpack.pack_weights_over_rows(hand, 4, 32, False)
    assert hp.item() == np.int32(np.uint32(0x87654321).astype(np.int32))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
def test_unpack_output_dtypes(dev, dtype):
    announce("unpack dtype", dtype)
    w = torch.randint(0, 16, (64, 40), dtype=torch.uint8, device=dev)
    p, _ = bitpack.pack_weights_over_rows(w, 4, 32, False)
    u = bitpack.unpack_over_rows(p, 4, 64, dtype=dtype)
    assert u.dtype == dtype and torch.equal(u.to(torch.uint8), w)
    pc, _ = bitpack.pack_weights_over_cols(w, 4, 32, False)
    uc = bitpack.unpack_over_cols(pc, 4, 40, dtype=dtype)
    assert torch.equal(uc.to(torch.uint8), w)


def test_large_and_empty(dev):
    announce("bitpack 4096x4096")
    torch.manual_seed(1)
    w = torch.randint(0, 16, (4096, 4096), dtype=torch.uint8, device=dev)
    p, _ = bitpack.pack_weights_over_rows(w, 4, 32, False)          # w4a8 layout [N/8, K]
    assert p.shape == (512, 4096)
    assert torch.equal(bitpack.unpack_over_rows(p, 4, 4096), w)
    pc, _ = bitpack.pack_weights_over_cols(w, 4, 32, False)         # config-1 layout [N, K/8]
    assert pc.shape == (4096, 512)
    assert torch.equal(bitpack.unpack_over_cols(pc, 4, 4096), w)
    opr, _ = bp.pack_rows(w[:64].cpu().numpy(), 4, 32)
    assert torch.equal(p[:8].cpu(), torch.from_numpy(opr))
    # checksum of checksums: every nibble counted once
    assert int(bitpack.unpack_over_cols(pc, 4, 4096).sum(dtype=torch.int64)) == int(w.sum(dtype=torch.int64))
    z = torch.zeros((0, 16), dtype=torch.uint8, device=dev)
    pz, _ = bitpack.pack_weights_over_rows(z, 4, 32, False)
    assert pz.shape == (0, 16)


def test_int4_quant_utils(dev):
    announce("Int4QuantUtils")
    torch.manual_seed(2)
    w = torch.randint(-8, 8, (32, 48), dtype=torch.int8, device=dev)
    for direction in ("row", "column"):
        for bits in (16, 32):
            p = quant_utils.Int4QuantUtils.pack(w, bits, 4, direction)
            op = bp.int4_pack(w.cpu().numpy(), bits, 4, direction)
            assert torch.equal(p.cpu(), torch.from_numpy(op))
            u = quant_utils.Int4QuantUtils.unpack(p, bits, 4, direction)
            assert u.dtype == torch.int8 and torch.equal(u.cpu(), (w & 0x0F).cpu())
