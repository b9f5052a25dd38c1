"""Pins oracle/bitpack_ref.py: closed forms, hand vectors, round trips (CPU)."""
import itertools

import numpy as np
import pytest

from oracle import bitpack_ref as bp


def test_hand_vector_rows_nibbles_1_to_8():
    w = np.arange(1, 9, dtype=np.uint8).reshape(8, 1)
    out, e = bp.pack_rows(w, 4, 32)
    assert e == 8 and out.dtype == np.int32
    assert out.view(np.uint32)[0, 0] == 0x87654321
    assert out[0, 0] < 0                      # nibble 7 >= 8 sets the sign bit
    back = bp.unpack_rows(out, 4, 8)
    assert (back == w).all()


def test_hand_vector_cols():
    w = np.array([[1, 2, 3, 4, 5, 6, 7, 8, 15, 0, 15, 0, 15, 0, 15, 0]], dtype=np.uint8)
    out, e = bp.pack_cols(w, 4, 32)
    assert out.view(np.uint32).tolist() == [[0x87654321, 0x0F0F0F0F]]
    assert (bp.unpack_cols(out, 4, 16) == w).all()


def test_two_bit_and_one_bit_hand_vectors():
    w = np.array([[3], [0], [1], [2]], dtype=np.uint8)            # 2-bit into 8-bit: 3 | 0<<2 | 1<<4 | 2<<6
    out, _ = bp.pack_rows(w, 2, 8)
    assert out.dtype == np.uint8 and out[0, 0] == 0b10010011
    w1 = np.array([[1, 0, 1, 1, 0, 0, 0, 1]], dtype=np.uint8)
    out, _ = bp.pack_cols(w1, 1, 8)
    assert out[0, 0] == 0b10001101


@pytest.mark.parametrize("nbits,width", list(itertools.product([1, 2, 4, 8], [8, 16, 32, 64])))
@pytest.mark.parametrize("direction", ["rows", "cols"])
def test_round_trip_and_closed_form(nbits, width, direction):
    rng = np.random.default_rng(nbits * 100 + width)
    e = width // nbits
    w = rng.integers(0, 2 ** nbits, size=(3 * e, 2 * e), dtype=np.uint8)
    if direction == "rows":
        out, ee = bp.pack_rows(w, nbits, width)
        back = bp.unpack_rows(out, nbits, w.shape[0])
        # closed form with python integers
        for r, c in [(0, 0), (2, 2 * e - 1), (1, 3 % (2 * e))]:
            exp = sum(int(w[r * e + i, c]) << (i * nbits) for i in range(e))
            assert int(out.view(bp._UINT[width])[r, c]) == exp
    else:
        out, ee = bp.pack_cols(w, nbits, width)
        back = bp.unpack_cols(out, nbits, w.shape[1])
        for r, c in [(0, 0), (3 * e - 1, 1), (e, 0)]:
            exp = sum(int(w[r, c * e + i]) << (i * nbits) for i in range(e))
            assert int(out.view(bp._UINT[width])[r, c]) == exp
    assert ee == e
    assert back.dtype == np.uint8 and (back == w).all()


def test_reference_recipe_8x16_uint4():
    # recipe of the reference's only exact check (bitpack.py:381-396): 8x16 random uint4, rows, 32-bit
    rng = np.random.default_rng(0)
    w = rng.integers(0, 16, size=(8, 16), dtype=np.uint8)
    packed, e = bp.pack_rows(w, 4, 32)
    assert packed.shape == (1, 16) and e == 8
    assert (bp.unpack_rows(packed, 4, 8) == w).all()


def test_int4_utils_cross_identity_and_masking():
    rng = np.random.default_rng(1)
    w = rng.integers(0, 16, size=(16, 24), dtype=np.uint8)
    assert (bp.int4_pack(w, 32, 4, "row") == bp.pack_rows(w, 4, 32)[0]).all()
    assert (bp.int4_pack(w, 32, 4, "column") == bp.pack_cols(w, 4, 32)[0]).all()
    assert (bp.int4_pack(w, 16, 4, "row") == bp.pack_rows(w, 4, 16)[0]).all()
    signed = w.astype(np.int8) - 8                                 # two's complement nibbles
    p = bp.int4_pack(signed, 32, 4, "row")
    u = bp.int4_unpack(p, 32, 4, "row")
    assert u.dtype == np.int8 and ((u == (signed & 0x0F))).all() and u.min() >= 0 and u.max() <= 15
    assert (bp.int4_unpack(bp.int4_pack(w, 32, 4, "column"), 32, 4, "column") == w).all()


def test_unpack_other_dtypes_and_signed_words():
    w = np.full((8, 4), 15, dtype=np.uint8)
    packed, _ = bp.pack_rows(w, 4, 32)
    assert (packed == -1).all()
    for dt in (np.int16, np.int32, np.int64):
        out = bp.unpack_rows(packed, 4, 8, dtype=dt)
        assert out.dtype == dt and (out == 15).all()
