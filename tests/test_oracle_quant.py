"""Pins oracle/quant_ref.py (CPU): rounding tables, hand-computed groups, invariants."""
import numpy as np
import pytest
import torch

from oracle import quant_ref as q


def test_rounding_tables():
    v = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.49999997, -0.49999997, 2.4999998, 126.5, -126.5, 0.0])
    away = q.round_half_away(v)
    up = q.round_half_up(v)
    even = torch.round(v)
    assert away.tolist() == [1, 2, 3, -1, -2, -3, 0, -0.0, 2, 127, -127, 0]
    assert up.tolist()[:6] == [1, 2, 3, 0, -1, -2]
    assert even.tolist()[:6] == [0, 2, 2, -0.0, -2, -2]
    # floor(v + 0.5) rounds 0.49999997 up because the fp32 add rounds to 1.0: that is the w4a8 rule
    assert up[6].item() == 1.0 and away[6].item() == 0.0


def test_act_quant_int8_hand_group():
    x = torch.zeros(1, 128)
    x[0, 0], x[0, 1], x[0, 2], x[0, 3], x[0, 4] = 127.0, -63.5, 0.5, -0.5, 1.5
    y, s = q.act_quant_int8(x, 128, "away")
    assert s.dtype == torch.float16 and s.item() == 1.0
    assert y[0, :5].tolist() == [127, -64, 1, -1, 2]
    y2, _ = q.act_quant_int8(x, 128, "up")
    assert y2[0, :5].tolist() == [127, -63, 1, 0, 2]


def test_act_quant_int8_invariants():
    torch.manual_seed(0)
    x = torch.randn(7, 512).bfloat16()
    for mode in ("away", "up"):
        y, s = q.act_quant_int8(x, 128, mode)
        assert y.dtype == torch.int8 and s.shape == (7, 4) and s.dtype == torch.float16
        assert y.abs().max() <= 127
        s32 = x.float().reshape(-1, 128).abs().amax(1) / 127.0
        err = (x.float().reshape(-1, 128) - y.float().reshape(-1, 128) * s32[:, None]).abs()
        assert (err <= s32[:, None] * 0.5 * (1 + 1e-5)).all()
        # every group uses the full range at its absmax element
        assert (y.reshape(-1, 128).abs().amax(1) == 127).all()
        # the stored scale is the fp16 rounding of the fp32 scale used for the division
        assert torch.equal(s.reshape(-1), s32.to(torch.float16))


def test_weight_quant_int8_blocks_and_ragged():
    torch.manual_seed(1)
    w = torch.randn(200, 300) * 0.02
    y, s = q.weight_quant_int8(w, 128)
    assert y.shape == w.shape and s.shape == (2, 3)
    for bi, bj in [(0, 0), (1, 2), (0, 2)]:
        blk = w[bi * 128:(bi + 1) * 128, bj * 128:(bj + 1) * 128]
        sc = blk.abs().max() / 127.0
        assert s[bi, bj] == sc.to(torch.float16)
        assert torch.equal(y[bi * 128:(bi + 1) * 128, bj * 128:(bj + 1) * 128],
                           q.round_half_away(blk / sc).to(torch.int8))
    d = q.weight_dequant_block(y, s, 128)
    assert torch.nn.functional.cosine_similarity(d.flatten(), w.flatten(), dim=0) > 0.999


def test_fp8_act_quant():
    torch.manual_seed(2)
    x = torch.randn(5, 256).bfloat16()
    y, s = q.act_quant_fp8(x, 128)
    assert y.dtype == torch.float8_e4m3fn and s.dtype == torch.float32 and s.shape == (5, 2)
    yf = y.float()
    assert yf.abs().max() == 448.0                      # absmax element maps to the e4m3 maximum
    assert not yf.isnan().any()
    rel = ((yf.reshape(-1, 128) * s.reshape(-1, 1)) - x.float().reshape(-1, 128)).abs()
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normals, absolute 2^-10*s for subnormals
    bound = torch.maximum(x.float().reshape(-1, 128).abs() * 2 ** -4, s.reshape(-1, 1) * 2 ** -10)
    assert (rel <= bound * 1.001).all()
    # known e4m3 codes: 448 -> 0x7E, 1.0 -> 0x38, -2.0 -> 0xC0
    g = torch.zeros(1, 128); g[0, 0] = 448.0; g[0, 1] = 1.0; g[0, 2] = -2.0; g[0, 3] = 0.0009765625
    yy, ss = q.act_quant_fp8(g, 128)
    assert ss.item() == 1.0 and yy.view(torch.uint8)[0, :4].tolist() == [0x7E, 0x38, 0xC0, 0x00]


def test_fp8_zero_group_is_nan():
    y, s = q.act_quant_fp8(torch.zeros(1, 128), 128)
    assert s.item() == 0.0 and y.float().isnan().all()


def test_w4a8_levels_bounds_and_dequant():
    torch.manual_seed(3)
    w = torch.randn(256, 512) * 0.02
    qq, s, s4, z4 = q.w4a8_weight_quant_levels(w)
    assert qq.dtype == torch.uint8 and qq.min() >= 0 and qq.max() <= 15
    assert s.shape == (2, 4) and s4.shape == (256, 4) and z4.shape == (256, 4)
    assert s4.max() <= 16 and s4.min() >= 1
    # protective range: (q - z4) * s4 never leaves int8, so int8 evaluation equals exact evaluation
    exact = (qq.int() - z4.int().repeat_interleave(128, 1)) * s4.int().repeat_interleave(128, 1)
    assert exact.abs().max() <= 127
    assert torch.equal(q.w4a8_dequant_int8(qq, s4, z4).int(), exact)
    d = q.w4a8_weight_dequant(qq, s, s4, z4)
    assert d.dtype == torch.float16
    assert torch.nn.functional.cosine_similarity(d.float().flatten(), w.flatten(), dim=0) > 0.98


def test_w4a8_hand_group():
    # one 128x128 block whose absmax is 119 -> s = 1, level-1 y == x for integers
    w = torch.zeros(128, 128)
    w[0, :] = torch.arange(128).float() % 31 - 15        # row 0: values -15..15
    w[1, 0] = 119.0
    qq, s, s4, z4 = q.w4a8_weight_quant_levels(w)
    assert s[0, 0] == 1.0
    # row 0: max 15, min -15 -> s4 = floor(30/15+.5) = 2, z4 = floor(15/2+.5) = 8
    assert s4[0, 0] == 2 and z4[0, 0] == 8
    y0 = w[0]
    assert torch.equal(qq[0].float(), torch.clamp(torch.floor(y0 / 2 + 0.5) + 8, 0, 15))


def test_w4a8_int8_wrap_semantics():
    qq = torch.tensor([[15, 0]], dtype=torch.uint8).repeat(1, 64)
    s4 = torch.tensor([[20]], dtype=torch.int8)
    z4 = torch.tensor([[2]], dtype=torch.int8)
    d = q.w4a8_dequant_int8(qq, s4, z4, 128)
    assert d[0, 0].item() == ((13 * 20 + 128) % 256) - 128 == 4      # 260 wraps to 4
    assert d[0, 1].item() == -40


def test_w4a16_nk_quant():
    torch.manual_seed(4)
    w = torch.randn(64, 256) * 0.02
    qq, s = q.w4a16_quant_nk(w, 128)
    assert qq.min() >= 0 and qq.max() <= 15 and s.shape == (64, 2) and s.dtype == torch.float16
    deq = (qq.float() - 8) * s.float().repeat_interleave(128, 1)
    assert ((deq - w).abs() <= s.float().repeat_interleave(128, 1) * 0.5 * 1.01 + 1e-6).all()


def test_rowwise():
    torch.manual_seed(5)
    x = torch.randn(9, 384)
    y, s = q.int8_quant_rowwise(x)
    assert (y.abs().amax(1) == 127).all() and s.dtype == torch.float32
    # hand row with ties: absmax 127 -> s = 1.0 exactly, every .5 rounds away from zero
    # (half-up would give -0.5 -> 0 and -1.5 -> -1, half-even 0.5 -> 0 and 2.5 -> 2)
    y, s = q.int8_quant_rowwise(torch.tensor([[0.5, -0.5, 1.5, -1.5, 2.5, 127.0]]))
    assert s.tolist() == [1.0] and y.tolist() == [[1, -1, 2, -2, 3, 127]] and y.dtype == torch.int8
    # a second row with another scale: s = 63.5 / 127 = 0.5, ties at odd multiples of 0.25
    y, s = q.int8_quant_rowwise(torch.tensor([[0.25, -0.25, 0.75, -1.25, 63.5, -63.5]]))
    assert s.tolist() == [0.5] and y.tolist() == [[1, -1, 2, -3, 127, -127]]


# ----------------------------------------------------------------- fp8 128x128 weight quantizer
def _e4m3_table():
    """Every finite e4m3fn value from the bit layout (1 sign, 4 exponent bits with bias 7, 3 mantissa bits;
    exponent 15 with mantissa 7 is NaN), without going through torch's fp8 type."""
    vals = {}
    for code in range(256):
        sgn = -1.0 if code & 0x80 else 1.0
        e, mnt = (code >> 3) & 0xF, code & 7
        if e == 15 and mnt == 7:
            continue
        v = mnt * 2.0 ** -9 if e == 0 else (1 + mnt / 8.0) * 2.0 ** (e - 7)
        vals[code] = sgn * v
    return vals


def _e4m3_rne(v, table):
    """Nearest table value, ties to the even mantissa (brute force over the 254 finite codes)."""
    best = None
    for code, t in table.items():
        d = abs(t - v)
        if best is None or d < best[0] or (d == best[0] and (code & 1) == 0 and (best[1] & 1) == 1):
            best = (d, code)
    return best[1]


def test_e4m3_cast_is_rne_onto_the_bit_layout_table():
    """Pins the cast that act_quant_fp8 / weight_quant_fp8 rely on: torch's CPU fp32 -> e4m3fn conversion
    equals round-to-nearest-even onto the value table derived from the bit layout (ties included)."""
    table = _e4m3_table()
    assert len(table) == 254 and table[0x7E] == 448.0 and table[0x38] == 1.0 and table[0xC0] == -2.0
    torch.manual_seed(11)
    v = torch.cat([torch.randn(300) * 100, torch.randn(100) * 0.01,
                   torch.tensor([0.0, 17.0, 19.0, 0.0029296875, 432.0, 448.0, -448.0, 1.0625, 1.1875])])
    v = v.clamp(-448, 448)
    got = v.to(torch.float8_e4m3fn).view(torch.uint8).tolist()
    for x, c in zip(v.tolist(), got):
        want = _e4m3_rne(x, table)
        if x == 0.0:
            assert c in (0x00, 0x80)
        else:
            assert table[c] == table[want], (x, c, want)
    # 17 lies midway between 16 (mantissa 0) and 18 (mantissa 1): ties go to the even mantissa
    assert torch.tensor([17.0, 19.0]).to(torch.float8_e4m3fn).float().tolist() == [16.0, 20.0]


def test_weight_quant_fp8_hand_block():
    # one block whose absmax is 448 -> s = 1 exactly and the codes are the plain e4m3 encodings
    w = torch.zeros(128, 128)
    w[0, 0], w[0, 1], w[0, 2], w[5, 7], w[127, 127] = 448.0, 1.0, -2.0, 17.0, 0.0009765625
    y, s = q.weight_quant_fp8(w)
    assert s.shape == (1, 1) and s.dtype == torch.float32 and s.item() == 1.0
    yb = y.view(torch.uint8)
    assert [yb[0, 0].item(), yb[0, 1].item(), yb[0, 2].item()] == [0x7E, 0x38, 0xC0]
    assert y.float()[5, 7].item() == 16.0              # tie -> even mantissa
    assert yb[127, 127].item() == 0x00                 # 2^-10 is half the smallest subnormal: tie -> 0
    assert int((yb != 0).sum()) == 4
    # absmax 224 -> s = 0.5, the same codes for inputs scaled by 0.5
    y2, s2 = q.weight_quant_fp8(w * 0.5)
    assert s2.item() == 0.5 and torch.equal(y2.view(torch.uint8), yb)


def test_weight_quant_fp8_blocks_ragged_by_brute_force():
    """200 x 300 (ragged in both directions): block membership, scale and codes of every block against an
    independent slice-by-slice evaluation; every block's absmax element maps to +-448."""
    torch.manual_seed(12)
    w = torch.randn(200, 300) * 0.02
    y, s = q.weight_quant_fp8(w, 128)
    assert y.shape == w.shape and y.dtype == torch.float8_e4m3fn and s.shape == (2, 3) and s.dtype == torch.float32
    table = _e4m3_table()
    yb = y.view(torch.uint8)
    for bi in range(2):
        for bj in range(3):
            r0, r1, c0, c1 = bi * 128, min(200, bi * 128 + 128), bj * 128, min(300, bj * 128 + 128)
            blk = w[r0:r1, c0:c1]
            sc = blk.abs().max() / 448.0                       # fp32
            assert s[bi, bj] == sc
            assert torch.equal(yb[r0:r1, c0:c1], (blk / sc).to(torch.float8_e4m3fn).view(torch.uint8))
            assert y[r0:r1, c0:c1].float().abs().max() == 448.0
            # a few elements of the block through the brute-force encoder
            for (i, j) in [(0, 0), (r1 - r0 - 1, c1 - c0 - 1), ((r1 - r0) // 2, (c1 - c0) // 3)]:
                v = (blk[i, j] / sc).item()
                assert table[yb[r0 + i, c0 + j].item()] == table[_e4m3_rne(v, table)]
    d = q.weight_dequant_block(y, s, 128)
    assert ((d - w).abs() <= torch.maximum(w.abs() * 2 ** -4, s.repeat_interleave(128, 0)[:200]
                                           .repeat_interleave(128, 1)[:, :300] * 2 ** -10) * 1.001).all()
