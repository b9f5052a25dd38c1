"""Pins oracle/convert_ref.py: the reference's own recipes, hand vectors, closed forms."""
import numpy as np
import torch

from oracle import convert_ref as c


def test_pack_uint4_hand_vector_and_round_trip():
    assert c.pack_uint4([1, 2, 3, 4, 5, 6, 7, 8])[0] == 0x87654321
    assert c.pack_uint4([15] * 8)[0] == 0xFFFFFFFF
    assert list(c.pack_uint4([1, 2, 3])) == [0x321]                      # zero padded tail word
    v = np.arange(1000) % 16
    out = c.uint4_to_fp16(c.pack_uint4(v), 1000)
    assert out.dtype == np.float16 and np.array_equal(out.astype(np.float32), v.astype(np.float32) - 8.0)


def test_reference_recipes_for_the_byte_converters():
    x = torch.arange(1024) % 256                                          # fast_uint8_to_fp16.cu:85-88
    for dt in (torch.float16, torch.bfloat16):
        out = c.uint8_minus_128(x.to(torch.uint8), dt)
        assert out.dtype == dt and torch.equal(out.float(), x.float() - 128.0)   # -128..127 is exact in both


def test_gemm_recipe_against_closed_form():
    # mma_fp16.cu:218-221: A[i] = (i % 16) / 10, B[i] = (i % 8) / 10 with M = N = K = 16: every row of A is
    # 0.0 .. 1.5 and B[k][n] = ((16 k + n) % 8) / 10 = (n % 8) / 10, so C[m][n] = (n % 8) / 10 * sum(A row)
    a = ((torch.arange(256) % 16).float() / 10).half().view(16, 16)
    b = ((torch.arange(256) % 8).float() / 10).half().view(16, 16)
    cc = c.gemm_f16(a, b)
    expect = (b[0].float() * a[0].float().sum()).half()
    assert torch.equal(cc[3], expect) and torch.equal(cc[0], cc[15])


def test_int8_payload_quant_hand_group_and_bounds():
    x = torch.zeros(32)
    x[0], x[1], x[2], x[3] = 127.0, -127.0, 63.5, -63.5                   # s = 1: half-up -> 64 and -63
    y, s = c.int8_quant(x.view(1, 32), 32)
    assert s.dtype == torch.float16 and float(s[0, 0]) == 1.0
    assert y[0, :4].tolist() == [127, -127, 64, -63]
    torch.manual_seed(0)
    x = torch.randn(8, 256).half()
    y, s = c.int8_quant(x, 32)
    assert y.abs().max() <= 127 and s.shape == (8, 8)
    back = c.dequant(y, s, torch.float16)
    sf = s.float().repeat_interleave(32, dim=1)
    assert ((back.float() - x.float()).abs() <= 0.51 * sf + 2e-3 * x.float().abs()).all()


def test_fp8_payload_quant_codes_and_dequant_dtype_rule():
    x = torch.zeros(1, 128)
    x[0, 0], x[0, 1], x[0, 2] = 448.0, 1.0, -2.0                          # s = 1
    y, s = c.fp8_quant(x, 128)
    assert s.dtype == torch.float16 and float(s[0, 0]) == 1.0
    assert y.view(torch.uint8)[0, :3].tolist() == [0x7E, 0x38, 0xC0]
    # the product is rounded in the scale dtype: 1.125 (0x39) * 0.333 (fp16) differs between fp16 and fp32 scales
    yy = torch.tensor([[0x39] * 128], dtype=torch.uint8).view(torch.float8_e4m3fn)
    s16 = torch.tensor([[0.333]], dtype=torch.float16)
    d16 = c.dequant(yy, s16, torch.float32)
    assert float(d16[0, 0]) == float((torch.tensor(1.125).half() * s16[0, 0]))
    assert float(d16[0, 0]) != 1.125 * float(s16[0, 0])
