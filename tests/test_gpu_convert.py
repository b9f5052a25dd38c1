"""HIP converters, one-tile MFMA GEMM and communication payload quantisers vs the oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from oracle import convert_ref as c
from llm_kernels_amd.fast_dequant import fast_dtype_convert as fc
from llm_kernels_amd.quant_communication import quant_utils as qc
from helpers import announce, assert_close_scaled

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("size", [1024 * 1024, 8, 13, 1, 4099])
def test_uint4_to_fp16_reference_recipe(dev, size):
    """fast_uint4_to_fp16.cu:156-160: values i % 16, expected v - 8 (natural order)."""
    announce("uint4_to_fp16", size)
    v = np.arange(size) % 16
    packed = torch.from_numpy(c.pack_uint4(v).view(np.int32)).to(dev)
    out = fc.uint4_to_fp16(packed, size)
    assert out.dtype == torch.float16 and torch.equal(out.cpu().float(), torch.from_numpy(v).float() - 8.0)
    assert np.array_equal(out.cpu().numpy(), c.uint4_to_fp16(c.pack_uint4(v), size))
    assert torch.equal(fc.pack_uint4(torch.from_numpy(v).to(dev)).cpu(), packed.cpu())


@pytest.mark.parametrize("size", [1024, 7, 8, 1000003])
def test_uint8_converters_reference_recipe(dev, size):
    """fast_uint8_to_fp16.cu:85-88 / fast_uint8_to_bf16.cu: values i % 256, expected v - 128."""
    announce("uint8 converters", size)
    x = (torch.arange(size) % 256).to(torch.uint8)
    h = fc.uint8_to_fp16(x.to(dev))
    b = fc.uint8_to_bf16(x.to(dev))
    assert h.dtype == torch.float16 and b.dtype == torch.bfloat16
    assert torch.equal(h.cpu(), c.uint8_minus_128(x, torch.float16))
    assert torch.equal(b.cpu(), c.uint8_minus_128(x, torch.bfloat16))


@pytest.mark.parametrize("M,N,K", [(16, 8, 16), (16, 16, 32), (64, 48, 96), (33, 17, 40), (128, 128, 256)])
def test_mma_fp16_reference_recipe_and_random(dev, M, N, K):
    """mma_fp16.cu:218-221 operands ((i % 16) / 10, (i % 8) / 10), then random operands."""
    announce("mma_fp16", M, N, K)
    a = ((torch.arange(M * K) % 16).float() / 10).half().view(M, K)
    b = ((torch.arange(K * N) % 8).float() / 10).half().view(K, N)
    assert_close_scaled(fc.mma_fp16(a.to(dev), b.to(dev)), c.gemm_f16(a, b).double(), rtol=2e-3, atol=2e-3, what="mma recipe")
    torch.manual_seed(M + N)
    a, b = torch.randn(M, K).half(), torch.randn(K, N).half()
    assert_close_scaled(fc.mma_fp16(a.to(dev), b.to(dev)), c.gemm_f16(a, b).double(), rtol=2e-3, atol=2e-3, what="mma random")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(4, 64), (3, 5, 256), (1, 32)])
def test_int8_payload_round_trip_bit_exact(dev, dtype, shape):
    announce("comm int8", dtype, shape)
    torch.manual_seed(1)
    x = (torch.randn(*shape) * 4).to(dtype)
    y, s = qc.int8_quant(x.to(dev), 32)
    oy, os_ = c.int8_quant(x, 32)
    assert y.dtype == torch.int8 and s.dtype == torch.float16 and s.shape == os_.shape
    assert torch.equal(y.cpu(), oy) and torch.equal(s.cpu(), os_)
    for odt in (torch.float16, torch.float32, torch.bfloat16):
        assert torch.equal(qc.int8_dequant(y, s, odt).cpu(), c.dequant(oy, os_, odt))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fp8_payload_round_trip_bit_exact(dev, dtype):
    announce("comm fp8", dtype)
    torch.manual_seed(2)
    x = (torch.randn(6, 512) * 3).to(dtype)
    y, s = qc.fp8_quant(x.to(dev), 128)
    oy, os_ = c.fp8_quant(x, 128)
    assert y.dtype == torch.float8_e4m3fn and s.dtype == torch.float16
    assert torch.equal(y.view(torch.uint8).cpu(), oy.view(torch.uint8)) and torch.equal(s.cpu(), os_)
    for odt in (torch.float16, torch.float32):
        assert torch.equal(qc.fp8_dequant(y, s, odt).cpu(), c.dequant(oy, os_, odt))
    # every e4m3 code, fp32 scale: the decode is exact
    codes = torch.arange(256, dtype=torch.uint8).repeat(4).view(8, 128)
    fin = (codes & 0x7F) != 0x7F
    sc = torch.full((8, 1), 0.75, dtype=torch.float32)
    d = qc.fp8_dequant(codes.view(torch.float8_e4m3fn).to(dev), sc.to(dev), torch.float32).cpu()
    ref = codes.view(torch.float8_e4m3fn).float() * 0.75
    assert torch.equal(d[fin], ref[fin]) and torch.isnan(d[~fin]).all()
    # reference recipe (quant_utils.py:228-251): cosine similarity of the round trip
    back = qc.fp8_dequant(y, s, dtype).float().cpu().flatten()
    assert torch.nn.functional.cosine_similarity(back, x.float().flatten(), dim=0) > 0.999


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_payload_dequantisers_keep_the_sign_of_zero(dev, dtype):
    """-0.0 survives quantisation as the e4m3 code 0x80 and comes back as -0.0 in every output dtype (compared as
    bit patterns: the float comparison calls the two zeros equal)."""
    announce("comm signed zeros", dtype)
    torch.manual_seed(4)
    x = (torch.randn(9, 384) * 2).to(dtype)
    x[::2, ::7] = -0.0
    y, s = qc.fp8_quant(x.to(dev), 128)
    oy, os_ = c.fp8_quant(x, 128)
    assert torch.equal(y.view(torch.uint8).cpu(), oy.view(torch.uint8)) and torch.equal(s.cpu(), os_)
    assert (oy.view(torch.uint8)[::2, ::7] == 0x80).all()
    for odt in (torch.float16, torch.bfloat16):
        d, ref = qc.fp8_dequant(y, s, odt).cpu(), c.dequant(oy, os_, odt)
        assert torch.equal(d.view(torch.int16), ref.view(torch.int16))
        assert (d.view(torch.int16)[::2, ::7] == -32768).all()
