"""HIP quantizers / dequantizers vs the torch-CPU oracle: bit-exact integers and scales."""
import ctypes

import pytest
import torch

from oracle import quant_ref as q, bitpack_ref as bp
from llm_kernels_amd.quantization import fp8_kernel, int8_kernel, w4a8_kernel
from llm_kernels_amd import _lib
from helpers import announce, default_dtype

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 128), (16, 4096), (3, 5, 256), (257, 14336)])
def test_act_quant_int8_both_roundings(dev, dtype, shape):
    announce("act_quant_i8", dtype, shape)
    torch.manual_seed(0)
    x = torch.randn(*shape).to(dtype)
    x.view(-1)[:8] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 127.0, -127.0]).to(dtype)  # ties in group 0
    xg = x.to(dev)
    for mod, mode in ((int8_kernel, "away"), (w4a8_kernel, "up")):
        y, s = mod.act_quant(xg)
        oy, os_ = q.act_quant_int8(x, 128, mode)
        assert y.dtype == torch.int8 and s.dtype == torch.float16 and s.shape == os_.shape
        assert torch.equal(s.cpu(), os_), mode
        assert torch.equal(y.cpu(), oy), mode


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 128), (16, 4096), (2, 3, 384), (300, 4096)])
def test_act_quant_fp8(dev, dtype, shape):
    announce("act_quant_fp8", dtype, shape)
    torch.manual_seed(1)
    x = torch.randn(*shape).to(dtype)
    y, s = fp8_kernel.act_quant(x.to(dev))
    oy, os_ = q.act_quant_fp8(x)
    assert y.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    assert torch.equal(s.cpu(), os_)
    assert torch.equal(y.cpu().view(torch.uint8), oy.view(torch.uint8))


def test_act_quant_fp8_zero_group_nan_and_asserts(dev):
    announce("act_quant_fp8 zero group")
    x = torch.randn(2, 256)
    x[1, 128:] = 0
    y, s = fp8_kernel.act_quant(x.to(dev))
    assert s[1, 1].item() == 0.0 and y[1, 128:].float().isnan().all() and not y[0].float().isnan().any()
    with pytest.raises(AssertionError):
        fp8_kernel.act_quant(torch.randn(4, 100, device=dev))
    with pytest.raises(AssertionError):
        int8_kernel.act_quant(torch.randn(4, 256, device=dev).t())


@pytest.mark.parametrize("shape", [(128, 128), (512, 1024), (200, 300), (4096, 4096), (136, 4144), (72, 14336)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_weight_quant_int8_and_dequant(dev, shape, dtype):
    announce("weight_quant_i8", shape, dtype)
    torch.manual_seed(2)
    w = (torch.randn(*shape) * 0.02).to(dtype)
    y, s = int8_kernel.weight_quant(w.to(dev))
    oy, os_ = q.weight_quant_int8(w)
    assert torch.equal(s.cpu(), os_) and torch.equal(y.cpu(), oy)
    for dd in (torch.float16, torch.bfloat16, torch.float32):
        with default_dtype(dd):
            d = int8_kernel.weight_dequant(y, s)
        assert d.dtype == dd
        assert torch.equal(d.cpu(), q.weight_dequant_block(oy, os_, 128, dd))


@pytest.mark.parametrize("shape", [(128, 256), (300, 200), (4096, 4096), (130, 7168), (40, 4144)])
def test_weight_quant_fp8_and_dequant(dev, shape):
    announce("weight_quant_fp8", shape)
    torch.manual_seed(3)
    w = torch.randn(*shape) * 0.02
    y, s = fp8_kernel.weight_quant(w.to(dev))
    oy, os_ = q.weight_quant_fp8(w)
    assert torch.equal(s.cpu(), os_)
    assert torch.equal(y.cpu().view(torch.uint8), oy.view(torch.uint8))
    for dd in (torch.bfloat16, torch.float16, torch.float32):
        with default_dtype(dd):
            d = fp8_kernel.weight_dequant(y, s)
        assert d.dtype == dd and torch.equal(d.cpu(), q.weight_dequant_block(oy, os_, 128, dd))


@pytest.mark.parametrize("shape", [(128, 128), (1024, 7168), (4096, 4096)])
def test_w4a8_weight_quant_dequant(dev, shape):
    announce("w4a8 weight_quant", shape)
    torch.manual_seed(4)
    w = (torch.randn(*shape) * 0.02).half()
    yp, s, s4, z4 = w4a8_kernel.weight_quant(w.to(dev))
    oq, os_, os4, oz4 = q.w4a8_weight_quant_levels(w)
    assert yp.dtype == torch.int32 and yp.shape == (shape[0] // 8, shape[1])
    assert torch.equal(s.cpu(), os_) and torch.equal(s4.cpu(), os4) and torch.equal(z4.cpu(), oz4)
    opacked, _ = bp.pack_rows(oq.numpy(), 4, 32)
    assert torch.equal(yp.cpu(), torch.from_numpy(opacked))
    d = w4a8_kernel.weight_dequant(yp, s, s4, z4)
    assert d.dtype == torch.float16 and torch.equal(d.cpu(), q.w4a8_weight_dequant(oq, os_, os4, oz4))
    cos = torch.nn.functional.cosine_similarity(d.float().flatten().cpu(), w.float().flatten(), dim=0)
    assert cos > 0.98
    # an output that is not 16-byte aligned takes the one-word-per-thread form of the kernel: same bits
    buf = torch.empty(shape[0] * shape[1] + 1, dtype=torch.float16, device=dev)
    _lib.call("llmk_weight_dequant_w4a8", _lib.ptr(yp), _lib.ptr(s), _lib.ptr(s4), _lib.ptr(z4),
              ctypes.c_void_p(buf.data_ptr() + 2), shape[0], shape[1], 128, 128, None)
    torch.cuda.synchronize()
    assert torch.equal(buf[1:].view(shape), d)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 1), (5, 100), (16, 4096), (7, 14336), (3, 4, 333), (130, 1000), (2, 4104)])
def test_rowwise_int8_quantizer(dev, dtype, shape):
    """Per-token / per-channel int8 (one fp32 scale per row, any row length): integers and scales bit-exact,
    ties away from zero included."""
    announce("rowwise int8", dtype, shape)
    torch.manual_seed(7)
    x = torch.randn(*shape).to(dtype)
    flat = x.view(-1, shape[-1])
    if shape[-1] >= 8:
        flat[0, :8] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 127.0, -127.0]).to(dtype)   # absmax 127 -> s = 1: ties
    y, s = int8_kernel.act_quant_per_token(x.to(dev))
    oy, os_ = q.int8_quant_rowwise(flat)
    assert y.dtype == torch.int8 and s.dtype == torch.float32 and y.shape == x.shape and s.shape == x.shape[:-1]
    assert torch.equal(s.cpu().view(-1), os_)
    assert torch.equal(y.cpu().view(-1, shape[-1]), oy)
    y2, s2 = int8_kernel.weight_quant_per_channel(x.to(dev))
    assert torch.equal(y2, y) and torch.equal(s2, s)


def test_rowwise_int8_quantizer_zero_row_is_nan_free_of_crash(dev):
    """An all-zero row gives s = 0 and 0/0 in the division, as the 1 x 128 quantizers do; other rows are untouched."""
    announce("rowwise int8 zero row")
    x = torch.zeros(2, 256)
    x[1] = torch.linspace(-1, 1, 256)
    y, s = int8_kernel.act_quant_per_token(x.to(dev))
    oy, os_ = q.int8_quant_rowwise(x)
    assert s.cpu()[0].item() == 0.0 and torch.equal(s.cpu(), os_)
    assert torch.equal(y.cpu()[1], oy[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_fp8_quantisers_keep_the_sign_of_zero(dev, dtype):
    """-0.0 / s is -0.0, which e4m3 stores as 0x80: the quotient by the shared reciprocal must not turn it into
    +0 (fp16 weights of small magnitude underflow to -0.0 often enough to meet this in 4096 x 4096 elements)."""
    announce("fp8 quantisers, signed zeros", dtype)
    torch.manual_seed(11)
    x = (torch.randn(256, 512) * 0.02).to(dtype)
    x[::3, ::5] = -0.0
    x[1::3, 1::5] = 0.0
    y, s = fp8_kernel.act_quant(x.to(dev))
    oy, os_ = q.act_quant_fp8(x)
    assert torch.equal(s.cpu(), os_) and torch.equal(y.cpu().view(torch.uint8), oy.view(torch.uint8))
    assert (oy.view(torch.uint8)[::3, ::5] == 0x80).all()
    y, s = fp8_kernel.weight_quant(x.to(dev))
    oy, os_ = q.weight_quant_fp8(x)
    assert torch.equal(s.cpu(), os_) and torch.equal(y.cpu().view(torch.uint8), oy.view(torch.uint8))
