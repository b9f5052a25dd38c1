"""Seeded sweeps of the streaming operators against the oracle, compared as bit patterns: ragged shapes on every
form of the kernels (whole 16-byte chunks and single elements), and edge values (signed zeros, fp16 subnormals,
magnitudes from 1e-6 to 6e4)."""
import random

import numpy as np
import pytest
import torch

from oracle import quant_ref as q, bitpack_ref as bp, convert_ref as cr, moe_ref
from llm_kernels_amd.quantization import fp8_kernel, int8_kernel, w4a8_kernel, bitpack
from llm_kernels_amd.quant_communication import quant_utils as qu
from llm_kernels_amd.fast_dequant import w4a16
from llm_kernels_amd.moe import group_gemm_kernel as gk
from helpers import announce, default_dtype

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _u8(t):
    return t.view(torch.uint8)


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("seed", range(8))
def test_block_quantisers_and_dequantisers_ragged_shapes(dev, seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    M = rnd.choice([1, 7, 128, 130, 257, 640])
    N = rnd.choice([16, 48, 128, 200, 272, 4096 + 16 * rnd.randint(0, 9), 8192])
    dt = DTYPES[seed % 3]
    announce("block quant sweep", M, N, dt)
    w = (torch.randn(M, N) * 0.02).to(dt)
    y, s = int8_kernel.weight_quant(w.to(dev))
    oy, os_ = q.weight_quant_int8(w)
    assert torch.equal(y.cpu(), oy) and torch.equal(s.cpu(), os_)
    y8, s8 = fp8_kernel.weight_quant(w.to(dev))
    oy8, os8 = q.weight_quant_fp8(w)
    assert torch.equal(_u8(y8).cpu(), _u8(oy8)) and torch.equal(s8.cpu(), os8)
    for dd in DTYPES:
        with default_dtype(dd):
            d, d8 = int8_kernel.weight_dequant(y, s), fp8_kernel.weight_dequant(y8, s8)
        assert torch.equal(_bits(d.cpu()), _bits(q.weight_dequant_block(oy, os_, 128, dd)))
        assert torch.equal(_bits(d8.cpu()), _bits(q.weight_dequant_block(oy8, os8, 128, dd)))


@pytest.mark.parametrize("seed", range(8))
def test_w4_quantisers_and_bit_packers_ragged_shapes(dev, seed):
    rnd = random.Random(100 + seed)
    torch.manual_seed(seed)
    dt = DTYPES[seed % 3]
    gs = rnd.choice([8, 16, 32, 64, 128, 256, 512])
    N, K = rnd.choice([1, 5, 33, 300]), gs * rnd.randint(1, 9)
    announce("w4 / bitpack sweep", N, K, gs, dt)
    w = (torch.randn(N, K) * 0.02).to(dt)
    pk, s, qd = w4a16.quantize_nk(w.to(dev), gs)
    oq, os_ = q.w4a16_quant_nk(w, gs)
    assert torch.equal(qd.cpu(), oq) and torch.equal(s.cpu(), os_)
    assert torch.equal(pk.cpu(), torch.from_numpy(bp.pack_cols(oq.numpy(), 4, 32)[0]))
    nbits = rnd.choice([1, 2, 4, 8])
    width = rnd.choice([w_ for w_ in (8, 16, 32, 64) if w_ >= nbits])
    e = width // nbits
    R, C = e * rnd.randint(1, 40), e * rnd.randint(1, 40)
    wq = torch.randint(0, 2 ** nbits, (R, C), dtype=torch.uint8)
    pr = bitpack.pack_weights_over_rows(wq.to(dev), nbits, width, False)[0]
    pc = bitpack.pack_weights_over_cols(wq.to(dev), nbits, width, False)[0]
    assert np.array_equal(pr.cpu().numpy(), bp.pack_rows(wq.numpy(), nbits, width)[0])
    assert np.array_equal(pc.cpu().numpy(), bp.pack_cols(wq.numpy(), nbits, width)[0])
    assert torch.equal(bitpack.unpack_over_rows(pr, nbits, R).cpu(), wq)
    assert torch.equal(bitpack.unpack_over_cols(pc, nbits, C).cpu(), wq)
    Mw, Kw = 128 * rnd.randint(1, 3), 128 * rnd.randint(1, 5)
    ww = (torch.randn(Mw, Kw) * 0.02).half()
    yp, s, s4, z4 = w4a8_kernel.weight_quant(ww.to(dev))
    oq, os_, os4, oz4 = q.w4a8_weight_quant_levels(ww)
    assert torch.equal(w4a8_kernel.weight_dequant(yp, s, s4, z4).cpu(), q.w4a8_weight_dequant(oq, os_, os4, oz4))


@pytest.mark.parametrize("seed", range(9))
def test_activation_quantisers_edge_values(dev, seed):
    rnd = random.Random(200 + seed)
    torch.manual_seed(seed)
    dt = DTYPES[seed % 3]
    rows, K = rnd.randint(1, 50), 128 * rnd.randint(1, 6)
    mag = rnd.choice([1e-6, 1e-3, 1.0, 300.0, 6e4 if dt != torch.float16 else 3e3])
    announce("activation quantisers, edge values", dt, rows, K, mag)
    x = (torch.randn(rows, K) * mag).to(dt)
    m = torch.rand(rows, K)
    x[m < 0.05] = -0.0
    x[(m >= 0.05) & (m < 0.1)] = 0.0
    if dt == torch.float16:
        x[(m >= 0.1) & (m < 0.13)] = 6e-8                 # the smallest fp16 subnormal
        x[(m >= 0.13) & (m < 0.16)] = -3e-6
    x[:, ::32] = mag                                       # no group of zeros: 0 / 0 is the reference's NaN, tested elsewhere
    xd = x.to(dev)
    y, s = fp8_kernel.act_quant(xd)
    oy, os_ = q.act_quant_fp8(x)
    assert torch.equal(_u8(y).cpu(), _u8(oy)) and torch.equal(s.cpu(), os_)
    y, s = int8_kernel.act_quant(xd)
    oy, os_ = q.act_quant_int8(x)
    assert torch.equal(y.cpu(), oy) and torch.equal(s.cpu(), os_)
    y, s = w4a8_kernel.act_quant(xd)
    oy, os_ = q.act_quant_int8(x, rounding="up")
    assert torch.equal(y.cpu(), oy) and torch.equal(s.cpu(), os_)
    y, s = int8_kernel.act_quant_per_token(xd)
    oy, os_ = q.int8_quant_rowwise(x)
    assert torch.equal(y.cpu(), oy) and torch.equal(s.cpu().flatten(), os_.flatten())
    if dt == torch.float32:
        return
    y, s = qu.fp8_quant(xd)
    oy, os_ = cr.fp8_quant(x)
    assert torch.equal(_u8(y).cpu(), _u8(oy)) and torch.equal(s.cpu(), os_)
    for od in (torch.float16, torch.bfloat16):
        assert torch.equal(_bits(qu.fp8_dequant(y, s, od).cpu()), _bits(cr.dequant(oy, os_, od)))
    y, s = qu.int8_quant(xd)
    oy, os_ = cr.int8_quant(x)
    assert torch.equal(y.cpu(), oy) and torch.equal(s.cpu(), os_)
    for od in (torch.float16, torch.bfloat16):
        assert torch.equal(_bits(qu.int8_dequant(y, s, od).cpu()), _bits(cr.dequant(oy, os_, od)))


@pytest.mark.parametrize("seed", range(6))
def test_moe_helpers_random_shapes_bit_patterns(dev, seed):
    rnd = random.Random(300 + seed)
    torch.manual_seed(seed)
    dt = [torch.float16, torch.bfloat16][seed % 2]
    T, H = rnd.randint(1, 90), rnd.choice([8, 40, 128, 384, 1000, 4096])
    E = rnd.choice([2, 8, 16, 60])
    topk = min(rnd.choice([1, 2, 4]), E)
    lo, hi = sorted(rnd.sample(range(E), 2))
    announce("moe helpers sweep", dt, T, H, E, topk, lo, hi)
    x = torch.randn(T, H).to(dt)
    x[torch.rand(T, H) < 0.05] = -0.0
    ids = torch.stack([torch.randperm(E)[:topk] for _ in range(T)])
    w = torch.rand(T, topk)
    rids, s2d, seg = gk.run_moe_ep_preproess(ids.to(dev), E)
    orids, os2d, oseg = moe_ref.run_moe_ep_preprocess(ids, E)
    assert torch.equal(rids.cpu(), orids) and torch.equal(s2d.cpu(), os2d) and torch.equal(seg.cpu(), oseg)
    gin = torch.full((T * topk, H), 7.0, dtype=dt, device=dev)
    gk.pre_reorder(x.to(dev), gin, s2d, ids.to(dev), None, lo, hi, topk, H)
    ogin = moe_ref.pre_reorder(x, os2d, ids, None, lo, hi, topk, out=torch.full((T * topk, H), 7.0, dtype=dt))
    assert torch.equal(_bits(gin.cpu()), _bits(ogin))
    do = torch.randn(T * topk, H).to(dt)
    out = torch.full((T, H), 5.0, dtype=dt, device=dev)
    gk.post_reorder(do.to(dev), out, s2d, ids.to(dev), w.to(dev), lo, hi, topk, H)
    assert torch.equal(out.cpu(), moe_ref.post_reorder(do, os2d, ids, w, lo, hi, topk))
