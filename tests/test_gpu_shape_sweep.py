"""Seeded sweep of irregular shapes through every GEMM entry point, against the float64 oracle.

The dispatch behind each entry point picks between a dozen kernels by (M, N, K): weight streaming with
resident or double-buffered activations, K ranges, 64 / 128 / 256-row tiles with or without split-K, the
256 x 256 tile, and the tile kernels that expand 4-bit weights themselves.  The shapes here are drawn so that
every M band and both short and long K occur with ragged rows and columns; the tolerance is the one of the
other GEMM tests (rtol 1e-2 / atol 1e-2 relative to the output scale), integer results bit-exact.
"""
import random

import pytest
import torch

from oracle import gemm_ref as g, marlin_ref as mr, quant_ref as q, bitpack_ref as bp
from llm_kernels_amd.quantization import fp8_kernel, int8_kernel, w4a8_kernel
from llm_kernels_amd.fast_dequant.simple_marlin.marlin import mul
from llm_kernels_amd.fast_dequant import w4a16
from helpers import announce, assert_close_scaled, default_dtype

pytestmark = pytest.mark.gpu

M_BANDS = [(1, 16), (17, 32), (33, 64), (65, 128), (129, 512), (513, 1300)]


def _shapes(seed, n_mult, k_mult, count=12, max_nk=6 << 20):
    """`count` shapes: M from each band in turn, N a multiple of n_mult, K a multiple of k_mult (short and long)."""
    rnd = random.Random(seed)
    out = []
    for i in range(count):
        lo, hi = M_BANDS[i % len(M_BANDS)]
        M = rnd.randint(lo, hi)
        K = k_mult * rnd.randint(1, (9000 if i % 3 else 4096) // k_mult)
        N = n_mult * rnd.randint(1, max(1, min(3000, max_nk // K) // n_mult))
        out.append((M, N, K))
    return out


@pytest.mark.parametrize("M,N,K", _shapes(1, 1, 128))
def test_sweep_fp8(dev, M, N, K):
    announce("sweep fp8", M, N, K)
    torch.manual_seed(M * 31 + N)
    a, a_s = q.act_quant_fp8(torch.randn(M, K).bfloat16())
    b, b_s = q.weight_quant_fp8(torch.randn(N, K) * 0.02)
    with default_dtype(torch.bfloat16):
        c = fp8_kernel.fp8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="sweep fp8")


@pytest.mark.parametrize("M,N,K", _shapes(2, 1, 128))
def test_sweep_int8_block_exact(dev, M, N, K):
    """Unit scales, small integers: every kernel variant has to return the exact integer product."""
    announce("sweep int8 block", M, N, K)
    torch.manual_seed(M * 31 + N)
    a = torch.randint(-15, 16, (M, K), dtype=torch.int8)
    b = torch.randint(-15, 16, (N, K), dtype=torch.int8)
    a_s = torch.ones(M, K // 128, dtype=torch.float16)
    b_s = torch.ones((N + 127) // 128, K // 128, dtype=torch.float16)
    with default_dtype(torch.float32):
        c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert torch.equal(c.cpu().long(), a.long() @ b.long().T)


@pytest.mark.parametrize("M,N,K", _shapes(3, 1, 128))
def test_sweep_int8_per_token(dev, M, N, K):
    announce("sweep int8 per token", M, N, K)
    torch.manual_seed(M * 31 + N)
    a, a_s = q.int8_quant_rowwise(torch.randn(M, K))
    b, b_s = q.int8_quant_rowwise(torch.randn(N, K) * 0.02)
    with default_dtype(torch.bfloat16):
        c, acc = int8_kernel.int8_gemm_per_token(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev), return_int32=True)
    assert torch.equal(acc.cpu(), g.int8_gemm_int32(a, b))
    assert_close_scaled(c, g.int8_gemm_rowcol(a, a_s, b, b_s), what="sweep int8 per token")


@pytest.mark.parametrize("M,N,K", _shapes(4, 8, 128))
def test_sweep_w4a8(dev, M, N, K):
    announce("sweep w4a8", M, N, K)
    torch.manual_seed(M * 31 + N)
    wq, s, s4, z4 = q.w4a8_weight_quant_levels(torch.randn(N, K) * 0.02)
    a, a_s = q.act_quant_int8(torch.randn(M, K).bfloat16(), rounding="up")
    packed, _ = bp.pack_rows(wq.numpy(), 4, 32)
    with default_dtype(torch.bfloat16):
        c = w4a8_kernel.w4a8_gemm(a.to(dev), a_s.to(dev), torch.from_numpy(packed).to(dev), s.to(dev),
                                  s4.to(dev), z4.to(dev), 128, 8, "row")
    assert_close_scaled(c, g.w4a8_gemm(a, a_s, wq, s, s4, z4), what="sweep w4a8")


@pytest.mark.parametrize("M,N,K", _shapes(5, 1, 128))
@pytest.mark.parametrize("gs", [64, 128])
def test_sweep_w4a16_nk(dev, M, N, K, gs):
    announce("sweep w4a16 nk", M, N, K, gs)
    torch.manual_seed(M * 31 + N)
    x = torch.randn(M, K).half()
    qn, s = q.w4a16_quant_nk(torch.randn(N, K) * 0.02, gs)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    y = w4a16.w4a16_gemm(x.to(dev), torch.from_numpy(packed).to(dev), s.to(dev), gs)
    ref = g.w4a16_gemm(x, qn.t().int().contiguous(), s.t().contiguous(), gs)
    assert_close_scaled(y, ref, what="sweep w4a16 nk")


@pytest.mark.parametrize("M,N,K", [(16 * ((m + 15) // 16), n, k) for m, n, k in _shapes(6, 64, 128)])
@pytest.mark.parametrize("gs", [128, -1])
def test_sweep_marlin_mul(dev, M, N, K, gs):
    announce("sweep marlin mul", M, N, K, gs)
    torch.manual_seed(M * 31 + N)
    A = (torch.randn(M, K) * 0.3).half()
    W = (torch.randn(K, N) * 0.05).half()
    _, q4, s = mr.fake_quantize(W, gs)
    B, sp = mr.pack(q4, s, K if gs == -1 else gs)
    C = torch.zeros(M, N, dtype=torch.half, device=dev)
    mul(A.to(dev), B.to(dev), C, sp.to(dev), torch.zeros(64, dtype=torch.int32, device=dev))
    assert_close_scaled(C, g.w4a16_gemm(A, q4, s, gs), what="sweep marlin mul")
