"""Parity at the full benchmark shapes (the Llama-3-8B GEMM grid of the five configurations).

The oracle is row-separable, so every case checks
  * a sample of rows of C (one random row out of every M/64-row slab, all columns) against the float64
    oracle at the stated tolerance (int32 accumulators: torch.equal),
  * every element of C for finiteness,
  * a checksum over ALL rows: the column sums of C against a one-row oracle GEMM of the scale-weighted
    column sums of A (exact integers for the int32 accumulators), which a wrong tile anywhere would move.
Operands are produced on the device by the product's quantizers, whose bits are pinned against the
oracle in test_gpu_quant.py; the oracle then works on the very same quantised operands.
"""
import pytest
import torch

from oracle import gemm_ref as g, quant_ref as q, bitpack_ref as bp
from llm_kernels_amd.quantization import fp8_kernel, int8_kernel, w4a8_kernel
from llm_kernels_amd.fast_dequant import w4a16
from llm_kernels_amd.fast_dequant.simple_marlin.utils import QuantUtils
from llm_kernels_amd.fast_dequant.simple_marlin.marlin import mul
from helpers import announce, assert_close_scaled, default_dtype

pytestmark = pytest.mark.gpu

LLAMA_NK = [(4096, 4096), (6144, 4096), (28672, 4096), (4096, 14336)]


def sample_rows(M, n=64, seed=0):
    """One random row out of each of min(n, M) equal slabs: every row tile of every kernel is touched."""
    n = min(n, M)
    gen = torch.Generator().manual_seed(seed)
    edges = torch.linspace(0, M, n + 1).long()
    return torch.stack([edges[i] + torch.randint(0, int(edges[i + 1] - edges[i]), (1,), generator=gen)[0]
                        for i in range(n)])


def blockwise_rows(a, a_s, b, b_s, chunk=8192):
    """gemm_blockwise evaluated over column chunks of B (bounds the float64 temporaries)."""
    N = b.shape[0]
    out = []
    for n0 in range(0, N, chunk):
        n1 = min(N, n0 + chunk)
        out.append(g.gemm_blockwise(a, a_s, b[n0:n1], b_s[n0 // 128:(n1 + 127) // 128]))
    return torch.cat(out, dim=-1)


def check_float_gemm(c, a, a_s, b, b_s, what, seed=0):
    """c on the device; a, a_s, b, b_s on the host (quantised operands)."""
    M = a.shape[0]
    assert bool(torch.isfinite(c).all()), "%s: non-finite output" % what
    rows = sample_rows(M, seed=seed)
    ref = blockwise_rows(a[rows], a_s[rows], b, b_s)
    assert_close_scaled(c[rows.to(c.device)], ref, what=what + " sampled rows")
    # all-rows checksum: sum_m C[m, n] = sum_kb ((sum_m a_s[m, kb] a[m, kb-block]) . b[n, kb-block]) b_s[n/128, kb]
    K = a.shape[1]
    wsum = (a.float().double().reshape(M, K // 128, 128) * a_s.double()[:, :, None]).sum(0).reshape(1, K)
    want = blockwise_rows(wsum, torch.ones(1, K // 128, dtype=torch.float64), b.float(), b_s)[0]
    got = c.double().sum(0).cpu()
    rms = ref.pow(2).mean().sqrt().item()
    bound = 1e-2 * rms * (M ** 0.5) + 1e-2 * want.abs()
    bad = (got - want).abs() > bound
    assert not bad.any(), "%s: column checksum off in %d columns (max %.3e, bound %.3e)" % (
        what, int(bad.sum()), (got - want).abs().max().item(), bound.min().item())


def _fp8_operands(dev, M, N, K, seed):
    torch.manual_seed(seed)
    x = torch.randn(M, K, device=dev).bfloat16()
    w = torch.randn(N, K, device=dev) * 0.02
    a, a_s = fp8_kernel.act_quant(x)
    b, b_s = fp8_kernel.weight_quant(w)
    return a, a_s, b, b_s


@pytest.mark.parametrize("N,K", LLAMA_NK)
@pytest.mark.parametrize("M", [1, 16, 256, 4096])
def test_fp8_gemm_config3_grid(dev, M, N, K):
    announce("fp8 grid", M, N, K)
    a, a_s, b, b_s = _fp8_operands(dev, M, N, K, M + N + K)
    with default_dtype(torch.bfloat16):
        c = fp8_kernel.fp8_gemm(a, a_s, b, b_s)
    assert c.shape == (M, N) and c.dtype == torch.bfloat16
    check_float_gemm(c, a.cpu(), a_s.cpu(), b.cpu(), b_s.cpu(), "fp8 %dx%dx%d" % (M, N, K))


def test_fp8_gemm_lm_head_shape(dev):
    """16 x 128256 x 4096 (the widest benchmarked weight): all 16 rows against the oracle."""
    M, N, K = 16, 128256, 4096
    announce("fp8 lm_head", M, N, K)
    a, a_s, b, b_s = _fp8_operands(dev, M, N, K, 77)
    with default_dtype(torch.bfloat16):
        c = fp8_kernel.fp8_gemm(a, a_s, b, b_s)
    check_float_gemm(c, a.cpu(), a_s.cpu(), b.cpu(), b_s.cpu(), "fp8 lm_head")


@pytest.mark.parametrize("N,K", [(4096, 4096), (14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("M", [1, 16, 128, 2048, 4096])
def test_int8_config2_grid_int32_bit_exact(dev, M, N, K):
    """Per-token x per-channel W8A8: the int32 accumulators equal the integer product (sampled rows plus exact
    row and column checksums over the whole matrix), the scaled bf16 output is within tolerance."""
    announce("int8 per-token grid", M, N, K)
    torch.manual_seed(M + N + K)
    a, a_s = int8_kernel.act_quant_per_token(torch.randn(M, K, device=dev))
    b, b_s = int8_kernel.weight_quant_per_channel(torch.randn(N, K, device=dev) * 0.02)
    with default_dtype(torch.bfloat16):
        c, acc = int8_kernel.int8_gemm_per_token(a, a_s, b, b_s, return_int32=True)
    assert acc.dtype == torch.int32 and c.dtype == torch.bfloat16
    ah, bh = a.cpu(), b.cpu()
    rows = sample_rows(M, seed=K)
    assert torch.equal(acc[rows.to(dev)].cpu(), g.int8_gemm_int32(ah[rows], bh))
    col = (ah.double().sum(0, keepdim=True) @ bh.double().T)[0].long()
    row = (ah.double() @ bh.double().sum(0))[..., None].long()[:, 0]
    assert torch.equal(acc.sum(0, dtype=torch.int64).cpu(), col)
    assert torch.equal(acc.sum(1, dtype=torch.int64).cpu(), row)
    assert bool(torch.isfinite(c).all())
    assert_close_scaled(c[rows.to(dev)], g.int8_gemm_rowcol(ah[rows], a_s.cpu()[rows], bh, b_s.cpu()),
                        what="int8 per-token scaled")


@pytest.mark.parametrize("M,N,K", [(4096, 14336, 4096), (2048, 4096, 14336), (4096, 4096, 4096), (128, 14336, 4096),
                                   (2048, 14336, 4096), (4096, 4096, 14336)])
def test_int8_block_gemm_bench_shapes(dev, M, N, K):
    """The reference signature (1 x 128 / 128 x 128 block scales, fp16) at the benchmarked shapes."""
    announce("int8 block", M, N, K)
    torch.manual_seed(M + N + K)
    a, a_s = int8_kernel.act_quant(torch.randn(M, K, device=dev))
    b, b_s = int8_kernel.weight_quant(torch.randn(N, K, device=dev) * 0.02)
    with default_dtype(torch.bfloat16):
        c = int8_kernel.int8_gemm(a, a_s, b, b_s)
    check_float_gemm(c, a.cpu(), a_s.cpu(), b.cpu(), b_s.cpu(), "int8 block %dx%dx%d" % (M, N, K))


def test_int8_block_accumulators_exact_at_4096_cubed(dev):
    """Unit scales, |values| <= 3, fp32 out: every 128-K partial and the full sum are exact integers."""
    M = N = K = 4096
    announce("int8 block exact", M, N, K)
    torch.manual_seed(3)
    a = torch.randint(-3, 4, (M, K), dtype=torch.int8)
    b = torch.randint(-3, 4, (N, K), dtype=torch.int8)
    ones_a = torch.ones(M, K // 128, dtype=torch.float16, device=dev)
    ones_b = torch.ones(N // 128, K // 128, dtype=torch.float16, device=dev)
    with default_dtype(torch.float32):
        c = int8_kernel.int8_gemm(a.to(dev), ones_a, b.to(dev), ones_b)
    rows = sample_rows(M, seed=5)
    assert torch.equal(c[rows.to(dev)].cpu().long(), a[rows].long() @ b.long().T)
    col = (a.double().sum(0, keepdim=True) @ b.double().T)[0]
    assert torch.equal(c.double().sum(0).cpu(), col)


@pytest.mark.parametrize("N,K", [(4096, 4096), (14336, 4096)])
@pytest.mark.parametrize("M", [16, 128, 1024, 4096])
def test_w4a8_config4_grid(dev, M, N, K):
    announce("w4a8 grid", M, N, K)
    torch.manual_seed(M + N)
    w = torch.randn(N, K, device=dev) * 0.02
    packed, s, s4, z4 = w4a8_kernel.weight_quant(w)
    a, a_s = w4a8_kernel.act_quant(torch.randn(M, K, device=dev).bfloat16())
    with default_dtype(torch.bfloat16):
        c = w4a8_kernel.w4a8_gemm(a, a_s, packed, s, s4, z4, 128, 8, "row")
    assert c.shape == (M, N) and c.dtype == torch.bfloat16
    wq = torch.from_numpy(bp.unpack_rows(packed.cpu().numpy(), 4, N))
    b8 = q.w4a8_dequant_int8(wq, s4.cpu(), z4.cpu())
    check_float_gemm(c, a.cpu(), a_s.cpu(), b8, s.cpu(), "w4a8 %dx%dx%d" % (M, N, K))


def _w4a16_check(C, A, w_deq_kn, what, seed=0):
    """A [M, K] fp16 (host), w_deq_kn [K, N] fp16 dequantised weights (host), C on the device."""
    M = A.shape[0]
    assert bool(torch.isfinite(C).all())
    rows = sample_rows(M, seed=seed)
    wd = w_deq_kn.double()
    ref = A[rows].double() @ wd
    assert_close_scaled(C[rows.to(C.device)], ref, what=what + " sampled rows")
    want = (A.double().sum(0, keepdim=True) @ wd)[0]
    got = C.double().sum(0).cpu()
    bound = 1e-2 * ref.pow(2).mean().sqrt().item() * (M ** 0.5) + 1e-2 * want.abs()
    assert bool(((got - want).abs() <= bound).all()), what + ": column checksum"
    return ref, rows


CONFIG1_GRID = [(M, N, K) for (N, K) in [(4096, 4096), (14336, 4096), (28672, 4096), (4096, 14336)] for M in (16, 128, 4096)]


@pytest.mark.parametrize("M,N,K", CONFIG1_GRID)
def test_mul_bench_shapes(dev, M, N, K):
    """simple-Marlin `mul` on every shape of configuration 1, beyond the 2048 rows of the reference's own recipe
    (test.py:139-157): same inputs recipe (randn * 0.1) and its 0.05 threshold on the sampled rows."""
    announce("marlin mul bench shape", M, N, K)
    torch.manual_seed(42)
    A = (torch.randn(M, K, device=dev) * 0.1).half()
    W = (torch.randn(K, N, device=dev) * 0.1).half()
    ref_deq, W_int4, scales = QuantUtils.fake_quantize(W, 128)
    B, sp = QuantUtils.pack(W_int4, scales, 128)
    C = torch.zeros(M, N, dtype=torch.half, device=dev)
    mul(A, B, C, sp, torch.zeros(N // 128 * 16, dtype=torch.int32, device=dev))
    deq = g.w4a16_dequant_kn(W_int4.cpu(), scales.cpu(), 128)
    assert torch.equal(deq, ref_deq.cpu())
    ref, rows = _w4a16_check(C, A.cpu(), deq, "mul %dx%dx%d" % (M, N, K))
    assert (C[rows.to(dev)].cpu().double() - ref).abs().max() <= 0.05


@pytest.mark.parametrize("M,N,K", CONFIG1_GRID + [(16, 128256, 4096), (2048, 28672, 4096)])
def test_w4a16_nk_bench_shapes(dev, M, N, K):
    """Configuration 1 layout ([N, K/8] bit-packed, s = absmax / 7) on every shape of the configuration and the
    widest weights; M = 4096 with N >= 14336 and the last shape take two or more rounds of 256 x 256 tiles and run on
    the tile kernel that expands the packed words itself."""
    announce("w4a16 nk bench shape", M, N, K)
    torch.manual_seed(1)
    x = torch.randn(M, K, device=dev).half()
    w = torch.randn(N, K, device=dev) * 0.02
    packed, s, qd = w4a16.quantize_nk(w, 128)
    y = w4a16.w4a16_gemm(x, packed, s, 128)
    deq_kn = g.w4a16_dequant_kn(qd.cpu().t().int().contiguous(), s.cpu().t().contiguous(), 128)
    _w4a16_check(y, x.cpu(), deq_kn, "w4a16 nk %dx%dx%d" % (M, N, K))
