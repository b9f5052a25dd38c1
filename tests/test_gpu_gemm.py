"""HIP block-scaled GEMMs vs the float64 oracle.

Tolerance: |c - ref| <= 1e-2 * rms(ref) + 1e-2 * |ref| (rtol 1e-2 / atol 1e-2 relative to the output
scale).  Integer accumulators are checked bit-exactly.
"""
import pytest
import torch

from oracle import gemm_ref as g, quant_ref as q, bitpack_ref as bp
from llm_kernels_amd import _lib
from llm_kernels_amd.quantization import fp8_kernel, int8_kernel, w4a8_kernel
from helpers import announce, assert_close_scaled, default_dtype

pytestmark = pytest.mark.gpu

SMALL = [(1, 128, 128), (16, 256, 512), (5, 130, 256), (33, 200, 384), (70, 64, 1024), (128, 512, 256)]


def _quant_inputs_fp8(M, N, K, seed):
    torch.manual_seed(seed)
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    a, a_s = q.act_quant_fp8(x)
    b, b_s = q.weight_quant_fp8(w)
    return a, a_s, b, b_s


@pytest.mark.parametrize("M,N,K", SMALL)
@pytest.mark.parametrize("out", [torch.bfloat16, torch.float16, torch.float32])
def test_fp8_gemm_small(dev, M, N, K, out):
    announce("fp8_gemm", M, N, K, out)
    a, a_s, b, b_s = _quant_inputs_fp8(M, N, K, M + N)
    with default_dtype(out):
        c = fp8_kernel.fp8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert c.dtype == out and c.shape == (M, N)
    assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="fp8_gemm")


def test_fp8_gemm_batched_leading_dims_and_asserts(dev):
    announce("fp8_gemm leading dims")
    a, a_s, b, b_s = _quant_inputs_fp8(6, 256, 256, 3)
    with default_dtype(torch.bfloat16):
        c = fp8_kernel.fp8_gemm(a.view(2, 3, 256).to(dev), a_s.view(2, 3, 2).to(dev), b.to(dev), b_s.to(dev))
    assert c.shape == (2, 3, 256)
    assert_close_scaled(c.view(6, 256), g.gemm_blockwise(a, a_s, b, b_s))
    with pytest.raises(AssertionError):
        fp8_kernel.fp8_gemm(a.to(dev).t(), a_s.to(dev), b.to(dev), b_s.to(dev))


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (16, 4096, 4096), (16, 6144, 4096), (256, 4096, 4096)])
def test_fp8_gemm_llama_shapes(dev, M, N, K):
    announce("fp8_gemm llama", M, N, K)
    a, a_s, b, b_s = _quant_inputs_fp8(M, N, K, 11)
    with default_dtype(torch.bfloat16):
        c = fp8_kernel.fp8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="fp8 llama")


def test_fp8_gemm_quantize_on_device_end_to_end(dev):
    """act_quant + weight_quant + fp8_gemm on the GPU against the unquantised product (reference-style check)."""
    announce("fp8 end to end 64x4096x14336")
    torch.manual_seed(5)
    x = torch.randn(64, 14336, device=dev).bfloat16()
    w = (torch.randn(4096, 14336, device=dev) * 0.02)
    a, a_s = fp8_kernel.act_quant(x)
    b, b_s = fp8_kernel.weight_quant(w)
    with default_dtype(torch.bfloat16):
        c = fp8_kernel.fp8_gemm(a, a_s, b, b_s)
    ref = x.float() @ w.t()
    cos = torch.nn.functional.cosine_similarity(c.float().flatten(), ref.flatten(), dim=0)
    assert cos > 0.999
    assert_close_scaled(c, g.gemm_blockwise(a.cpu(), a_s.cpu(), b.cpu(), b_s.cpu()), what="fp8 e2e")


# ------------------------------------------------------------------------------------------- int8
@pytest.mark.parametrize("M,N,K", SMALL + [(16, 4096, 4096), (128, 14336, 4096)])
def test_int8_gemm(dev, M, N, K):
    announce("int8_gemm", M, N, K)
    torch.manual_seed(M * 7 + N)
    a, a_s = q.act_quant_int8(torch.randn(M, K))
    b, b_s = q.weight_quant_int8(torch.randn(N, K) * 0.02)
    with default_dtype(torch.bfloat16):
        c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert c.dtype == torch.bfloat16
    assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="int8_gemm")


@pytest.mark.parametrize("M,N,K", [(1, 128, 128), (16, 256, 4096), (37, 130, 512), (128, 512, 14336), (3850, 4110, 640)])
def test_int8_block_accumulators_bit_exact(dev, M, N, K):
    """Unit scales and fp32 output: the result is the exact integer product (every 128-K int32 partial
    and their sum stay below 2^24 for |values| <= 15)."""
    announce("int8 exact", M, N, K)
    torch.manual_seed(K)
    a = torch.randint(-15, 16, (M, K), dtype=torch.int8)
    b = torch.randint(-15, 16, (N, K), dtype=torch.int8)
    a_s = torch.ones(M, K // 128, dtype=torch.float16)
    b_s = torch.ones((N + 127) // 128, K // 128, dtype=torch.float16)
    with default_dtype(torch.float32):
        c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert torch.equal(c.cpu().long(), a.long() @ b.long().T)
    # full-range values, one K block: a single int32 partial (|sum| <= 128*127*127 < 2^24) is exact in fp32
    a1 = torch.randint(-127, 128, (M, 128), dtype=torch.int8)
    b1 = torch.randint(-127, 128, (N, 128), dtype=torch.int8)
    with default_dtype(torch.float32):
        c1 = int8_kernel.int8_gemm(a1.to(dev), a_s[:, :1].contiguous().to(dev), b1.to(dev), b_s[:, :1].contiguous().to(dev))
    assert torch.equal(c1.cpu().long(), a1.long() @ b1.long().T)


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (16, 4096, 4096), (130, 200, 1024), (128, 4096, 14336),
                                   (65, 136, 128), (300, 264, 640), (1000, 521, 1152), (2048, 4096, 2048),
                                   (4096, 4096, 1024), (3850, 4110, 640),
                                   (300, 1000, 8192), (70, 1001, 8192), (100, 2050, 4096)])   # K split into 7, 8, 4
def test_int8_per_token_int32_bit_exact(dev, M, N, K):
    announce("int8 rowcol", M, N, K)
    torch.manual_seed(M + K)
    a, a_s = q.int8_quant_rowwise(torch.randn(M, K))
    b, b_s = q.int8_quant_rowwise(torch.randn(N, K) * 0.02)
    with default_dtype(torch.bfloat16):
        c, acc = int8_kernel.int8_gemm_per_token(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev), return_int32=True)
    assert acc.dtype == torch.int32 and torch.equal(acc.cpu(), g.int8_gemm_int32(a, b))
    assert_close_scaled(c, g.int8_gemm_rowcol(a, a_s, b, b_s), what="int8 rowcol")
    # without scratch the entry point cannot split K: the slices' integer sums must give the same bits
    ad, bd, asd, bsd = a.to(dev), b.to(dev), a_s.to(dev).float().contiguous(), b_s.to(dev).float().contiguous()
    c0 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    _lib.call("llmk_gemm_i8_rowcol", _lib.ptr(ad), _lib.ptr(asd), _lib.ptr(bd), _lib.ptr(bsd), _lib.ptr(c0),
              _lib.dt(c0.dtype), None, M, N, K, None, 0, _lib.stream(ad))
    assert torch.equal(c0, c), "int8 rowcol: split and unsplit K differ"
    with default_dtype(torch.float32):     # scaled output alone (no accumulator buffer), full-range operands
        a2 = torch.randint(-128, 128, (M, K), dtype=torch.int8)
        b2 = torch.randint(-128, 128, (N, K), dtype=torch.int8)
        c2 = int8_kernel.int8_gemm_per_token(a2.to(dev), a_s.to(dev), b2.to(dev), b_s.to(dev))
    assert_close_scaled(c2, g.int8_gemm_rowcol(a2, a_s, b2, b_s), what="int8 rowcol full range")
    ag, asg = int8_kernel.act_quant_per_token(torch.randn(M, K, device=dev))
    assert ag.dtype == torch.int8 and asg.shape == (M,)


# ------------------------------------------------------------------------------------------- w4a8
@pytest.mark.parametrize("M,N,K", [(1, 128, 128), (16, 256, 512), (37, 136, 256), (16, 4096, 4096), (128, 1024, 7168),
                                   (5, 8, 128), (33, 264, 2048), (64, 4096, 4096), (17, 1032, 2176), (16, 14336, 4096),
                                   (16, 512, 4224), (16, 4096, 14336), (64, 520, 12416)])
def test_w4a8_gemm(dev, M, N, K):
    announce("w4a8_gemm", M, N, K)
    torch.manual_seed(N + K)
    wq, s, s4, z4 = q.w4a8_weight_quant_levels(torch.randn(N, K) * 0.02)
    a, a_s = q.act_quant_int8(torch.randn(M, K).bfloat16(), rounding="up")
    packed, _ = bp.pack_rows(wq.numpy(), 4, 32)
    with default_dtype(torch.bfloat16):
        c = w4a8_kernel.w4a8_gemm(a.to(dev), a_s.to(dev), torch.from_numpy(packed).to(dev), s.to(dev),
                                  s4.to(dev), z4.to(dev), 128, 8, "row")
    assert c.shape == (M, N) and c.dtype == torch.bfloat16
    assert_close_scaled(c, g.w4a8_gemm(a, a_s, wq, s, s4, z4), what="w4a8_gemm")


def test_w4a8_exact_and_wrap(dev):
    """Unit block scales + fp32 out: exact integers, including out-of-contract s4/z4 that wrap in int8."""
    announce("w4a8 exact/wrap")
    torch.manual_seed(9)
    M, N, K = 8, 64, 256
    wq = torch.randint(0, 16, (N, K), dtype=torch.uint8)
    s4 = torch.randint(1, 4, (N, K // 128), dtype=torch.int8)
    z4 = torch.randint(0, 16, (N, K // 128), dtype=torch.int8)
    s4[0, 0], z4[0, 0] = 20, 2            # (15 - 2) * 20 = 260 wraps
    s4[1, 1], z4[1, 1] = -9, 15           # negative scale
    a = torch.randint(-7, 8, (M, K), dtype=torch.int8)
    ones_a = torch.ones(M, K // 128, dtype=torch.float16)
    ones_b = torch.ones(1, K // 128, dtype=torch.float16)
    packed, _ = bp.pack_rows(wq.numpy(), 4, 32)
    with default_dtype(torch.float32):
        c = w4a8_kernel.w4a8_gemm(a.to(dev), ones_a.to(dev), torch.from_numpy(packed).to(dev), ones_b.to(dev),
                                  s4.to(dev), z4.to(dev))
    b8 = q.w4a8_dequant_int8(wq, s4, z4)
    assert torch.equal(c.cpu().long(), a.long() @ b8.long().T)


@pytest.mark.parametrize("M,N,K,sdt", [(16, 5000, 1024, torch.float16), (40, 8192, 4096, torch.float32),
                                       (3, 312, 384, torch.bfloat16), (16, 1032, 8320, torch.float16),
                                       (50, 264, 14336, torch.float32)])
def test_w4a8_decode_exact_mixed_wrap(dev, M, N, K, sdt):
    """Decode-size shapes over many column tiles with a sprinkle of out-of-contract (s4, z4): exact integers."""
    announce("w4a8 decode exact", M, N, K, sdt)
    torch.manual_seed(M + N)
    wq = torch.randint(0, 16, (N, K), dtype=torch.uint8)
    s4 = torch.randint(1, 9, (N, K // 128), dtype=torch.int8)
    z4 = torch.randint(0, 16, (N, K // 128), dtype=torch.int8)
    wild = torch.rand(N, K // 128) < 0.02
    s4[wild] = torch.randint(-128, 128, (int(wild.sum()),), dtype=torch.int8)
    z4[wild] = torch.randint(-128, 128, (int(wild.sum()),), dtype=torch.int8)
    a = torch.randint(-3, 4, (M, K), dtype=torch.int8)
    ones_a = torch.ones(M, K // 128, dtype=sdt)
    ones_b = torch.ones((N + 127) // 128, K // 128, dtype=sdt)
    packed, _ = bp.pack_rows(wq.numpy(), 4, 32)
    with default_dtype(torch.float32):
        c = w4a8_kernel.w4a8_gemm(a.to(dev), ones_a.to(dev), torch.from_numpy(packed).to(dev), ones_b.to(dev),
                                  s4.to(dev), z4.to(dev))
    b8 = q.w4a8_dequant_int8(wq, s4, z4)
    assert torch.equal(c.cpu().long(), a.long() @ b8.long().T)


@pytest.mark.parametrize("M,N,K,sdt", [(160, 4096, 1024, torch.float16), (200, 520, 3200, torch.float32),
                                       (256, 1032, 2176, torch.bfloat16), (161, 8, 128, torch.float16),
                                       (250, 2048, 8192, torch.float16), (256, 264, 14336, torch.float32),
                                       (130, 4104, 4096, torch.bfloat16),
                                       # more than 256 tiles of 64 columns, up to 128 rows: the 128-column tile kernel
                                       (97, 9000, 4096, torch.float16), (128, 8200, 4224, torch.float32)])
def test_w4a8_mid_m_fused_tiles_exact_mixed_wrap(dev, M, N, K, sdt):
    """Mid-size M: the tile kernels unpack and dequantise the packed words inside their K loop (no int8 copy of
    W).  Unit block scales, fp32 out, 2 % out-of-contract (s4, z4) pairs: exact integers with the int8 wrap,
    over ragged row and column tiles, K tails, split K (few tiles, long K) and every scale dtype."""
    announce("w4a8 fused tiles exact", M, N, K, sdt)
    lib = _lib.load()
    # these shapes take the fused tile path: their scratch is that of the int8 tile kernels (activation scales,
    # split-K partial sums) with no int8 copy of the weights in front
    assert lib.llmk_gemm_w4a8_workspace_bytes(M, N, K, 128) == lib.llmk_gemm_workspace_bytes(M, N, K)
    torch.manual_seed(M + N)
    wq = torch.randint(0, 16, (N, K), dtype=torch.uint8)
    s4 = torch.randint(1, 9, (N, K // 128), dtype=torch.int8)
    z4 = torch.randint(0, 16, (N, K // 128), dtype=torch.int8)
    wild = torch.rand(N, K // 128) < 0.02
    s4[wild] = torch.randint(-128, 128, (int(wild.sum()),), dtype=torch.int8)
    z4[wild] = torch.randint(-128, 128, (int(wild.sum()),), dtype=torch.int8)
    a = torch.randint(-3, 4, (M, K), dtype=torch.int8)
    ones_a = torch.ones(M, K // 128, dtype=sdt)
    ones_b = torch.ones((N + 127) // 128, K // 128, dtype=sdt)
    packed, _ = bp.pack_rows(wq.numpy(), 4, 32)
    with default_dtype(torch.float32):
        c = w4a8_kernel.w4a8_gemm(a.to(dev), ones_a.to(dev), torch.from_numpy(packed).to(dev), ones_b.to(dev),
                                  s4.to(dev), z4.to(dev))
    b8 = q.w4a8_dequant_int8(wq, s4, z4)
    assert torch.equal(c.cpu().long(), (a.double() @ b8.double().T).long())      # exact: every sum is far below 2^53


@pytest.mark.parametrize("M,N,K", [(128, 4096, 4096), (256, 1024, 7168), (512, 4096, 4096), (384, 14336, 4096),
                                   (96, 2056, 14336)])
def test_w4a8_mid_m_fused_tiles(dev, M, N, K):
    """The same path on quantised operands with real scales, against the float64 oracle."""
    announce("w4a8 fused tiles", M, N, K)
    torch.manual_seed(N + K)
    wq, s, s4, z4 = q.w4a8_weight_quant_levels(torch.randn(N, K) * 0.02)
    a, a_s = q.act_quant_int8(torch.randn(M, K).bfloat16(), rounding="up")
    packed, _ = bp.pack_rows(wq.numpy(), 4, 32)
    with default_dtype(torch.bfloat16):
        c = w4a8_kernel.w4a8_gemm(a.to(dev), a_s.to(dev), torch.from_numpy(packed).to(dev), s.to(dev),
                                  s4.to(dev), z4.to(dev), 128, 8, "row")
    assert_close_scaled(c, g.w4a8_gemm(a, a_s, wq, s, s4, z4), what="w4a8 fused tiles")


@pytest.mark.parametrize("sdt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(128, 4096, 4096), (200, 520, 3200), (257, 1032, 8192)])
def test_int8_mid_m_scale_dtypes(dev, M, N, K, sdt):
    """Mid-size M, int8 blocks: the kernel stages 16-bit activation scales as they are; every scale dtype gives the
    oracle's result on the same (rounded) scales."""
    announce("int8 mid-M scale dtype", M, N, K, sdt)
    torch.manual_seed(M + K)
    a, a_s = q.act_quant_int8(torch.randn(M, K).bfloat16() * 3)
    b, b_s = q.weight_quant_int8(torch.randn(N, K) * 0.02)
    a_s, b_s = a_s.to(sdt), b_s.to(sdt)
    with default_dtype(torch.float32):
        c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="int8 mid-M scales " + str(sdt))


def _random_mid_shapes(n, seed):
    import random
    rnd = random.Random(seed)
    shapes = []
    for _ in range(n):
        M = rnd.choice([65, 66, 96, 127, 128, 129, 160, 255, 256, 257, 300, 384, 511, 512, 513, 700, 1024])
        N = rnd.choice([8, 24, 64, 72, 128, 136, 520, 1000, 2048, 2056, 4096, 4104, 6144])
        K = 128 * rnd.choice([1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 32, 40, 64])
        shapes.append((M, N, K))
    return shapes


@pytest.mark.parametrize("M,N,K", _random_mid_shapes(28, 7))
def test_mid_and_small_tile_kernels_exact_integers(dev, M, N, K):
    """Random mid-size shapes (ragged row and column tiles, K tails, split K, one or more rounds of tiles) with small
    integer operands, unit block scales of a random dtype and fp32 output: the block-scaled int8 and fp8 GEMMs and the
    per-token int8 GEMM must return the exact integer product (every partial sum is below 2^24)."""
    announce("mid-size exact", M, N, K)
    torch.manual_seed(M * 7 + N + K)
    a = torch.randint(-7, 8, (M, K), dtype=torch.int8)
    b = torch.randint(-7, 8, (N, K), dtype=torch.int8)
    ref = (a.double() @ b.double().T).long()
    sdt = [torch.float16, torch.bfloat16, torch.float32][(M + N + K // 128) % 3]
    a_s = torch.ones(M, K // 128, dtype=sdt)
    b_s = torch.ones((N + 127) // 128, K // 128, dtype=sdt)
    with default_dtype(torch.float32):
        c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
        assert torch.equal(c.cpu().long(), ref), "int8 block"
        # the same integers are exact in e4m3 (|v| <= 7)
        c8 = fp8_kernel.fp8_gemm(a.float().to(torch.float8_e4m3fn).to(dev), a_s.float().to(dev),
                                 b.float().to(torch.float8_e4m3fn).to(dev), b_s.float().to(dev))
        assert torch.equal(c8.cpu().long(), ref), "fp8 block"
        _, acc = int8_kernel.int8_gemm_per_token(a.to(dev), torch.ones(M).to(dev), b.to(dev), torch.ones(N).to(dev),
                                                 return_int32=True)
        assert torch.equal(acc.cpu().long(), ref), "int8 per token"


@pytest.mark.parametrize("M,N,K", [(130, 9000, 640), (300, 5000, 1152), (500, 3208, 384), (100, 16000, 256), (128, 20000, 640),
                                   (256, 14336, 4096), (512, 6144, 8192)])
def test_fp8_one_round_of_128_column_tiles(dev, M, N, K):
    """fp8 block GEMM on weights too wide for the 64-column mid-size kernel that fit one round of 64- or 128-row by
    128-column tiles (the 128-column form of the producer / consumer kernel): ragged rows and columns, odd numbers of
    K blocks.  Small integers with unit scales must come out exactly; quantised random operands within 1e-2 of the
    oracle."""
    announce("fp8 128-column mid-size", M, N, K)
    torch.manual_seed(M + N + K)
    a = torch.randint(-7, 8, (M, K), dtype=torch.int8)
    b = torch.randint(-7, 8, (N, K), dtype=torch.int8)
    with default_dtype(torch.float32):
        c = fp8_kernel.fp8_gemm(a.float().to(torch.float8_e4m3fn).to(dev), torch.ones(M, K // 128).to(dev),
                                b.float().to(torch.float8_e4m3fn).to(dev), torch.ones((N + 127) // 128, K // 128).to(dev))
    assert torch.equal(c.cpu().long(), (a.double() @ b.double().T).long())
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    aq, a_s = q.act_quant_fp8(x)
    bq, b_s = q.weight_quant_fp8(w)
    with default_dtype(torch.bfloat16):
        c = fp8_kernel.fp8_gemm(aq.to(dev), a_s.to(dev), bq.to(dev), b_s.to(dev))
    assert_close_scaled(c, g.gemm_blockwise(aq, a_s, bq, b_s), what="fp8 128-column mid-size")


@pytest.mark.parametrize("kind", ["fp8", "int8"])
@pytest.mark.parametrize("M,N,K,out", [(128, 1024, 4096, torch.bfloat16), (200, 520, 3200, torch.float32),
                                       (70, 136, 1152, torch.float16), (300, 2048, 8192, torch.bfloat16),
                                       (48, 2560, 16384, torch.bfloat16), (64, 14336, 4096, torch.float16),
                                       (256, 4096, 14336, torch.bfloat16),
                                       # fp8: K slices of the 128-column form of the mid-size kernel (rows beyond 8 KB on few tiles)
                                       (128, 4096, 14336, torch.bfloat16), (100, 3000, 10240, torch.float32),
                                       (256, 14336, 14336, torch.float16)])
def test_mid_m_split_k_shapes(dev, kind, M, N, K, out):
    """Mid-size M with few column tiles: the K range is split over workgroups (uneven slices included)."""
    announce("split-K", kind, M, N, K, out)
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    with default_dtype(out):
        if kind == "fp8":
            a, a_s = q.act_quant_fp8(x)
            b, b_s = q.weight_quant_fp8(w)
            c = fp8_kernel.fp8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
        else:
            a, a_s = q.act_quant_int8(x)
            b, b_s = q.weight_quant_int8(w)
            c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert c.dtype == out
    assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="split-K " + kind)


@pytest.mark.parametrize("kind", ["fp8", "int8"])
@pytest.mark.parametrize("M,N,K,out", [(16, 4096, 14336, torch.bfloat16), (1, 1000, 8192, torch.float32),
                                       (13, 264, 4224, torch.float16), (50, 520, 12416, torch.bfloat16),
                                       (16, 28672, 4224, torch.bfloat16), (33, 136, 16384, torch.float32)])
def test_decode_k_ranges(dev, kind, M, N, K, out):
    """Decode-sized M with K > 4096: the weight-streaming kernel runs on K ranges side by side and a second
    kernel adds the fp32 partial sums (ragged last range, ragged rows and columns included)."""
    announce("K ranges", kind, M, N, K, out)
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    with default_dtype(out):
        if kind == "fp8":
            a, a_s = q.act_quant_fp8(x)
            b, b_s = q.weight_quant_fp8(w)
            c = fp8_kernel.fp8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
        else:
            a, a_s = q.act_quant_int8(x)
            b, b_s = q.weight_quant_int8(w)
            c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert c.dtype == out
    assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="K ranges " + kind)


def test_int8_decode_k_ranges_exact(dev):
    """Unit scales, small integers: the sum over K ranges is the exact integer product."""
    announce("K ranges exact")
    torch.manual_seed(9)
    M, N, K = 16, 1032, 12416
    a = torch.randint(-15, 16, (M, K), dtype=torch.int8)
    b = torch.randint(-15, 16, (N, K), dtype=torch.int8)
    a_s = torch.ones(M, K // 128, dtype=torch.float32)
    b_s = torch.ones((N + 127) // 128, K // 128, dtype=torch.float32)
    with default_dtype(torch.float32):
        c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert torch.equal(c.cpu().long(), a.long() @ b.long().T)


def test_fp8_gemm_without_scratch_takes_the_streaming_kernel(dev):
    """The scratch is optional: the same call without it runs another kernel and agrees with the oracle too."""
    announce("fp8 no scratch")
    torch.manual_seed(5)
    M, N, K = 48, 2560, 8192
    a, a_s = q.act_quant_fp8(torch.randn(M, K).bfloat16())
    b, b_s = q.weight_quant_fp8(torch.randn(N, K) * 0.02)
    ad, asd, bd, bsd = a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev)
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    _lib.call("llmk_gemm_fp8_block", _lib.ptr(ad), _lib.ptr(asd), _lib.ptr(bd), _lib.ptr(bsd), _lib.ptr(c),
              _lib.dt(c.dtype), M, N, K, None, 0, _lib.stream(ad))
    ref = g.gemm_blockwise(a, a_s, b, b_s)
    assert_close_scaled(c, ref, what="fp8 without scratch")
    with default_dtype(torch.bfloat16):
        c2 = fp8_kernel.fp8_gemm(ad, asd, bd, bsd)
    assert_close_scaled(c2, ref, what="fp8 with scratch")


@pytest.mark.parametrize("kind", ["fp8", "int8"])
@pytest.mark.parametrize("M,N,K", [(65, 128, 128), (130, 200, 256), (300, 384, 512), (520, 256, 384), (1100, 130, 256)])
def test_tiled_kernels_ragged_shapes(dev, kind, M, N, K):
    """Shapes that exercise every tile height of the large-M kernel, with ragged M and N."""
    announce("tiled ragged", kind, M, N, K)
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    if kind == "fp8":
        a, a_s = q.act_quant_fp8(x)
        b, b_s = q.weight_quant_fp8(w)
        fn = fp8_kernel.fp8_gemm
    else:
        a, a_s = q.act_quant_int8(x)
        b, b_s = q.weight_quant_int8(w)
        fn = int8_kernel.int8_gemm
    for out in (torch.bfloat16, torch.float32):
        with default_dtype(out):
            c = fn(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
        assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="tiled %s" % kind)


@pytest.mark.parametrize("kind", ["fp8", "int8", "int8_f32scales"])
@pytest.mark.parametrize("M,N,K", [(4000, 4100, 256), (4096, 4096, 384), (3900, 4352, 128)])
def test_wide_tile_kernel_ragged_shapes(dev, kind, M, N, K):
    """Shapes large enough for the 256 x 256 tile, with ragged M and N, odd and single K step counts."""
    announce("wide ragged", kind, M, N, K)
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    if kind == "fp8":
        a, a_s = q.act_quant_fp8(x)
        b, b_s = q.weight_quant_fp8(w)
        fn = fp8_kernel.fp8_gemm
    else:
        a, a_s = q.act_quant_int8(x)
        b, b_s = q.weight_quant_int8(w)
        if kind == "int8_f32scales":
            a_s, b_s = a_s.float(), b_s.float()
        fn = int8_kernel.int8_gemm
    ref = g.gemm_blockwise(a, a_s, b, b_s)
    for out in (torch.bfloat16, torch.float32):
        with default_dtype(out):
            c = fn(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
        assert_close_scaled(c, ref, what="wide %s" % kind)


@pytest.mark.parametrize("kind", ["fp8", "int8"])
@pytest.mark.parametrize("M,N,K,out", [(5120, 10240, 8192, torch.bfloat16), (4096, 4608, 8192, torch.float32),
                                       (5000, 10200, 8192, torch.float16), (1100, 1300, 8192, torch.bfloat16)])
def test_large_tiles_split_last_round(dev, kind, M, N, K, out):
    """Long K and a tile count that leaves a short last round of 256 workgroups: 800 tiles of 256 x 256 (three
    rounds and 32 tiles, split eight ways), 576 tiles of 128 x 256 (two rounds and 64 tiles, split four ways), the
    first again with ragged rows and columns, and a small problem on smaller tiles for contrast.  The tiles of the
    short round are split along K and a second kernel adds the fp32 partial sums.  Every output dtype."""
    announce("split last round", kind, M, N, K, out)
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    with default_dtype(out):
        if kind == "fp8":
            a, a_s = q.act_quant_fp8(x)
            b, b_s = q.weight_quant_fp8(w)
            c = fp8_kernel.fp8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
        else:
            a, a_s = q.act_quant_int8(x)
            b, b_s = q.weight_quant_int8(w)
            c = int8_kernel.int8_gemm(a.to(dev), a_s.to(dev), b.to(dev), b_s.to(dev))
    assert c.dtype == out
    rows = torch.randperm(M)[:96].sort().values                     # 96 random rows, all columns; every element finite
    assert bool(torch.isfinite(c).all())
    assert_close_scaled(c[rows.to(dev)], g.gemm_blockwise(a[rows], a_s[rows], b, b_s), what="split last round " + kind)
    # all rows: column sums against a one-row oracle GEMM of the scale-weighted column sums of A
    wsum = (a.float().double().reshape(M, K // 128, 128) * a_s.double()[:, :, None]).sum(0).reshape(1, K)
    want = g.gemm_blockwise(wsum, torch.ones(1, K // 128, dtype=torch.float64), b.float(), b_s)[0]
    got = c.double().sum(0).cpu()
    ref_rms = g.gemm_blockwise(a[rows], a_s[rows], b, b_s).pow(2).mean().sqrt().item()
    assert bool(((got - want).abs() <= 1e-2 * ref_rms * (M ** 0.5) + 1e-2 * want.abs()).all()), "column sums"
