"""W4A16 GEMMs (simple-Marlin layout `mul`, and the [N, K/8] bit-packed layout) vs the oracle."""
import pytest
import torch

from oracle import gemm_ref as g, marlin_ref as mr, quant_ref as q, bitpack_ref as bp
from llm_kernels_amd.fast_dequant.simple_marlin.utils import QuantUtils
from llm_kernels_amd.fast_dequant.simple_marlin.marlin import mul
from llm_kernels_amd.fast_dequant import w4a16
from llm_kernels_amd import _lib
from helpers import announce, assert_close_scaled

pytestmark = pytest.mark.gpu

# the 14 shapes of the reference's own accuracy test (fast_dequant/simple_marlin/test.py:139-157)
REFERENCE_CASES = [
    (16, 64, 128, 128), (16, 128, 128, 128), (16, 64, 512, 128), (16, 64, 1024, 128),
    (256, 512, 1024, 128), (512, 256, 1024, 128), (1024, 1024, 512, 128), (128, 2048, 1024, 128),
    (1024, 2048, 2048, 128), (2048, 1024, 1024, 128), (512, 4096, 2048, 128),
    (256, 512, 1024, 64), (256, 512, 1024, 256), (512, 512, 512, 512),
]


@pytest.mark.parametrize("M,N,K,groupsize", REFERENCE_CASES)
def test_mul_reference_recipe(dev, M, N, K, groupsize):
    """Recipe of the reference test: seed 42, inputs randn * 0.1, pass = every |diff| <= 0.05."""
    announce("marlin mul", M, N, K, groupsize)
    torch.manual_seed(42)
    A = (torch.randn(M, K) * 0.1).half()
    W = (torch.randn(K, N) * 0.1).half()
    ref_deq, W_int4, scales = mr.fake_quantize(W, groupsize)
    B, sp = mr.pack(W_int4, scales, groupsize)
    C = torch.zeros(M, N, dtype=torch.half, device=dev)
    workspace = torch.zeros(N // 128 * 16 + 16, dtype=torch.int32, device=dev)
    ret = mul(A.to(dev), B.to(dev), C, sp.to(dev), workspace)
    assert ret is None
    ref = g.w4a16_gemm(A, W_int4, scales, groupsize)
    assert (C.cpu().double() - ref).abs().max() <= 0.05            # the reference's acceptance threshold
    assert_close_scaled(C, ref, what="marlin mul")
    assert torch.allclose(ref, A.double() @ ref_deq.double())


def test_mul_quantize_and_pack_on_device(dev):
    announce("marlin device-side pack")
    torch.manual_seed(1)
    M, N, K, g_ = 16, 4096, 4096, 128
    A = torch.randn(M, K, device=dev).half()
    W = (torch.randn(K, N, device=dev) * 0.02).half()
    ref_deq, W_int4, scales = QuantUtils.fake_quantize(W, g_)
    B, sp = QuantUtils.pack(W_int4, scales, g_)
    assert B.shape == (K // 16, 2 * N) and B.dtype == torch.int32 and B.device == W.device
    oB, osp = mr.pack(W_int4.cpu(), scales.cpu(), g_)
    assert torch.equal(B.cpu(), oB) and torch.equal(sp.cpu(), osp)
    C = torch.zeros(M, N, dtype=torch.half, device=dev)
    mul(A, B, C, sp, torch.zeros(512, dtype=torch.int32, device=dev))
    assert_close_scaled(C, A.double().cpu() @ ref_deq.double().cpu(), what="marlin 16x4096x4096")


@pytest.mark.parametrize("M,N,K,groupsize", [(16, 64, 16, 16), (16, 192, 48, 16), (32, 64, 256, 32), (48, 320, 128, -1)])
def test_mul_edge_shapes(dev, M, N, K, groupsize):
    announce("marlin edge", M, N, K, groupsize)
    torch.manual_seed(M + N + K)
    A = (torch.randn(M, K) * 0.5).half()
    W = (torch.randn(K, N) * 0.1).half()
    _, W_int4, scales = mr.fake_quantize(W, groupsize)
    # the kernel reads scales in the grouped permutation; pack with an explicit group size of K for -1
    B, sp = mr.pack(W_int4, scales, K if groupsize == -1 else groupsize)
    C = torch.full((M, N), 7.0, dtype=torch.half, device=dev)
    mul(A.to(dev), B.to(dev), C, sp.to(dev), torch.zeros(64, dtype=torch.int32, device=dev))
    assert_close_scaled(C, g.w4a16_gemm(A, W_int4, scales, groupsize), what="marlin edge")


def test_mul_error_behaviour(dev):
    announce("marlin errors")
    A = torch.zeros(16, 64, dtype=torch.half, device=dev)
    B = torch.zeros(4, 128, dtype=torch.int32, device=dev)
    C = torch.zeros(16, 64, dtype=torch.half, device=dev)
    s = torch.ones(1, 64, dtype=torch.half, device=dev)
    ws = torch.zeros(16, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        mul(A[:15], B, C[:15], s, ws)                       # M % 16
    with pytest.raises(RuntimeError):
        mul(A.float(), B, C, s, ws)                         # dtype
    with pytest.raises(RuntimeError):
        mul(A, B.long(), C, s, ws)
    with pytest.raises(RuntimeError):
        mul(A, B, C, s[:, :32].contiguous(), ws)            # scale N mismatch
    with pytest.raises(RuntimeError):
        mul(A, B, C.cpu(), s, ws)                           # device mismatch


# ----------------------------------------------------------------------------- [N, K/8] layout (config 1)
@pytest.mark.parametrize("M,N,K,gs", [(16, 4096, 4096, 128), (1, 64, 128, 128), (7, 100, 256, 64), (16, 256, 512, 32),
                                      (40, 512, 1024, 128), (16, 128, 384, -1), (16, 28672, 4096, 128), (16, 1000, 14336, 128),
                                      (3, 8200, 4096, 256), (32, 4100, 2048, 128), (64, 520, 8192, 128), (33, 4096, 512, 512),
                                      (300, 1000, 512, 64), (4096, 4096, 256, 128), (48, 1000, 12416, 128), (1, 4096, 14336, 128),
                                      (64, 264, 8448, 256), (20, 129, 4224, 128), (16, 264, 8320, 128)])
def test_w4a16_nk(dev, M, N, K, gs):
    announce("w4a16 nk", M, N, K, gs)
    torch.manual_seed(0)
    x = torch.randn(M, K).half()
    w = torch.randn(N, K) * 0.02
    grp = K if gs == -1 else gs
    qn, s = q.w4a16_quant_nk(w, grp)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    y = w4a16.w4a16_gemm(x.to(dev), torch.from_numpy(packed).to(dev), s.to(dev), gs)
    assert y.dtype == torch.half and y.shape == (M, N)
    ref = g.w4a16_gemm(x, qn.t().int().contiguous(), s.t().contiguous(), grp)
    assert_close_scaled(y, ref, what="w4a16 nk")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,K,gs", [(4096, 4096, 128), (257, 1024, 64), (96, 512, 32), (33, 1024, 512), (5, 64, 8)])
def test_w4a16_nk_device_quantize_round_trip(dev, dtype, N, K, gs):
    """One-pass quantiser of the [N, K/8] layout: codes, scales and packed words bit-exact against the oracle's
    absmax/7 rule and the bit-packing oracle (every division is an IEEE fp32 division on both sides)."""
    announce("w4a16 nk quantize on device", dtype, N, K, gs)
    torch.manual_seed(3)
    from llm_kernels_amd.quantization.bitpack import unpack_over_cols
    w = (torch.randn(N, K) * 0.02).to(dtype)
    w[N // 2, :gs] = 0                                              # a group of zeros: scale 0, codes 8
    packed, s, qd = w4a16.quantize_nk(w.to(dev), gs)
    oq, os_ = q.w4a16_quant_nk(w, gs)
    oq[N // 2, :gs] = 8
    assert packed.shape == (N, K // 8) and packed.dtype == torch.int32
    assert torch.equal(s.cpu(), os_)
    assert torch.equal(qd.cpu(), oq)
    opacked, _ = bp.pack_cols(oq.numpy(), 4, 32)
    assert torch.equal(packed.cpu(), torch.from_numpy(opacked))
    assert torch.equal(unpack_over_cols(packed, 4, K), qd)          # pack/unpack round trip, bit exact


def test_w4a16_nk_device_quantize_refuses_bad_shapes(dev):
    w = torch.randn(16, 256, device=dev)
    with pytest.raises(AssertionError):
        w4a16.quantize_nk(w, 96)                                    # not a divisor of K
    with pytest.raises(AssertionError):
        w4a16.quantize_nk(w[:, :48].contiguous(), 48)               # not a power of two
    with pytest.raises(AssertionError):
        w4a16.quantize_nk(w.double(), 128)


@pytest.mark.parametrize("M,N,K", [(16, 4096, 4096), (32, 1024, 4096), (64, 512, 8192), (16, 256, 14336)])
def test_mul_split_k_is_deterministic_and_rearms(dev, M, N, K):
    """Decode shapes split K over workgroups inside one launch; repeated launches must give identical bits
    (fixed summation order) and leave the ticket counters re-armed."""
    announce("marlin split-k repeat", M, N, K)
    torch.manual_seed(7)
    A = (torch.randn(M, K) * 0.3).half()
    W = (torch.randn(K, N) * 0.05).half()
    _, q, s = mr.fake_quantize(W, 128)
    B, sp = mr.pack(q, s, 128)
    Ag, Bg, sg = A.to(dev), B.to(dev), sp.to(dev)
    ws = torch.zeros(64, dtype=torch.int32, device=dev)
    outs = []
    for _ in range(20):
        C = torch.empty(M, N, dtype=torch.half, device=dev)
        mul(Ag, Bg, C, sg, ws)
        outs.append(C)
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    assert_close_scaled(outs[0], g.w4a16_gemm(A, q, s, 128), what="marlin split-k")


# ------------------------------------------------- compute-bound shapes: dequantise to fp16, then the 256 x 256 tile kernel
@pytest.mark.parametrize("M,N,K,gs", [(4096, 4096, 256, 128), (4000, 4032, 192, 64), (3856, 4160, 64, 16), (4096, 4096, 128, -1)])
def test_mul_large_tile_shapes(dev, M, N, K, gs):
    announce("marlin large tiles", M, N, K, gs)
    torch.manual_seed(M + K)
    A = (torch.randn(M, K) * 0.3).half()
    W = (torch.randn(K, N) * 0.05).half()
    _, q4, s = mr.fake_quantize(W, gs)
    B, sp = mr.pack(q4, s, K if gs == -1 else gs)          # the kernel reads scales in the grouped permutation
    C = torch.zeros(M, N, dtype=torch.half, device=dev)
    mul(A.to(dev), B.to(dev), C, sp.to(dev), torch.zeros(64, dtype=torch.int32, device=dev))
    assert_close_scaled(C, g.w4a16_gemm(A, q4, s, gs), what="marlin large tiles")


@pytest.mark.parametrize("M,N,K,gs", [(80, 192, 192, 64), (128, 4096, 4096, 128), (272, 1088, 8192, -1), (512, 320, 1024, 128),
                                      (96, 28672, 512, 128), (144, 64, 14336, 128), (256, 4160, 2048, 256),
                                      (48, 4096, 14336, 128), (64, 28672, 4096, 128)])
def test_mul_mid_m_fused_tiles(dev, M, N, K, gs):
    """64 < M <= 512, and 32 < M <= 64 with large weights: the tile kernels expand the Marlin units themselves
    (odd chunk counts, one or several K slices, group sizes from 64 to the whole column)."""
    announce("marlin fused tiles", M, N, K, gs)
    torch.manual_seed(M + N + K)
    A = (torch.randn(M, K) * 0.3).half()
    W = (torch.randn(K, N) * 0.05).half()
    _, q4, s = mr.fake_quantize(W, gs)
    B, sp = mr.pack(q4, s, K if gs == -1 else gs)
    C = torch.zeros(M, N, dtype=torch.half, device=dev)
    mul(A.to(dev), B.to(dev), C, sp.to(dev), torch.zeros(64, dtype=torch.int32, device=dev))
    assert_close_scaled(C, g.w4a16_gemm(A, q4, s, gs), what="marlin fused tiles")


@pytest.mark.parametrize("M,N,K,gs", [(65, 136, 128, 64), (128, 4096, 4096, 128), (200, 1000, 1152, 128), (256, 520, 8192, 256),
                                      (512, 264, 2048, 64), (100, 129, 14336, -1), (130, 4100, 4224, 128), (96, 28672, 1024, 128),
                                      (48, 4096, 14336, 128), (64, 28672, 4096, 128), (33, 2400, 14336, 256),
                                      # one round of 128-column tiles of the producer / consumer kernel: 64- and 128-row tiles,
                                      # ragged rows and columns, groups of 64 and of the whole row
                                      (130, 9000, 640, 64), (300, 5000, 1152, 128), (100, 16000, 256, -1), (128, 20000, 384, 64),
                                      (128, 14336, 4096, 128)])
def test_w4a16_nk_mid_m_fused_tiles(dev, M, N, K, gs):
    """64 < M <= 512, and 32 < M <= 64 with large weights: the tile kernels expand the packed words themselves
    (one or several K slices, ragged rows and columns, group sizes from 64 to the whole row)."""
    announce("w4a16 nk fused tiles", M, N, K, gs)
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).half()
    w = torch.randn(N, K) * 0.02
    grp = K if gs == -1 else gs
    qn, s = q.w4a16_quant_nk(w, grp)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    y = w4a16.w4a16_gemm(x.to(dev), torch.from_numpy(packed).to(dev), s.to(dev), gs)
    assert y.dtype == torch.half and y.shape == (M, N)
    ref = g.w4a16_gemm(x, qn.t().int().contiguous(), s.t().contiguous(), grp)
    assert_close_scaled(y, ref, what="w4a16 nk fused tiles")


@pytest.mark.parametrize("M,N,K,gs", [(2300, 14400, 384, 128), (4100, 8200, 128, 64), (2560, 14336, 256, 128),
                                      (600, 61000, 640, 64)])
def test_w4a16_nk_fused_256_column_tiles(dev, M, N, K, gs):
    """More than 512 rows and two or more rounds of 256 x 256 tiles: the packed words are expanded inside the
    256-column tile kernel (two, four, six and ten K steps of 64: from no steady-state step to eight; ragged rows
    and columns; groups of one K step and of two)."""
    announce("w4a16 nk fused 256-column tiles", M, N, K, gs)
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).half()
    w = torch.randn(N, K) * 0.02
    qn, s = q.w4a16_quant_nk(w, gs)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    y = w4a16.w4a16_gemm(x.to(dev), torch.from_numpy(packed).to(dev), s.to(dev), gs)
    assert y.dtype == torch.half and y.shape == (M, N)
    ref = g.w4a16_gemm(x, qn.t().int().contiguous(), s.t().contiguous(), gs)
    assert_close_scaled(y, ref, what="w4a16 nk fused 256-column tiles")


@pytest.mark.parametrize("M,N,K,gs", [(4096, 4096, 256, 128), (3990, 4100, 384, 64), (4096, 3848, 128, 32)])
def test_w4a16_nk_large_tile_shapes(dev, M, N, K, gs):
    announce("w4a16 nk large tiles", M, N, K, gs)
    torch.manual_seed(N + K)
    x = torch.randn(M, K).half()
    w = torch.randn(N, K) * 0.02
    qn, s = q.w4a16_quant_nk(w, gs)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    y = w4a16.w4a16_gemm(x.to(dev), torch.from_numpy(packed).to(dev), s.to(dev), gs)
    ref = g.w4a16_gemm(x, qn.t().int().contiguous(), s.t().contiguous(), gs)
    assert_close_scaled(y, ref, what="w4a16 nk large tiles")


@pytest.mark.parametrize("M,N,K", [(128, 1024, 4096), (48, 4096, 14336), (300, 520, 1152), (16, 264, 8320)])
def test_w4a16_without_scratch(dev, M, N, K):
    """The scratch of both w4a16 entry points is optional: without it the kernels run with one K slice (or the
    weight-streaming variant) and must agree with the oracle all the same."""
    announce("w4a16 without scratch", M, N, K)
    torch.manual_seed(M + N)
    x = torch.randn(M, K).half()
    qn, s = q.w4a16_quant_nk(torch.randn(N, K) * 0.02, 128)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    xd, pd, sd = x.to(dev), torch.from_numpy(packed).to(dev), s.to(dev)
    y = torch.empty(M, N, dtype=torch.half, device=dev)
    _lib.call("llmk_gemm_w4a16_nk", _lib.ptr(xd), _lib.ptr(pd), _lib.ptr(y), _lib.ptr(sd), _lib.dt(xd.dtype),
              M, N, K, 128, None, 0, _lib.stream(xd))
    assert_close_scaled(y, g.w4a16_gemm(x, qn.t().int().contiguous(), s.t().contiguous(), 128), what="nk without scratch")
    if M % 16 == 0 and N % 64 == 0:
        A = (torch.randn(M, K) * 0.3).half()
        W = (torch.randn(K, N) * 0.05).half()
        _, q4, sm = mr.fake_quantize(W, 128)
        B, sp = mr.pack(q4, sm, 128)
        Ad, Bd, spd = A.to(dev), B.to(dev), sp.to(dev)
        C = torch.zeros(M, N, dtype=torch.half, device=dev)
        _lib.call("llmk_gemm_w4a16_marlin", _lib.ptr(Ad), _lib.ptr(Bd), _lib.ptr(C), _lib.ptr(spd),
                  M, N, K, 128, None, 0, _lib.stream(Ad))
        assert_close_scaled(C, g.w4a16_gemm(A, q4, sm, 128), what="marlin without scratch")


@pytest.mark.parametrize("M,N,K,gs", [(16, 4096, 4096, 128), (1, 256, 512, 128), (7, 1000, 1024, 128), (40, 520, 2048, 128),
                                      (16, 28672, 4096, 128), (16, 1032, 14336, 128), (64, 264, 8192, 128),
                                      (16, 256, 384, 128), (33, 300, 4608, 128), (16, 512, 1024, 64), (20, 129, 512, 256),
                                      (300, 1000, 512, 128), (2048, 4096, 1024, 128),
                                      # K > 4096 with M * N not a multiple of 4: the ring kernel's summing pass does not take it
                                      (1, 1001, 8192, 128), (3, 50257, 8192, 128)])
def test_w4a16_nk_bf16(dev, M, N, K, gs):
    """bf16 activations / outputs for the [N, K/8] layout: the weight-streaming kernel at decode sizes (128-wide
    groups, whole four-step K shares), the bf16 copy of W plus the bf16 tile GEMM everywhere else."""
    announce("w4a16 nk bf16", M, N, K, gs)
    torch.manual_seed(2)
    x = torch.randn(M, K).bfloat16()
    w = torch.randn(N, K) * 0.02
    qn, s = q.w4a16_quant_nk(w, gs)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    y = w4a16.w4a16_gemm(x.to(dev), torch.from_numpy(packed).to(dev), s.to(dev), gs)
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    deq = (qn.double() - 8) * s.double().repeat_interleave(gs, 1)            # [N, K], exact
    assert_close_scaled(y, x.double() @ deq.T, what="w4a16 nk bf16")


def test_w4a16_nk_bf16_decode_is_exact_for_small_integers(dev):
    """Integer activations, unit scales: the bf16 decode kernel (nibbles as 128 + q, the -136 * sum(a) bias in the
    accumulator) returns the exact integer product wherever it is representable in bf16."""
    announce("w4a16 nk bf16 exact")
    torch.manual_seed(3)
    M, N, K = 16, 512, 1024
    x = torch.randint(-2, 3, (M, K)).float()
    qn = torch.randint(0, 16, (N, K), dtype=torch.uint8)
    s = torch.ones(N, K // 128, dtype=torch.float16)
    packed, _ = bp.pack_cols(qn.numpy(), 4, 32)
    y = w4a16.w4a16_gemm(x.bfloat16().to(dev), torch.from_numpy(packed).to(dev), s.to(dev), 128)
    ref = x.double() @ (qn.double() - 8).T
    assert torch.equal(y.cpu().double(), ref.bfloat16().double())
