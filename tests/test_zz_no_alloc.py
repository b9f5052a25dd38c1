"""llmk_gemm_fp8_block_static: the fp8 block GEMM whose scratch is a device array inside the library.

Checked through the C ABI against llmk_gemm_fp8_block (caller-provided workspace) bit for bit, on calls in a
row that share the built-in array, the later ones smaller than the first.
"""
import pytest
import torch

from oracle import gemm_ref as g
from llm_kernels_amd import _lib
from llm_kernels_amd.quantization import fp8_kernel
from helpers import announce, assert_close_scaled

pytestmark = pytest.mark.gpu


def _both(dev, M, N, K, seed, out=torch.bfloat16):
    torch.manual_seed(seed)
    a, a_s = fp8_kernel.act_quant(torch.randn(M, K, device=dev).bfloat16())
    b, b_s = fp8_kernel.weight_quant(torch.randn(N, K, device=dev) * 0.02)
    st = _lib.stream(a)
    need = _lib.load().llmk_gemm_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    c_ref = torch.empty(M, N, dtype=out, device=dev)
    _lib.call("llmk_gemm_fp8_block", _lib.ptr(a), _lib.ptr(a_s), _lib.ptr(b), _lib.ptr(b_s), _lib.ptr(c_ref),
              _lib.dt(out), M, N, K, _lib.ptr(ws), need, st)
    c = torch.full((M, N), float("nan"), dtype=out, device=dev)
    _lib.call("llmk_gemm_fp8_block_static", _lib.ptr(a), _lib.ptr(a_s), _lib.ptr(b), _lib.ptr(b_s), _lib.ptr(c),
              _lib.dt(out), M, N, K, st)
    torch.cuda.synchronize()
    return c, c_ref, need, (a, a_s, b, b_s)


def test_static_scratch_matches_workspace_entry_on_consecutive_calls(dev):
    # K ranges (4 planes of partial sums), then a smaller K-range call, then split-K tiles, then a shape that
    # needs no scratch at all, then the first shape again
    shapes = [(16, 4096, 14336), (8, 1024, 8192), (128, 2048, 4096), (16, 4096, 4096), (16, 4096, 14336)]
    used = []
    for i, (M, N, K) in enumerate(shapes):
        announce("fp8 static scratch", M, N, K)
        c, c_ref, need, ops = _both(dev, M, N, K, 100 + i)
        used.append(need)
        assert torch.equal(c.view(torch.int16), c_ref.view(torch.int16)), (M, N, K)
        if i < 2:
            a, a_s, b, b_s = (t.cpu() for t in ops)
            assert_close_scaled(c, g.gemm_blockwise(a, a_s, b, b_s), what="fp8 static %dx%dx%d" % (M, N, K))
    assert used[0] > used[1] > 0 and used[2] > 0 and used[3] == 0


def test_static_scratch_large_m_long_k_within_tolerance(dev):
    """M > 512 with K >= 8192: the workspace entry may split its last round of tiles along K (64 MiB of partial
    sums that the built-in array does not hold), so the two entries may differ in fp32 summation order: both are
    held to the oracle's tolerance, and to each other's within twice that."""
    M, N, K = 1100, 1300, 8192
    announce("fp8 static scratch, large M", M, N, K)
    c, c_ref, need, ops = _both(dev, M, N, K, 7)
    assert need > 64 << 20
    a, a_s, b, b_s = (t.cpu() for t in ops)
    ref = g.gemm_blockwise(a, a_s, b, b_s)
    assert_close_scaled(c, ref, what="fp8 static %dx%dx%d" % (M, N, K))
    assert_close_scaled(c_ref, ref, what="fp8 workspace %dx%dx%d" % (M, N, K))
    assert_close_scaled(c, c_ref.double(), rtol=2e-2, atol=2e-2, what="static vs workspace entry")


def test_static_scratch_rejects_oversized_shapes(dev):
    M, N, K = 16, 128256, 20480
    assert _lib.load().llmk_gemm_workspace_bytes(M, N, K) > 32 << 20
    x = torch.zeros(16, device=dev)
    with pytest.raises(_lib.LlmkError, match="built-in"):
        _lib.call("llmk_gemm_fp8_block_static", _lib.ptr(x), _lib.ptr(x), _lib.ptr(x), _lib.ptr(x), _lib.ptr(x),
                  _lib.BF16, M, N, K, _lib.stream(x))
