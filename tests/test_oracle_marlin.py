"""Pins oracle/marlin_ref.py and the product's QuantUtils (pure torch host code) on CPU."""
import numpy as np
import pytest
import torch

from oracle import marlin_ref as mr, gemm_ref
from llm_kernels_amd.fast_dequant.simple_marlin.utils import QuantUtils


def test_weight_perm_is_bijection_with_fragment_coordinates():
    perm = mr.weight_perm()
    assert sorted(perm.tolist()) == list(range(1024))
    # lane i, sub-tile j, nibble t: (t & 1) selects k+8, ((t >> 1) & 1) the column block, (t >> 2) the odd k
    for i in (0, 5, 31):
        for j in range(4):
            for t in range(8):
                src = int(perm[32 * i + 8 * j + t])
                tile, row, col = src // 256, (src % 256) // 16, src % 16
                assert tile == j
                assert row == 2 * (i % 4) + (t >> 2) + 8 * (t & 1)
                assert col == i // 4 + 8 * ((t >> 1) & 1)


def test_scale_perm():
    sp = mr.scale_perm(True)
    assert sorted(sp.tolist()) == list(range(64))
    assert sp[8 * 3 + 5] == 3 + 8 * 5
    sps = mr.scale_perm(False)
    assert sorted(sps.tolist()) == list(range(32)) and sps[:8].tolist() == [0, 1, 8, 9, 16, 17, 24, 25]


@pytest.mark.parametrize("K,N,g", [(16, 64, 16), (128, 128, 128), (64, 192, 32)])
def test_pack_matches_kernel_emulation(K, N, g):
    """pack() -> walk the words the way the reference CUDA kernel consumes them -> original q and scales."""
    torch.manual_seed(K + N)
    q = torch.randint(0, 16, (K, N), dtype=torch.int32)
    s = torch.randn(K // g, N).half()
    B, sp = mr.pack(q, s, g)
    assert B.shape == (K // 16, 2 * N) and B.dtype == torch.int32 and sp.shape == s.shape
    q2, s2 = mr.emulate_unpack(B, sp, K, N, g)
    assert torch.equal(q2, q)
    assert torch.equal(s2, s)


def test_pack_tiny_hand_case():
    # K=16, N=64, all zero except q[k=1, n=8] = 0xA: lane i = 4*c + k0/2 with c = 0 (col 8 = block 1), k0 = 0
    q = torch.zeros(16, 64, dtype=torch.int32)
    q[1, 8] = 0xA
    B, _ = mr.pack(q, torch.ones(1, 64).half(), 16)
    words = B.numpy().view(np.uint32).reshape(32, 4)
    assert np.count_nonzero(words) == 1
    # odd k (k0 + 1) of column block 1 sits at bits 27:24 of word j = 0 of lane 0
    assert words[0, 0] == 0xA << 24


def test_product_quantutils_equals_oracle():
    torch.manual_seed(7)
    for K, N, g in [(128, 64, 128), (256, 128, 64), (64, 64, -1)]:
        w = (torch.randn(K, N) * 0.1).half()
        ref, q, s = QuantUtils.fake_quantize(w, g)
        oref, oq, os_ = mr.fake_quantize(w, g)
        assert torch.equal(ref, oref) and torch.equal(q, oq) and torch.equal(s, os_)
        B, sp = QuantUtils.pack(q, s, g)
        oB, osp = mr.pack(q, s, g)
        assert B.dtype == torch.int32 and torch.equal(B, oB) and torch.equal(sp, osp)


def test_fake_quantize_properties():
    torch.manual_seed(8)
    w = (torch.randn(256, 64) * 0.1).half()
    ref, q, s = mr.fake_quantize(w, 128)
    assert q.dtype == torch.int32 and q.min() >= 0 and q.max() <= 15 and s.shape == (2, 64)
    amax = w.reshape(2, 128, 64).abs().amax(1)
    assert torch.equal(s, amax * (2 / 15))
    assert torch.equal(ref, gemm_ref.w4a16_dequant_kn(q, s, 128))
    assert ((ref.float() - w.float()).abs() <= s.float().repeat_interleave(128, 0) * 0.5 * 1.01 + 1e-3).all()
    # a value exactly at +absmax maps to 7.5 -> rne 8 -> +8 = 16 -> clamped to 15
    w2 = torch.zeros(16, 64).half(); w2[0, 0] = 1.5; w2[1, 0] = -1.5
    _, q2, s2 = mr.fake_quantize(w2, 16)
    assert q2[0, 0] == 15 and q2[1, 0] == 0 and s2[0, 0] == torch.tensor(1.5).half() * (2 / 15)
