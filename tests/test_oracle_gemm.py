"""Pins oracle/gemm_ref.py and oracle/moe_ref.py (CPU)."""
import torch

from oracle import gemm_ref as g, quant_ref as q, moe_ref as m


def _fp8_case(M=5, N=130, K=256, seed=0):
    torch.manual_seed(seed)
    a, a_s = q.act_quant_fp8(torch.randn(M, K).bfloat16())
    b, b_s = q.weight_quant_fp8(torch.randn(N, K) * 0.02)
    return a, a_s, b, b_s


def test_blockwise_equals_dequant_then_matmul_fp8():
    a, a_s, b, b_s = _fp8_case()
    c1 = g.gemm_blockwise(a, a_s, b, b_s)
    c2 = g.gemm_dequant(a, a_s, b, b_s)
    assert c1.shape == (5, 130)
    assert torch.allclose(c1, c2, rtol=1e-12, atol=1e-12)


def test_blockwise_equals_dequant_then_matmul_int8_and_brute():
    torch.manual_seed(1)
    a, a_s = q.act_quant_int8(torch.randn(4, 256))
    b, b_s = q.weight_quant_int8(torch.randn(9, 256) * 0.02)
    c1 = g.gemm_blockwise(a, a_s, b, b_s)
    assert torch.allclose(c1, g.gemm_dequant(a, a_s, b, b_s), rtol=1e-12, atol=1e-12)
    assert torch.allclose(c1, g.brute_gemm_blockwise(a, a_s, b, b_s), rtol=1e-12, atol=1e-12)
    # close to the unquantised product (what the reference's own test prints as cosine similarity)
    ref = (torch.randn(1), )  # placeholder to keep the seed stream independent
    del ref


def test_unit_scales_reduce_to_integer_matmul():
    torch.manual_seed(2)
    a = torch.randint(-127, 128, (3, 384), dtype=torch.int8)
    b = torch.randint(-127, 128, (7, 384), dtype=torch.int8)
    ones_a, ones_b = torch.ones(3, 3), torch.ones(1, 3)
    c = g.gemm_blockwise(a, ones_a, b, ones_b)
    exact = a.long() @ b.long().T
    assert torch.equal(c.long(), exact) and torch.equal(g.int8_gemm_int32(a, b).long(), exact)
    d = g.block_dots(a, b)
    assert d.shape == (3, 3, 7) and torch.equal(d[1].long(), a[:, 128:256].long() @ b[:, 128:256].long().T)


def test_identity_activation_returns_dequantised_weight_rows():
    torch.manual_seed(3)
    b, b_s = q.weight_quant_int8(torch.randn(6, 128) * 0.02)
    a = torch.zeros(2, 128, dtype=torch.int8); a[0, 5] = 1; a[1, 77] = 1
    c = g.gemm_blockwise(a, torch.ones(2, 1), b, b_s)
    wd = q.weight_dequant_block(b, b_s).double()
    assert torch.allclose(c[0], wd[:, 5]) and torch.allclose(c[1], wd[:, 77])


def test_w4a8_gemm_equals_dequant_form():
    torch.manual_seed(4)
    qq, s, s4, z4 = q.w4a8_weight_quant_levels(torch.randn(128, 256) * 0.02)
    a, a_s = q.act_quant_int8(torch.randn(3, 256), rounding="up")
    c = g.w4a8_gemm(a, a_s, qq, s, s4, z4)
    wd = q.w4a8_weight_dequant(qq, s, s4, z4).double()
    ad = a.double() * a_s.double().repeat_interleave(128, 1)
    # weight_dequant rounds (int8 * s) to fp16: agreement to fp16 precision
    assert torch.allclose(c, ad @ wd.T, rtol=2e-3, atol=1e-3)
    exact_w = q.w4a8_dequant_int8(qq, s4, z4).double() * s.double().repeat_interleave(128, 0).repeat_interleave(128, 1)
    assert torch.allclose(c, ad @ exact_w.T, rtol=1e-12, atol=1e-12)


def test_w4a16_gemm_tiny_brute():
    torch.manual_seed(5)
    K, N, M = 32, 16, 2
    qn = torch.randint(0, 16, (K, N), dtype=torch.int32)
    s = (torch.rand(2, N) * 0.1).half()
    a = torch.randn(M, K).half()
    c = g.w4a16_gemm(a, qn, s, 16)
    for mm, nn in [(0, 0), (1, 15)]:
        tot = sum(float(a[mm, k]) * float(((qn[k, nn] - 8).half() * s[k // 16, nn])) for k in range(K))
        assert abs(c[mm, nn].item() - tot) < 1e-9


def test_moe_worked_example_from_reference_comment():
    # moe/group_gemm_kernel.py:65-74: 6 tokens, top-2, 4 experts
    topk_ids = torch.tensor([[0, 2], [1, 3], [0, 1], [2, 3], [1, 2], [0, 3]])
    rids, src2dst, seg = m.run_moe_ep_preprocess(topk_ids, 4)
    assert src2dst.tolist() == [0, 6, 3, 9, 1, 4, 7, 10, 5, 8, 2, 11]
    assert rids.tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2, 3, 3, 3]
    assert seg.tolist() == [0, 3, 6, 9, 12] and seg.dtype == torch.int64 and src2dst.dtype == torch.int32


def test_moe_permute_roundtrip_and_dense_equivalence():
    torch.manual_seed(6)
    T, H, I, E, topk = 24, 128, 128, 4, 2
    x = torch.randn(T, H)
    ids, w = m.softmax_top2_router(torch.randn(T, E), topk)
    assert torch.allclose(w.sum(1), torch.ones(T))
    rids, s2d, seg = m.run_moe_ep_preprocess(ids, E)
    gin = m.pre_reorder(x, s2d, ids, None, 0, E - 1, topk)
    for t in range(T):
        for j in range(topk):
            assert torch.equal(gin[s2d[t * topk + j]], x[t])
            assert rids[s2d[t * topk + j]] == ids[t, j]
    # post_reorder of the permuted input with weights summing to 1 gives the input back
    back = m.post_reorder(gin, s2d, ids, w, 0, E - 1, topk)
    assert torch.allclose(back, x, atol=1e-6)
    # unquantised grouped path == dense per-expert loop
    w13 = torch.randn(E, 2 * I, H) * 0.05
    w2 = torch.randn(E, H, I) * 0.05
    widx = torch.arange(E)
    gu = m.grouped_gemm(gin, w13, seg, widx).float()
    di, mask = m.silu_and_mul(gu, rids, None, 0, E - 1)
    assert mask.all()
    do = m.grouped_gemm(di, w2, seg, widx).float()
    out = m.post_reorder(do, s2d, ids, w, 0, E - 1, topk)
    dense = m.dense_moe_forward(x, ids, w, w13, w2)
    assert torch.allclose(out.double(), dense, rtol=1e-4, atol=1e-5)


def test_silu_rounding_points_bf16():
    gu = torch.tensor([[1.0, -2.0, 3.0, 0.5]]).bfloat16()
    out, _ = m.silu_and_mul(gu, torch.tensor([0]), None, 0, 0)
    g32 = gu[:, :2].float()
    exp = ((g32 * torch.sigmoid(g32)).bfloat16() * gu[:, 2:])
    assert torch.equal(out, exp)


def test_gelu_branch_equals_torch_tanh_gelu():
    """moe_ref.silu_and_mul(act='gelu') restates group_gemm_kernel.py:214-228; in fp32 (no rounding points)
    it must be torch's tanh-approximated GELU times up."""
    torch.manual_seed(8)
    g32 = torch.cat([torch.randn(7, 64) * 3, torch.tensor([[0.0, 1.0, -1.0, 10.0, -10.0, 0.5, -0.5, 25.0] * 8])])
    up = torch.randn(8, 64)
    out, mask = m.silu_and_mul(torch.cat([g32, up], 1), torch.zeros(8, dtype=torch.long), None, 0, 0, act="gelu")
    assert mask.all()
    want = torch.nn.functional.gelu(g32.double(), approximate="tanh") * up.double()
    assert torch.allclose(out.double(), want, rtol=2e-6, atol=2e-7)
    # known values: gelu(0) = 0, gelu(x) -> x for large x, -> 0 for very negative x
    one = torch.ones(1, 3)
    o2, _ = m.silu_and_mul(torch.cat([torch.tensor([[0.0, 25.0, -25.0]]), one], 1), torch.tensor([0]), None, 0, 0,
                           act="gelu")
    assert o2.tolist() == [[0.0, 25.0, 0.0]] or o2.abs().tolist() == [[0.0, 25.0, 0.0]]


def test_pre_reorder_scale_branch_hand_rows():
    """group_gemm_kernel.py:100-115: row * (1 / a1_scales[e - start]) for local experts only."""
    x = torch.tensor([[2.0, 4.0, -8.0, 1.0], [3.0, 6.0, 9.0, -12.0]])
    topk_ids = torch.tensor([[1, 2], [3, 1]])            # experts 1..2 are local, 3 is not
    src2dst = torch.tensor([0, 2, 3, 1], dtype=torch.int32)
    a1 = torch.tensor([2.0, 4.0])                        # scales of experts 1 and 2
    out = m.pre_reorder(x, src2dst, topk_ids, a1, 1, 2, 2)
    assert out[0].tolist() == [1.0, 2.0, -4.0, 0.5]      # token 0 -> expert 1: / 2
    assert out[2].tolist() == [0.5, 1.0, -2.0, 0.25]     # token 0 -> expert 2: / 4
    assert out[1].tolist() == [1.5, 3.0, 4.5, -6.0]      # token 1 -> expert 1: / 2
    assert out[3].tolist() == [0.0, 0.0, 0.0, 0.0]       # token 1 -> expert 3: not local, row untouched
    # rounding point: the product is formed in fp32 and cast once to the output dtype
    xb = torch.tensor([[1.0078125, 3.0]]).bfloat16()
    ob = m.pre_reorder(xb, torch.tensor([0], dtype=torch.int32), torch.tensor([[0]]), torch.tensor([3.0]), 0, 0, 1)
    assert torch.equal(ob, (xb.float() * (1.0 / 3.0)).bfloat16())


def test_silu_and_mul_scale_branch_hand_rows():
    """group_gemm_kernel.py:145-166: (1 / scale[e - start]) is cast to the tensor dtype first, then
    silu(gate) (cast) * up (rounded) * scale (rounded)."""
    # silu(20) = 20 in fp32 to 8 digits; up = 3; expert 2 -> 1/4, expert 1 -> 1/2
    gu = torch.tensor([[20.0, 3.0], [20.0, 3.0], [20.0, 3.0]]).bfloat16()
    rids = torch.tensor([1, 2, 3])
    out, mask = m.silu_and_mul(gu, rids, torch.tensor([2.0, 4.0]), 1, 2)
    assert mask.tolist() == [True, True, False]
    assert out.flatten().tolist() == [30.0, 15.0, 0.0]
    # 1/3 is rounded to bf16 before the multiplication (not applied as an fp32 factor)
    gu2 = torch.tensor([[20.0, 1.0]]).bfloat16()
    o2, _ = m.silu_and_mul(gu2, torch.tensor([0]), torch.tensor([3.0]), 0, 0)
    third = torch.tensor(1.0 / 3.0).bfloat16()
    assert o2.item() == (torch.tensor(20.0).bfloat16() * third).item() != torch.tensor(20.0 / 3.0).bfloat16().item()
