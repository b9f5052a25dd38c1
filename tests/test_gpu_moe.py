"""Single-GPU EP-MoE path vs the torch-CPU oracle."""
import pytest
import torch

from oracle import moe_ref as m, quant_ref as q, gemm_ref as g
from llm_kernels_amd.moe import group_gemm_kernel as gk
from llm_kernels_amd.moe.ep_moe import ep_moe_forward, softmax_topk_router, EPMoE
from llm_kernels_amd.moe.config import Config
from llm_kernels_amd.quantization import int8_kernel, fp8_kernel
from helpers import announce, assert_close_scaled

pytestmark = pytest.mark.gpu


def test_preprocess_worked_example(dev):
    announce("moe preprocess example")
    topk_ids = torch.tensor([[0, 2], [1, 3], [0, 1], [2, 3], [1, 2], [0, 3]], device=dev)
    rids, src2dst, seg = gk.run_moe_ep_preproess(topk_ids, 4)
    assert src2dst.tolist() == [0, 6, 3, 9, 1, 4, 7, 10, 5, 8, 2, 11]
    assert rids.tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2, 3, 3, 3]
    assert seg.tolist() == [0, 3, 6, 9, 12] and seg.dtype == torch.int64 and src2dst.dtype == torch.int32


@pytest.mark.parametrize("T,E,topk", [(4096, 8, 2), (37, 16, 4), (1, 4, 2), (64, 8, 1)])
def test_preprocess_random_incl_empty_experts(dev, T, E, topk):
    announce("moe preprocess", T, E, topk)
    torch.manual_seed(T)
    logits = torch.randn(T, E)
    logits[:, E - 1] = -1e9                                     # last expert never chosen -> empty segment
    ids = torch.topk(logits, topk, dim=-1)[1]
    rids, s2d, seg = gk.run_moe_ep_preproess(ids.to(dev), E)
    orids, os2d, oseg = m.run_moe_ep_preprocess(ids, E)
    assert torch.equal(rids.cpu(), orids) and torch.equal(s2d.cpu(), os2d) and torch.equal(seg.cpu(), oseg)
    assert seg[-1].item() == T * topk and seg[E].item() == seg[E - 1].item()


@pytest.mark.parametrize("n,E,dtype", [(8192, 8, torch.int64), (32768, 512, torch.int32), (1025, 256, torch.int64),
                                       (1023, 3, torch.int32), (64, 160, torch.int64), (5000, 1, torch.int64),
                                       (0, 8, torch.int64)])
def test_preprocess_one_launch_equals_sort(dev, n, E, dtype):
    """The one-workgroup counting sort returns what the stable sort + segment pointers + map return: many
    rounds, every wave holding many distinct ids (E = 512), a single bucket, ragged last round, no ids."""
    announce("moe preprocess one launch", n, E, dtype)
    torch.manual_seed(n + E)
    ids = torch.randint(0, E, (n,), dtype=dtype)
    if n > 100:
        ids[n // 3: n // 3 + 70] = E - 1                        # a run longer than a wave of one id
    rids, s2d, seg = gk.run_moe_ep_preproess(ids.to(dev), E)
    orids, order = torch.sort(ids, stable=True)
    os2d = torch.empty(n, dtype=torch.int32)
    os2d[order] = torch.arange(n, dtype=torch.int32)
    oseg = torch.zeros(E + 1, dtype=torch.int64)
    oseg[1:] = torch.cumsum(torch.bincount(ids.long(), minlength=E), 0)
    assert rids.dtype == dtype and torch.equal(rids.cpu(), orids)
    assert torch.equal(s2d.cpu(), os2d) and torch.equal(seg.cpu(), oseg)


def test_preprocess_ids_outside_the_expert_range(dev):
    """Ids below 0 or at / above num_experts (padding conventions of some routers): the launch must stay inside
    its tables and still return a permutation whose in-range part is the stable sort; negative ids lead,
    too-large ids trail, and seg_indptr[e + 1] counts the ids <= e as the reference's binary search does."""
    announce("moe preprocess out-of-range ids")
    n, E = 3000, 8
    torch.manual_seed(9)
    ids = torch.randint(0, E, (n,))
    ids[::17] = -1
    ids[5::29] = E + 3
    ids[7::31] = E
    rids, s2d, seg = gk.run_moe_ep_preproess(ids.to(dev), E)
    rids, s2d, seg = rids.cpu(), s2d.cpu().long(), seg.cpu()
    assert sorted(s2d.tolist()) == list(range(n))                   # a permutation
    assert torch.equal(rids[s2d], ids)                               # every id sits where src2dst says
    neg, big = int((ids < 0).sum()), int((ids >= E).sum())
    assert (rids[:neg] < 0).all() and (rids[n - big:] >= E).all()
    mid = rids[neg:n - big]
    assert torch.equal(mid, torch.sort(ids[(ids >= 0) & (ids < E)], stable=True)[0])
    inr = torch.nonzero((ids >= 0) & (ids < E)).flatten()            # stable: equal ids keep their order
    for e in range(E):
        pos = s2d[inr[ids[inr] == e]]
        assert (pos[1:] > pos[:-1]).all()
    assert seg.tolist() == [0] + [int((ids <= e).sum()) for e in range(E)]


def test_preprocess_beyond_one_workgroup(dev):
    """More ids than the one-launch sort takes: the wrapper goes through torch.sort, the entry point refuses."""
    announce("moe preprocess large")
    from llm_kernels_amd import _lib
    n, E = gk.PREPROCESS_MAX_IDS + 5, 8
    torch.manual_seed(3)
    ids = torch.randint(0, E, (n,))
    rids, s2d, seg = gk.run_moe_ep_preproess(ids.to(dev), E)
    orids, os2d, oseg = m.run_moe_ep_preprocess(ids, E)
    assert torch.equal(rids.cpu(), orids) and torch.equal(s2d.cpu(), os2d) and torch.equal(seg.cpu(), oseg)
    d = ids.to(dev)
    with pytest.raises(RuntimeError, match="exceed the limits"):
        _lib.call("llmk_moe_ep_preprocess", _lib.ptr(d), 8, n, E, _lib.ptr(rids), _lib.ptr(s2d), _lib.ptr(seg), None)
    with pytest.raises(RuntimeError, match="exceed the limits"):
        _lib.call("llmk_moe_ep_preprocess", _lib.ptr(d), 8, 16, gk.PREPROCESS_MAX_EXPERTS + 1, _lib.ptr(rids),
                  _lib.ptr(s2d), _lib.ptr(seg), None)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_reorder_and_activation_kernels(dev, dtype):
    announce("moe aux", dtype)
    torch.manual_seed(1)
    T, H, I, E, topk = 50, 384, 256, 8, 2
    x = torch.randn(T, H).to(dtype)
    ids, w = m.softmax_top2_router(torch.randn(T, E), topk)
    rids, s2d, seg = m.run_moe_ep_preprocess(ids, E)
    # local experts 2..5 only: other destination rows stay untouched
    gin = torch.full((T * topk, H), -3.0, dtype=dtype, device=dev)
    gk.pre_reorder_triton_kernel[(T,)](x.to(dev), gin, s2d.to(dev), ids.to(dev), None, 2, 5, topk, H, BLOCK_SIZE=512)
    ogin = m.pre_reorder(x, s2d, ids, None, 2, 5, topk, out=torch.full((T * topk, H), -3.0, dtype=dtype))
    assert torch.equal(gin.cpu(), ogin)
    # the copy keeps the sign of a zero (compared as bit patterns)
    xz = x.clone()
    xz[:, ::3] = -0.0
    ginz = torch.zeros((T * topk, H), dtype=dtype, device=dev)
    gk.pre_reorder(xz.to(dev), ginz, s2d.to(dev), ids.to(dev), None, 0, E - 1, topk, H)
    oginz = m.pre_reorder(xz, s2d, ids, None, 0, E - 1, topk)
    as_bits = lambda t: t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)
    assert torch.equal(as_bits(ginz.cpu()), as_bits(oginz))
    a1 = torch.rand(4) + 0.5
    gin2 = torch.zeros((T * topk, H), dtype=dtype, device=dev)
    gk.pre_reorder(x.to(dev), gin2, s2d.to(dev), ids.to(dev), a1.to(dev), 2, 5, topk, H)
    assert_close_scaled(gin2, m.pre_reorder(x, s2d, ids, a1, 2, 5, topk), rtol=4e-3, atol=1e-6)

    gu = torch.randn(T * topk, 2 * I).to(dtype)
    for act, fn in (("silu", gk.silu_and_mul_triton_kernel), ("gelu", gk.gelu_and_mul_triton_kernel)):
        di = torch.zeros(T * topk, I, dtype=dtype, device=dev)
        fn[(T * topk,)](gu.to(dev), di, 2 * I, rids.to(dev), None, 0, E - 1, BLOCK_SIZE=512)
        odi, _ = m.silu_and_mul(gu, rids, None, 0, E - 1, act=act)
        # sigmoid differs by an ulp between libraries; after rounding to the tensor dtype at most one step
        assert_close_scaled(di, odi, rtol=2 ** -7 if dtype == torch.bfloat16 else 2e-3, atol=1e-5, what=act)
        if dtype != torch.float32:      # in fp32 the libraries' exp differs in the last place
            exact = (di.cpu() == odi).float().mean().item()
            assert exact > 0.97, exact

    do = torch.randn(T * topk, H).to(dtype)
    out = torch.empty(T, H, dtype=dtype, device=dev)
    gk.post_reorder_triton_kernel[(T,)](do.to(dev), out, s2d.to(dev), ids.to(dev), w.to(dev), 0, E - 1, topk, H,
                                        BLOCK_SIZE=512)
    ref_out = m.post_reorder(do, s2d, ids, w, 0, E - 1, topk)
    if dtype == torch.float32:          # fp32: the device may contract v*w + sum into one fma
        assert torch.allclose(out.cpu(), ref_out, rtol=1e-6, atol=1e-6)
    else:                               # 16-bit types: every rounding point is explicit -> bit exact
        assert torch.equal(out.cpu(), ref_out)
    out2 = torch.full((T, H), 9.0, dtype=dtype, device=dev)
    gk.post_reorder(do.to(dev), out2, s2d.to(dev), ids.to(dev), w.to(dev), 2, 5, topk, H)
    assert torch.allclose(out2.cpu().float(), m.post_reorder(do, s2d, ids, w, 2, 5, topk).float(), rtol=1e-6, atol=1e-6)


def _segments(T, E, topk, seed, empty_last=True):
    torch.manual_seed(seed)
    logits = torch.randn(T, E)
    if empty_last:
        logits[:, E - 1] = -1e9
    ids, w = m.softmax_top2_router(logits, topk)
    return ids, w, m.run_moe_ep_preprocess(ids, E)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("I", [100, 2056, 4096 + 8])
def test_activation_kernel_row_lengths(dev, dtype, I):
    """Row lengths on both forms of the activation kernel (8 outputs per thread when I % 8 == 0, single elements
    otherwise; 2056 = 257 passes of 8 ends on an odd pass), per-expert scales, a local expert range."""
    announce("moe activation rows", dtype, I)
    torch.manual_seed(5)
    E, rows = 6, 37
    rids = torch.sort(torch.randint(0, E, (rows,), dtype=torch.int64))[0]
    gu = torch.randn(rows, 2 * I).to(dtype)
    sc = torch.rand(4) + 0.5
    for act, fn in (("silu", gk.silu_and_mul), ("gelu", gk.gelu_and_mul)):
        di = torch.full((rows, I), -3.0, dtype=dtype, device=dev)
        fn(gu.to(dev), di, 2 * I, rids.to(dev), sc.to(dev), 1, 4)
        odi, mask = m.silu_and_mul(gu, rids, sc, 1, 4, act=act)
        assert 0 < mask.sum() < rows
        assert_close_scaled(di.cpu()[mask], odi[mask], rtol=2 ** -6 if dtype == torch.bfloat16 else 4e-3, atol=1e-5,
                            what=act)
        assert torch.all(di.cpu()[~mask] == -3.0)                 # rows of other ranks' experts stay untouched


@pytest.mark.parametrize("kind", ["int8", "fp8", "fp16", "bf16"])
@pytest.mark.parametrize("T,E,N,K", [(40, 4, 256, 256), (300, 8, 200, 512), (9, 8, 128, 128)])
def test_grouped_gemm(dev, kind, T, E, N, K):
    announce("grouped_gemm", kind, T, E, N, K)
    topk = 2
    ids, w, (rids, s2d, seg) = _segments(T, E, topk, T + N)
    M = T * topk
    torch.manual_seed(3)
    a = torch.randn(M, K)
    wts = torch.randn(E, N, K) * 0.05
    widx = torch.arange(E)
    out_dt = torch.bfloat16 if kind != "fp16" else torch.float16
    c = torch.full((M, N), 5.0, dtype=out_dt, device=dev)
    if kind in ("int8", "fp8"):
        wq = q.weight_quant_int8 if kind == "int8" else q.weight_quant_fp8
        aq = q.act_quant_int8 if kind == "int8" else q.act_quant_fp8
        qs = [wq(wts[e]) for e in range(E)]
        b = torch.stack([x[0].view(torch.uint8) if kind == "fp8" else x[0] for x in qs])
        if kind == "fp8":
            b = b.view(torch.float8_e4m3fn)
        b_s = torch.stack([x[1] for x in qs])
        a_in = a.to(out_dt)
        ret = gk.grouped_gemm_triton(a_in.to(dev), b.to(dev), c, E, True, seg.to(dev), widx.to(dev), False, None,
                                     b_s.to(dev), [128, 128])
        a_q, a_s = aq(a_in)
        ref = m.grouped_gemm(a_q, b, seg, widx, a_s, b_s)
    else:
        dt = torch.float16 if kind == "fp16" else torch.bfloat16
        a_in, b = a.to(dt), wts.to(dt)
        ret = gk.grouped_gemm_triton(a_in.to(dev), b.to(dev), c, E, True, seg.to(dev), widx.to(dev))
        ref = m.grouped_gemm(a_in, b, seg, widx)
    assert ret is c
    assert_close_scaled(c, ref, what="grouped " + kind)


@pytest.mark.parametrize("M,N,K", [(8192, 2048, 256), (8192, 2304, 384), (8192, 3840, 256), (4096, 2048, 384)])
def test_grouped_gemm_large_tiles_exact(dev, M, N, K):
    """Shapes that the dispatch gives to the 256- and 128-row tiles of the large grouped kernel, with a number
    of column tiles that is and is not a multiple of the XCD count (the tile order differs), segments of very
    different length (one empty, one shorter than a tile, ragged ends) and permuted weight indices.  int8 with
    unit scales and small integers: every output must be the exact integer product; rows behind the last
    segment keep their fill value."""
    announce("grouped large tiles", M, N, K)
    E = 4
    torch.manual_seed(M + N)
    used = M - 7                                                # the last 7 rows belong to no segment
    seg = torch.tensor([0, 3000 if M > 4096 else 1300, 3000 if M > 4096 else 1300, 3041 if M > 4096 else 1341, used])
    widx = torch.tensor([2, 0, 3, 1])
    a = torch.randint(-15, 16, (M, K), dtype=torch.int8)
    b = torch.randint(-15, 16, (E, N, K), dtype=torch.int8)
    a_s = torch.ones(M, K // 128, dtype=torch.float32)
    b_s = torch.ones(E, (N + 127) // 128, K // 128, dtype=torch.float32)
    c = torch.full((M, N), 5.0, dtype=torch.float32, device=dev)
    _lib_call_grouped_i8(dev, a, a_s, b, b_s, c, seg, widx)
    out = c.cpu()
    for e in range(E):
        lo, hi = int(seg[e]), int(seg[e + 1])
        ref = a[lo:hi].double() @ b[widx[e]].double().T
        assert torch.equal(out[lo:hi].double(), ref), "segment %d" % e
    assert torch.all(out[used:] == 5.0)


@pytest.mark.parametrize("M,N,K,E", [(9000, 2048, 8192, 6), (9000, 1280, 8192, 6), (4700, 4096, 14336, 3)])
def test_grouped_gemm_split_last_round_exact(dev, M, N, K, E):
    """Long K and a number of 256 x 256 tiles that leaves a short last round: the tiles of that round are split
    along K (fp32 partial sums in the scratch, a second kernel adds them).  Same exact-integer check as above;
    column-tile counts that are and are not a multiple of the XCD count, an empty and a one-row segment."""
    announce("grouped split last round", M, N, K, E)
    torch.manual_seed(M + N + K)
    used = M - 5
    cuts = sorted(int(x) for x in torch.randperm(used - 2)[:E - 3] + 2)
    seg = torch.tensor([0, 0, 1] + cuts + [used])                             # an empty and a one-row segment first
    assert len(seg) == E + 1 and bool((seg[1:] >= seg[:-1]).all())
    widx = torch.randperm(E)
    a = torch.randint(-7, 8, (M, K), dtype=torch.int8)
    b = torch.randint(-7, 8, (E, N, K), dtype=torch.int8)
    a_s = torch.ones(M, K // 128, dtype=torch.float32)
    b_s = torch.ones(E, (N + 127) // 128, K // 128, dtype=torch.float32)
    c = torch.full((M, N), 5.0, dtype=torch.float32, device=dev)
    _lib_call_grouped_i8(dev, a, a_s, b, b_s, c, seg, widx)
    out = c.cpu()
    for e in range(E):
        lo, hi = int(seg[e]), int(seg[e + 1])
        ref = (a[lo:hi].float() @ b[widx[e]].float().T)                       # |sum| < 2^24: exact in fp32
        assert torch.equal(out[lo:hi], ref), "segment %d" % e
    assert torch.all(out[used:] == 5.0)


def _lib_call_grouped_i8(dev, a, a_s, b, b_s, c, seg, widx):
    """grouped_gemm_triton on activations that are already int8 with their 1 x 128 scales."""
    d = [t.to(dev).contiguous() for t in (a, a_s, b, b_s, seg.long(), widx.long())]
    gk.grouped_gemm_triton(d[0], d[2], c, b.shape[0], True, d[4], d[5], False, d[1], d[3], [128, 128])
    torch.cuda.synchronize()


def test_grouped_gemm_single_expert_equals_dense_and_weight_indices(dev):
    announce("grouped single expert")
    torch.manual_seed(4)
    M, N, K = 70, 256, 256
    a = torch.randn(M, K).bfloat16()
    w = (torch.randn(3, N, K) * 0.05).bfloat16()
    seg = torch.tensor([0, M])
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    gk.grouped_gemm_triton(a.to(dev), w.to(dev), c, 1, True, seg.to(dev), torch.tensor([2]).to(dev))
    assert_close_scaled(c, a.double() @ w[2].double().T, what="single expert")


@pytest.mark.parametrize("kind", ["int8", "fp8", "bf16"])
def test_ep_moe_forward_small(dev, kind):
    announce("ep_moe_forward", kind)
    torch.manual_seed(5)
    T, H, I, E, topk = 96, 256, 384, 8, 2
    dt = torch.bfloat16
    x = torch.randn(T, H).to(dt)
    logits = torch.randn(T, E)
    ids, w = m.softmax_top2_router(logits, topk)
    w13 = torch.randn(E, 2 * I, H) * 0.05
    w2 = torch.randn(E, H, I) * 0.05
    if kind == "bf16":
        out = ep_moe_forward(x.to(dev), ids.to(dev), w.to(dev), w13.to(dt).to(dev), w2.to(dt).to(dev))
        dense = m.dense_moe_forward(x, ids, w, w13.to(dt), w2.to(dt))
        assert_close_scaled(out, dense, rtol=3e-2, atol=3e-2, what="moe bf16 vs dense")
        return
    wq = q.weight_quant_int8 if kind == "int8" else q.weight_quant_fp8
    aq = q.act_quant_int8 if kind == "int8" else q.act_quant_fp8
    q13 = [wq(w13[e]) for e in range(E)]
    q2 = [wq(w2[e]) for e in range(E)]
    stack = (lambda xs: torch.stack([t.view(torch.uint8) for t in xs]).view(torch.float8_e4m3fn)) if kind == "fp8" else torch.stack
    w13q, w13s = stack([t[0] for t in q13]), torch.stack([t[1] for t in q13])
    w2q, w2s = stack([t[0] for t in q2]), torch.stack([t[1] for t in q2])
    out = ep_moe_forward(x.to(dev), ids.to(dev), w.to(dev), w13q.to(dev), w2q.to(dev), w13s.to(dev), w2s.to(dev),
                         block_shape=[128, 128])
    ref = m.ep_moe_forward(x, ids, w, w13q, w13s, w2q, w2s, aq, dtype=dt)
    assert out.shape == (T, H) and out.dtype == dt
    # two chained GEMMs with a requantisation in between: a one-ulp difference in the bf16 intermediate can
    # flip an 8-bit code, so the end-to-end bound is wider than the per-GEMM bound (checked in test_grouped_gemm)
    assert_close_scaled(out, ref, rtol=5e-2, atol=5e-2, what="moe " + kind)
    dense = m.dense_moe_forward(x, ids, w, w13, w2)
    cos = torch.nn.functional.cosine_similarity(out.float().cpu().flatten(), dense.float().flatten(), dim=0)
    assert cos > 0.99


@pytest.mark.parametrize("kind", ["int8", "fp8", "fp16"])
def test_epmoe_module(dev, kind):
    """The module as the reference's own test drives it (sglang_moe_all_gather_all_reduce_test.py:29-110): gate weight
    ~ N(0, 0.1), expert weights ~ N(0, 0.01) quantised per expert in 128 x 128 blocks, fp16 tokens [2, 24, H];
    forward against the oracle's forward on the module's own routing."""
    announce("EPMoE module", kind)
    torch.manual_seed(42)
    dt = torch.float16
    qm = {"int8": "blockwise_w8a8_int8_gemm", "fp8": "blockwise_w8a8_fp8_gemm", "fp16": None}[kind]
    wdt = {"int8": torch.int8, "fp8": torch.float8_e4m3fn, "fp16": dt}[kind]
    cfg = Config(hidden_size=256, moe_intermediate_size=384, n_routed_experts=16, num_experts_per_tok=4, n_group=4,
                 topk_group=2, quantize_method=qm, w_dtype=wdt, a_dtype=wdt)
    old = torch.get_default_dtype()
    torch.set_default_dtype(dt)
    try:
        mod = EPMoE(cfg).eval()
    finally:
        torch.set_default_dtype(old)
    E, I, H = 16, 384, 256
    w13 = torch.randn(E, 2 * I, H) * 0.01
    w2 = torch.randn(E, H, I) * 0.01
    with torch.no_grad():
        mod.gate.weight.normal_(0.0, 0.1)
        if kind == "fp16":
            mod.w13_weight.copy_(w13)
            mod.w2_weight.copy_(w2)
        else:
            wq = q.weight_quant_int8 if kind == "int8" else q.weight_quant_fp8
            for e in range(E):
                a, s_a = wq(w13[e])
                b, s_b = wq(w2[e])
                mod.w13_weight[e] = a
                mod.w13_weight_scale[e] = s_a
                mod.w2_weight[e] = b
                mod.w2_weight_scale[e] = s_b
    x = torch.randn(2, 24, H).to(dt)
    mod = mod.to(dev)
    with torch.no_grad():
        out = mod(x.to(dev))
        ids, w = mod.gate(x.to(dev))
    assert out.shape == (2, 24, H) and out.dtype == dt
    ids, w = ids.cpu(), w.cpu()
    # the routing itself: the token's expert set against the loop oracle (scores are far from ties at this size)
    oids, _ = m.deepseek_gate(x, mod.gate.weight.detach().cpu(), mod.gate.e_score_correction_bias.detach().cpu(), 4, 4, 2, True, 2.5)
    assert sum(set(ids[t].tolist()) == oids[t] for t in range(48)) >= 47
    if kind == "fp16":
        dense = m.dense_moe_forward(x.reshape(-1, H), ids, w, mod.w13_weight.detach().cpu(), mod.w2_weight.detach().cpu())
        assert_close_scaled(out.reshape(-1, H), dense, rtol=3e-2, atol=3e-2, what="EPMoE fp16 vs dense")
        return
    aq = q.act_quant_int8 if kind == "int8" else q.act_quant_fp8
    ref = m.ep_moe_forward(x.reshape(-1, H), ids, w, mod.w13_weight.detach().cpu(), mod.w13_weight_scale.detach().cpu(),
                           mod.w2_weight.detach().cpu(), mod.w2_weight_scale.detach().cpu(), aq, dtype=dt)
    assert_close_scaled(out.reshape(-1, H), ref, rtol=5e-2, atol=5e-2, what="EPMoE " + kind)


def test_router(dev):
    logits = torch.randn(33, 8)
    ids, w = softmax_topk_router(logits.to(dev), 2)
    oids, ow = m.softmax_top2_router(logits, 2)
    assert torch.equal(ids.cpu(), oids) and torch.allclose(w.cpu(), ow, atol=1e-6)


def _oracle_rows(a_rows, s_rows, w, ws, chunk=8192):
    """gemm_blockwise of a few activation rows against one expert's weights, over column chunks of the weights
    (bounds the float64 temporaries at Mixtral sizes)."""
    N = w.shape[0]
    out = []
    for n0 in range(0, N, chunk):
        n1 = min(N, n0 + chunk)
        out.append(g.gemm_blockwise(a_rows, s_rows, w[n0:n1], ws[n0 // 128:(n1 + 127) // 128]))
    return torch.cat(out, dim=-1)


def _check_grouped_gemm_per_segment(c, a, a_s, w, ws, seg, what, seed=0):
    """c [M, N] on the device against moe_ref.grouped_gemm's formula, expert by expert: the first, the last and two
    random rows of every segment (all columns) at rtol = atol = 1e-2, and the column sums of the WHOLE segment
    against a one-row oracle GEMM of the scale-weighted column sums of its activation rows (a wrong tile
    anywhere in the segment moves them)."""
    assert bool(torch.isfinite(c.float()).all()), what + ": non-finite output"
    gen = torch.Generator().manual_seed(seed)
    ah, ash, segl = a.cpu(), a_s.cpu(), seg.cpu().tolist()
    K = ah.shape[1]
    for e in range(len(segl) - 1):
        m0, m1 = segl[e], segl[e + 1]
        if m1 <= m0:
            continue
        rows = sorted({m0, m1 - 1, *(m0 + torch.randint(0, m1 - m0, (2,), generator=gen)).tolist()})
        rt = torch.tensor(rows)
        we, wse = w[e].cpu(), ws[e].cpu()
        ref = _oracle_rows(ah[rt], ash[rt], we, wse)
        assert_close_scaled(c[rt.to(c.device)], ref, what="%s expert %d rows %s" % (what, e, rows))
        n = m1 - m0
        wsum = (ah[m0:m1].float().double().reshape(n, K // 128, 128) * ash[m0:m1].double()[:, :, None]).sum(0).reshape(1, K)
        want = _oracle_rows(wsum, torch.ones(1, K // 128, dtype=torch.float64), we.float(), wse)[0]
        got = c[m0:m1].double().sum(0).cpu()
        bound = 1e-2 * ref.pow(2).mean().sqrt().item() * (n ** 0.5) + 1e-2 * want.abs()
        bad = (got - want).abs() > bound
        assert not bad.any(), "%s expert %d: column checksum off in %d columns (max %.3e)" % (
            what, e, int(bad.sum()), (got - want).abs().max().item())


@pytest.mark.parametrize("kind", ["fp8", "int8"])
def test_ep_moe_mixtral_dims_full_size(dev, kind):
    """8 experts, hidden 4096, intermediate 14336, 4096 tokens, top-2, 128x128 block-scaled weights (the MoE
    benchmark workloads, fp8 and int8).

    (1) Each of the two grouped GEMMs alone, on the operands the forward feeds it, against the oracle at
        rtol = atol = 1e-2: sampled rows of every segment plus a checksum over every row of every segment.
    (2) The whole forward on 256 sampled tokens against the CPU oracle with every rounding point reproduced
        (the forward is separable by token); two chained GEMMs with a requantisation in between, where one ulp of
        the bf16 intermediate can flip an 8-bit code, hence the wider end-to-end bound.
    (3) Per-expert segment lengths equal the router's histogram; every output is finite.
    """
    announce("ep_moe mixtral full size", kind)
    torch.manual_seed(11)
    T, H, I, E, topk = 4096, 4096, 14336, 8, 2
    fp8 = kind == "fp8"
    qdt = torch.float8_e4m3fn if fp8 else torch.int8
    sdt = torch.float32 if fp8 else torch.float16
    wq = fp8_kernel.weight_quant if fp8 else int8_kernel.weight_quant
    w13 = torch.empty(E, 2 * I, H, dtype=qdt, device=dev)
    w13s = torch.empty(E, 2 * I // 128, H // 128, dtype=sdt, device=dev)
    w2 = torch.empty(E, H, I, dtype=qdt, device=dev)
    w2s = torch.empty(E, H // 128, I // 128, dtype=sdt, device=dev)
    for e in range(E):
        w13[e], w13s[e] = wq(torch.randn(2 * I, H, device=dev) * 0.02)
        w2[e], w2s[e] = wq(torch.randn(H, I, device=dev) * 0.02)
    x = torch.randn(T, H, device=dev).bfloat16()
    ids, wts = softmax_topk_router(torch.randn(T, E, device=dev), topk)
    rids, src2dst, seg = gk.run_moe_ep_preproess(ids, E)
    assert (seg[1:] - seg[:-1]).tolist() == torch.bincount(ids.flatten(), minlength=E).tolist()
    widx = torch.arange(E, device=dev)

    # (1) gate / up projection: 8192 x 28672 x 4096
    a1, a1s = gk.pre_reorder_quant(x, src2dst, ids, None, 0, E - 1, topk, H, qdt)
    gu = torch.empty(T * topk, 2 * I, dtype=torch.bfloat16, device=dev)
    gk.grouped_gemm_triton(a1, w13, gu, E, True, seg, widx, False, a1s, w13s, [128, 128])
    _check_grouped_gemm_per_segment(gu, a1, a1s, w13, w13s, seg, "mixtral %s gate/up" % kind, seed=1)
    # down projection: 8192 x 4096 x 14336
    a2, a2s = gk.act_and_mul_quant(gu, 2 * I, rids, None, 0, E - 1, qdt, "silu")
    do = torch.empty(T * topk, H, dtype=torch.bfloat16, device=dev)
    gk.grouped_gemm_triton(a2, w2, do, E, True, seg, widx, False, a2s, w2s, [128, 128])
    _check_grouped_gemm_per_segment(do, a2, a2s, w2, w2s, seg, "mixtral %s down" % kind, seed=2)
    del a1, a1s, a2, a2s, gu, do

    # (2) whole forward, 256 sampled tokens against the oracle
    out = ep_moe_forward(x, ids, wts, w13, w2, w13s, w2s, block_shape=[128, 128])
    assert out.shape == (T, H) and bool(torch.isfinite(out.float()).all())
    sub = torch.arange(0, T, T // 256, device=dev)[:256]
    aq = q.act_quant_fp8 if fp8 else q.act_quant_int8
    ref = m.ep_moe_forward(x[sub].cpu(), ids[sub].cpu(), wts[sub].cpu(), w13.cpu(), w13s.cpu(), w2.cpu(), w2s.cpu(),
                           aq, dtype=torch.bfloat16)
    assert_close_scaled(out[sub], ref, rtol=5e-2, atol=5e-2, what="mixtral %s forward, 256 tokens vs oracle" % kind)
    # the same tokens through the decode-sized kernels (a 32-token forward) agree with the large-M run
    sub32 = sub[::8]
    out_sub = ep_moe_forward(x[sub32].contiguous(), ids[sub32].contiguous(), wts[sub32].contiguous(), w13, w2, w13s, w2s,
                             block_shape=[128, 128])
    assert_close_scaled(out[sub32], out_sub.float(), rtol=3e-2, atol=3e-2, what="full vs 32-token run")


# ------------------------------------------------------------------ fused permute / activation + quantisation
@pytest.mark.parametrize("qdt", [torch.float8_e4m3fn, torch.int8])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_scales", [False, True])
def test_fused_quant_kernels_equal_the_two_kernel_sequence(dev, qdt, dtype, with_scales):
    """pre_reorder_quant == act_quant(pre_reorder) and act_and_mul_quant == act_quant(silu/gelu_and_mul), bit for
    bit, on the rows of local experts (start/end expert window narrower than the expert set)."""
    announce("fused quant", qdt, dtype, with_scales)
    torch.manual_seed(3)
    T, H, I, E, topk = 70, 384, 256, 8, 2
    start_e, end_e = 1, 6
    act_quant = fp8_kernel.act_quant if qdt == torch.float8_e4m3fn else int8_kernel.act_quant
    x = (torch.randn(T, H) * 3).to(dtype).to(dev)
    ids = torch.stack([torch.randperm(E)[:topk] for _ in range(T)]).to(dev)
    reorder_ids, src2dst, seg = gk.run_moe_ep_preproess(ids, E)
    a1 = (torch.rand(end_e - start_e + 1) + 0.5).to(dev) if with_scales else None
    local_rows = ((reorder_ids >= start_e) & (reorder_ids <= end_e)).cpu()

    plain = torch.zeros(T * topk, H, dtype=dtype, device=dev)
    gk.pre_reorder(x, plain, src2dst, ids, a1, start_e, end_e, topk, H)
    q0, s0 = act_quant(plain)
    q1, s1 = gk.pre_reorder_quant(x, src2dst, ids, a1, start_e, end_e, topk, H, qdt)
    assert q1.dtype == qdt and s1.dtype == s0.dtype and s1.shape == s0.shape
    assert torch.equal(q1.view(torch.uint8).cpu()[local_rows], q0.view(torch.uint8).cpu()[local_rows])
    assert torch.equal(s1.cpu()[local_rows], s0.cpu()[local_rows])

    gateup = (torch.randn(T * topk, 2 * I) * 2).to(dtype).to(dev)
    for name, fn in (("silu", gk.silu_and_mul), ("gelu", gk.gelu_and_mul)):
        down = torch.zeros(T * topk, I, dtype=dtype, device=dev)
        fn(gateup, down, 2 * I, reorder_ids, a1, start_e, end_e)
        q0, s0 = act_quant(down)
        q1, s1 = gk.act_and_mul_quant(gateup, 2 * I, reorder_ids, a1, start_e, end_e, qdt, name)
        assert torch.equal(q1.view(torch.uint8).cpu()[local_rows], q0.view(torch.uint8).cpu()[local_rows]), name
        assert torch.equal(s1.cpu()[local_rows], s0.cpu()[local_rows]), name


@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_ep_moe_forward_fused_equals_unfused(dev, kind):
    announce("ep_moe fused vs unfused", kind)
    torch.manual_seed(9)
    T, H, I, E, topk = 200, 256, 384, 8, 2
    dt = torch.bfloat16
    x = torch.randn(T, H).to(dt).to(dev)
    ids, w = softmax_topk_router(torch.randn(T, E).to(dev), topk)
    wq = int8_kernel.weight_quant if kind == "int8" else fp8_kernel.weight_quant
    w13 = [wq((torch.randn(2 * I, H) * 0.05).to(dev)) for _ in range(E)]
    w2 = [wq((torch.randn(H, I) * 0.05).to(dev)) for _ in range(E)]
    cat = lambda xs: torch.stack([t.view(torch.uint8) for t in xs]).view(xs[0].dtype)
    args = (x, ids, w, cat([t[0] for t in w13]), cat([t[0] for t in w2]), torch.stack([t[1] for t in w13]),
            torch.stack([t[1] for t in w2]))
    a = ep_moe_forward(*args, block_shape=[128, 128], fuse_quant=True)
    b = ep_moe_forward(*args, block_shape=[128, 128], fuse_quant=False)
    assert torch.equal(a, b)


@pytest.mark.parametrize("qdt", [torch.float8_e4m3fn, torch.int8])
@pytest.mark.parametrize("dtype,act", [(torch.bfloat16, "silu"), (torch.float16, "gelu")])
@pytest.mark.parametrize("rows,two_i,K", [(8000, 4096, 256), (4800, 4096, 256), (8000, 3840, 384)])
def test_gate_up_gemm_with_activation_epilogue_equals_three_kernels(dev, qdt, dtype, act, rows, two_i, K):
    """grouped_gemm_swiglu_quant == act_and_mul_quant(grouped_gemm_triton(...)) bit for bit, values and scales, on shapes
    that the dispatch gives to the 256-row (8000 rows) and 128-row (4800 rows) tiles of the large grouped kernel: a
    number of column tiles that is and is not a multiple of the XCD count, one empty segment, one shorter than a tile,
    ragged ends, permuted weight indices, rows behind the last segment untouched."""
    announce("gate/up + activation epilogue", qdt, dtype, act, rows, two_i, K)
    E = 8
    torch.manual_seed(rows + two_i)
    used = rows - 5
    cuts = sorted(torch.randint(0, used, (E - 3,)).tolist())
    seg = torch.tensor([0, 37, 37] + cuts + [used], dtype=torch.int64, device=dev)     # segment 0: 37 rows, segment 1: empty
    widx = torch.randperm(E).to(dev)
    act_quant = fp8_kernel.act_quant if qdt == torch.float8_e4m3fn else int8_kernel.act_quant
    wq = fp8_kernel.weight_quant if qdt == torch.float8_e4m3fn else int8_kernel.weight_quant
    a, a_s = act_quant((torch.randn(rows, K) * 2).to(dtype).to(dev))
    ws = [wq((torch.randn(two_i, K) * 0.3).to(dev)) for _ in range(E)]
    b = torch.stack([t[0].view(torch.uint8) for t in ws]).view(qdt)
    b_s = torch.stack([t[1] for t in ws])
    assert gk.grouped_gemm_swiglu_quant_fused(a, b, E)
    q1, s1 = gk.grouped_gemm_swiglu_quant(a, a_s, b, b_s, E, seg, widx, dtype, act)

    c = torch.zeros(rows, two_i, dtype=dtype, device=dev)
    gk.grouped_gemm_triton(a=a, b=b, c=c, batch_size=E, weight_column_major=True, seg_indptr=seg, weight_indices=widx,
                           scale_a=a_s, scale_b=b_s, block_shape=[128, 128])
    ids = torch.zeros(rows, dtype=torch.int64, device=dev)
    q0, s0 = gk.act_and_mul_quant(c, two_i, ids, None, 0, E - 1, qdt, act)
    assert q1.shape == q0.shape and s1.shape == s0.shape and s1.dtype == s0.dtype
    assert torch.equal(s1[:used].cpu(), s0[:used].cpu())
    assert torch.equal(q1[:used].view(torch.uint8).cpu(), q0[:used].view(torch.uint8).cpu())
    assert float(s0[:used].float().abs().max()) > 0


def test_gate_up_activation_epilogue_refuses_small_shapes(dev):
    """Shapes that run on the smaller tile kernels are not taken: the query says so and the entry point fails."""
    a = torch.zeros(64, 256, dtype=torch.int8, device=dev)
    b = torch.zeros(4, 512, 256, dtype=torch.int8, device=dev)
    assert not gk.grouped_gemm_swiglu_quant_fused(a, b, 4)
    seg = torch.tensor([0, 16, 32, 48, 64], dtype=torch.int64, device=dev)
    with pytest.raises(AssertionError, match="not one the fused kernel takes"):
        gk.grouped_gemm_swiglu_quant(a, torch.ones(64, 2, dtype=torch.float16, device=dev), b,
                                     torch.ones(4, 4, 2, dtype=torch.float16, device=dev), 4, seg, None, torch.bfloat16)


def test_grouped_gemm_per_expert_scalar_scales(dev):
    """use_fp8_w8a8 without block_shape: c = (a . b^T) * scale_a[e] * scale_b[e] (reference :417-420, commented out there)."""
    announce("grouped gemm per-expert scales")
    torch.manual_seed(4)
    E, N, K = 4, 192, 256
    seg = torch.tensor([0, 5, 5, 40, 64], dtype=torch.int64)
    a = (torch.randn(64, K) * 0.5).to(torch.float8_e4m3fn)
    b = (torch.randn(E, N, K) * 0.5).to(torch.float8_e4m3fn)
    sa, sb = torch.rand(E) + 0.5, torch.rand(E) + 0.5
    c = torch.zeros(64, N, dtype=torch.bfloat16, device=dev)
    gk.grouped_gemm_triton(a.to(dev), b.to(dev), c, E, True, seg.to(dev), torch.arange(E, device=dev), True,
                           sa.to(dev), sb.to(dev), None)
    ref = torch.zeros(64, N, dtype=torch.float64)
    for e in range(E):
        r0, r1 = int(seg[e]), int(seg[e + 1])
        ref[r0:r1] = a[r0:r1].double() @ b[e].double().T * float(sa[e]) * float(sb[e])
    assert_close_scaled(c, ref, what="per-expert scales")
