"""EP-MoE single-GPU path restated with torch-CPU closed forms (test oracle).

run_moe_ep_preprocess  moe/group_gemm_kernel.py:19-78
pre_reorder            moe/group_gemm_kernel.py:81-117
silu_and_mul           moe/group_gemm_kernel.py:120-168   (gelu variant :176-235)
post_reorder           moe/group_gemm_kernel.py:238-288
grouped_gemm           moe/group_gemm_kernel.py:314-513, torch statement at
                       moe/sglang_moe_all_gather_all_reduce.py:58-159
ep_moe_forward         moe/sglang_moe_all_gather_all_reduce.py:267-446 (wiring)
dense_moe_forward      per-expert loop of moe/ep_moe_without_all2all.py:236-290 (independent check)
"""
import torch
import torch.nn.functional as F

from . import quant_ref, gemm_ref


def run_moe_ep_preprocess(topk_ids: torch.Tensor, num_experts: int):
    flat = topk_ids.reshape(-1)
    reorder_topk_ids, reorder_ids = torch.sort(flat, stable=True)
    counts = torch.bincount(flat.clamp(min=0), minlength=num_experts)[:num_experts]
    seg_indptr = torch.zeros(num_experts + 1, dtype=torch.int64)
    seg_indptr[1:] = torch.cumsum(counts, 0)
    src2dst = torch.empty(flat.numel(), dtype=torch.int32)
    src2dst[reorder_ids] = torch.arange(flat.numel(), dtype=torch.int32)
    return reorder_topk_ids, src2dst, seg_indptr


def pre_reorder(x, src2dst, topk_ids, a1_scales, start_expert, end_expert, topk, out=None):
    T, H = x.shape
    if out is None:
        out = torch.zeros(T * topk, H, dtype=x.dtype)
    for t in range(T):
        for j in range(topk):
            e = int(topk_ids[t, j])
            if start_expert <= e <= end_expert:
                scale = 1.0 if a1_scales is None else 1.0 / float(a1_scales[e - start_expert])
                out[int(src2dst[t * topk + j])] = (x[t].float() * scale).to(out.dtype)
    return out


def silu_and_mul(gateup, reorder_topk_ids, scales, start_expert, end_expert, out_dtype=None, act="silu"):
    """silu in fp32, cast to the input dtype, then gate*up*scale in the input dtype."""
    M, H2 = gateup.shape
    I = H2 // 2
    dt = gateup.dtype
    out = torch.zeros(M, I, dtype=out_dtype or dt)
    g32 = gateup[:, :I].float()
    if act == "silu":
        a = g32 * torch.sigmoid(g32)
    else:
        k = 0.7978845608028654
        a = 0.5 * g32 * (1 + (2 * torch.sigmoid(2 * (k * (g32 + 0.044715 * g32 * g32 * g32))) - 1))
    a = a.to(dt)
    res = a * gateup[:, I:]
    if scales is not None:
        sc = (1.0 / scales.float()).to(dt)[(reorder_topk_ids - start_expert).clamp(0, scales.numel() - 1)]
        res = res * sc[:, None]
    mask = (reorder_topk_ids >= start_expert) & (reorder_topk_ids <= end_expert)
    out[mask] = res[mask].to(out.dtype)
    return out, mask


def post_reorder(down_out, src2dst, topk_ids, topk_weights, start_expert, end_expert, topk):
    """out[t] = sum_j down_out[src2dst[t,j]] * dtype(w[t,j]), accumulated in down_out.dtype."""
    T = topk_ids.shape[0]
    H = down_out.shape[1]
    dt = down_out.dtype
    out = torch.zeros(T, H, dtype=dt)
    s2d = src2dst.reshape(T, topk).long()
    for j in range(topk):
        e = topk_ids[:, j]
        sel = (e >= start_expert) & (e <= end_expert)
        w = topk_weights[:, j].to(dt)
        rows = down_out[s2d[:, j].clamp(0, down_out.shape[0] - 1)]
        contrib = rows * w[:, None]
        out = torch.where(sel[:, None], out + contrib, out)
    return out


def grouped_gemm(a, b, seg_indptr, weight_indices, scale_a=None, scale_b=None, block=128):
    """float64 result [M,N] of C[seg[e]:seg[e+1]] = A[seg] @ W[weight_indices[e]]^T (optionally block scaled)."""
    M = a.shape[0]
    N = b.shape[1]
    c = torch.zeros(M, N, dtype=torch.float64)
    for e in range(seg_indptr.numel() - 1):
        m0, m1 = int(seg_indptr[e]), int(seg_indptr[e + 1])
        if m1 <= m0:
            continue
        w = b[int(weight_indices[e])]
        if scale_b is not None:
            c[m0:m1] = gemm_ref.gemm_blockwise(a[m0:m1], scale_a[m0:m1], w, scale_b[int(weight_indices[e])], block)
        else:
            c[m0:m1] = a[m0:m1].double() @ w.double().T
    return c


def softmax_top2_router(logits, topk=2):
    p = torch.softmax(logits.float(), dim=-1)
    w, ids = torch.topk(p, topk, dim=-1)
    w = w / w.sum(dim=-1, keepdim=True)
    return ids, w


def dense_moe_forward(x, topk_ids, topk_w, w13_deq, w2_deq):
    """Unquantized per-expert SwiGLU MLP loop in float64 (independent of the permute path)."""
    T, H = x.shape
    E = w13_deq.shape[0]
    I = w2_deq.shape[2]
    out = torch.zeros(T, H, dtype=torch.float64)
    xd = x.double()
    for e in range(E):
        tok, slot = torch.where(topk_ids == e)
        if tok.numel() == 0:
            continue
        h = xd[tok] @ w13_deq[e].double().T
        act = F.silu(h[:, :I]) * h[:, I:]
        y = act @ w2_deq[e].double().T
        out.index_add_(0, tok, y * topk_w[tok, slot].double()[:, None])
    return out


def ep_moe_forward(x, topk_ids, topk_w, w13, w13_s, w2, w2_s, act_quant, dtype=torch.bfloat16):
    """The reference EPMoE.forward order with every rounding point reproduced.

    act_quant(a) -> (a_q, a_s) is the 1x128 activation quantizer of the weight dtype
    (int8 in the reference, group_gemm_kernel.py:459-465; e4m3fn for fp8 weights).
    """
    T, H = x.shape
    E = w13.shape[0]
    topk = topk_ids.shape[1]
    rids, src2dst, seg = run_moe_ep_preprocess(topk_ids, E)
    gin = pre_reorder(x, src2dst, topk_ids, None, 0, E - 1, topk)
    widx = torch.arange(E)
    aq, as_ = act_quant(gin)
    gu = grouped_gemm(aq, w13, seg, widx, as_, w13_s).to(dtype)
    di, _ = silu_and_mul(gu, rids, None, 0, E - 1)
    dq, ds = act_quant(di)
    do = grouped_gemm(dq, w2, seg, widx, ds, w2_s).to(dtype)
    return post_reorder(do, src2dst, topk_ids, topk_w, 0, E - 1, topk)


def deepseek_gate(x, weight, bias, top_k, n_group, topk_group, norm_topk_prob=True, routed_scaling_factor=1.0):
    """The router EPMoE owns (MoEGate.forward, moe/all2all_moe.py:60-118), token by token in float64 loops.

    Returns (list of expert-id sets, list of {expert: weight}) so that the order inside a token's top-k, which
    the reference leaves open (topk(..., sorted=False)), does not enter a comparison."""
    import math
    xs = x.reshape(-1, x.shape[-1]).double()
    E = weight.shape[0]
    per = E // n_group
    ids_out, w_out = [], []
    for t in range(xs.shape[0]):
        score = [1.0 / (1.0 + math.exp(-float(xs[t] @ weight[e].double()))) for e in range(E)]     # :64-68
        biased = [score[e] + float(bias[e]) for e in range(E)]                                       # :77
        rank = []
        for gi in range(n_group):                                                                    # :80-82
            best = sorted(biased[gi * per:(gi + 1) * per], reverse=True)[:2]
            rank.append(sum(best))
        groups = sorted(range(n_group), key=lambda gi: -rank[gi])[:topk_group]                       # :84-85
        cand = [biased[e] if e // per in groups else 0.0 for e in range(E)]                          # :88-101
        chosen = sorted(range(E), key=lambda e: -cand[e])[:top_k]                                    # :104-106
        w = {e: score[e] for e in chosen}                                                            # :107 (unbiased)
        if top_k > 1 and norm_topk_prob:                                                             # :114-116
            den = sum(w.values()) + 1e-20
            w = {e: v / den for e, v in w.items()}
        w = {e: v * routed_scaling_factor for e, v in w.items()}                                     # :117
        ids_out.append(set(chosen))
        w_out.append(w)
    return ids_out, w_out
