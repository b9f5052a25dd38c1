"""One GPU's share of the EP-MoE forward: permute -> grouped GEMM -> SwiGLU -> grouped GEMM -> un-permute.

The call order, buffer shapes and dtypes are those of EPMoE.forward in the reference
(moe/sglang_moe_all_gather_all_reduce.py:267-446) with all experts local; the final all-reduce across
ranks is outside this path.
"""
from typing import List, Optional

import torch

from .group_gemm_kernel import (grouped_gemm_triton, post_reorder, pre_reorder, run_moe_ep_preproess,
                                silu_and_mul, gelu_and_mul, pre_reorder_quant, act_and_mul_quant)


def softmax_topk_router(router_logits: torch.Tensor, top_k: int = 2, renormalize: bool = True):
    p = torch.softmax(router_logits.float(), dim=-1)
    w, ids = torch.topk(p, top_k, dim=-1)
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)
    return ids, w


_widx_cache = {}


def _weight_indices(E, dev):
    """arange(E) on the device (reference sglang_moe_all_gather_all_reduce.py:327), built once per (E, device):
    the grouped GEMM only reads it, and a launch per forward is 5 us of a decode-sized forward."""
    key = (E, dev.type, dev.index)
    t = _widx_cache.get(key)
    if t is None:
        t = _widx_cache[key] = torch.arange(0, E, device=dev, dtype=torch.int64)
    return t


def ep_moe_forward(hidden_states: torch.Tensor, topk_ids: torch.Tensor, topk_weights: torch.Tensor,
                   w13_weight: torch.Tensor, w2_weight: torch.Tensor,
                   w13_weight_scale: Optional[torch.Tensor] = None, w2_weight_scale: Optional[torch.Tensor] = None,
                   block_shape: Optional[List[int]] = None, activation: str = "silu",
                   start_expert_id: int = 0, end_expert_id: Optional[int] = None, fuse_quant: bool = True):
    """hidden_states [T, H]; w13 [E, 2I, H] (gate rows first, then up), w2 [E, H, I]. Returns [T, H].

    With block-quantised weights and `fuse_quant`, the permutation and the gated activation write the
    1 x 128 quantised activations of the following grouped GEMM directly (same results bit for bit as the
    separate kernels, two activation round trips through HBM fewer)."""
    T, H = hidden_states.shape
    E = w13_weight.shape[0]
    top_k = topk_ids.shape[1]
    if end_expert_id is None:
        end_expert_id = start_expert_id + E - 1
    num_experts = end_expert_id + 1
    dev, dt = hidden_states.device, hidden_states.dtype
    topk_ids = topk_ids.contiguous()
    topk_weights = topk_weights.contiguous()

    reorder_topk_ids, src2dst, seg_indptr = run_moe_ep_preproess(topk_ids, num_experts)
    seg_cur = seg_indptr[start_expert_id:end_expert_id + 2]
    widx = _weight_indices(E, dev)
    quantised = block_shape is not None and w13_weight.dtype in (torch.int8, torch.float8_e4m3fn)
    fused = bool(fuse_quant and quantised and H % 128 == 0 and (w13_weight.shape[1] // 2) % 128 == 0
                 and dt in (torch.float16, torch.bfloat16))

    if fused:
        gateup_input, a1_s = pre_reorder_quant(hidden_states, src2dst, topk_ids, None, start_expert_id, end_expert_id,
                                               top_k, H, w13_weight.dtype)
    else:
        gateup_input, a1_s = torch.empty((T * top_k, H), device=dev, dtype=dt), None
        pre_reorder(hidden_states, gateup_input, src2dst, topk_ids, None, start_expert_id, end_expert_id, top_k, H)
    gateup_output = torch.empty(gateup_input.shape[0], w13_weight.shape[1], device=dev, dtype=dt)
    grouped_gemm_triton(a=gateup_input, b=w13_weight, c=gateup_output, batch_size=E, weight_column_major=True,
                        seg_indptr=seg_cur, weight_indices=widx, use_fp8_w8a8=False, scale_a=a1_s,
                        scale_b=w13_weight_scale, block_shape=block_shape)

    if fused:
        down_input, a2_s = act_and_mul_quant(gateup_output, gateup_output.shape[1], reorder_topk_ids, None,
                                             start_expert_id, end_expert_id, w2_weight.dtype, activation)
    else:
        down_input, a2_s = torch.empty(gateup_output.shape[0], gateup_output.shape[1] // 2, device=dev, dtype=dt), None
        act = {"silu": silu_and_mul, "gelu": gelu_and_mul}[activation]
        act(gateup_output, down_input, gateup_output.shape[1], reorder_topk_ids, None, start_expert_id, end_expert_id)
    down_output = torch.empty(down_input.shape[0], w2_weight.shape[1], device=dev, dtype=dt)
    grouped_gemm_triton(a=down_input, b=w2_weight, c=down_output, batch_size=E, weight_column_major=True,
                        seg_indptr=seg_cur, weight_indices=widx, use_fp8_w8a8=False, scale_a=a2_s,
                        scale_b=w2_weight_scale, block_shape=block_shape)

    output = torch.empty((T, H), device=dev, dtype=dt)
    post_reorder(down_output, output, src2dst, topk_ids, topk_weights, start_expert_id, end_expert_id, top_k, H)
    return output
