"""One GPU's share of the EP-MoE forward: permute -> grouped GEMM -> SwiGLU -> grouped GEMM -> un-permute.

The call order, buffer shapes and dtypes are those of EPMoE.forward in the reference
(moe/sglang_moe_all_gather_all_reduce.py:267-446) with all experts local; the final all-reduce across
ranks is outside this path.  `ep_moe_forward` is that forward as a function of (tokens, routing, weights);
`EPMoE` is the reference's module around it (gate + expert weights + scales, same attribute names), and
`MoEGate` the DeepSeek-V3 router it owns (moe/all2all_moe.py:31-118).
"""
import math
from typing import List, Optional

import torch
from torch import nn

from .group_gemm_kernel import (grouped_gemm_triton, post_reorder, pre_reorder, run_moe_ep_preproess,
                                silu_and_mul, gelu_and_mul, pre_reorder_quant, act_and_mul_quant,
                                grouped_gemm_swiglu_quant, grouped_gemm_swiglu_quant_fused)


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
    # large launches: the gated activation and the quantiser of the down projection run in the epilogue of the gate / up
    # GEMM (same bits, the [rows, 2I] tensor is never written)
    one_kernel = fused and w2_weight.dtype == w13_weight.dtype and grouped_gemm_swiglu_quant_fused(gateup_input, w13_weight, E)
    if one_kernel:
        down_input, a2_s = grouped_gemm_swiglu_quant(gateup_input, a1_s, w13_weight, w13_weight_scale, E, seg_cur, widx, dt,
                                                     activation)
    else:
        gateup_output = torch.empty(gateup_input.shape[0], w13_weight.shape[1], device=dev, dtype=dt)
        grouped_gemm_triton(a=gateup_input, b=w13_weight, c=gateup_output, batch_size=E, weight_column_major=True,
                            seg_indptr=seg_cur, weight_indices=widx, use_fp8_w8a8=False, scale_a=a1_s,
                            scale_b=w13_weight_scale, block_shape=block_shape)

    if one_kernel:
        pass
    elif fused:
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


class MoEGate(nn.Module):
    """Sigmoid scores, group-limited top-k ("noaux_tc"), as moe/all2all_moe.py:60-118.

    Per token: scores = sigmoid(x W^T) in fp32; the experts are split into n_group groups, a group is ranked by
    the sum of its two largest (score + e_score_correction_bias), only the experts of the best topk_group groups
    keep their biased score (the others count as 0.0), the top_k of those are the token's experts; their weights
    are the unbiased scores, normalised to sum 1 when norm_topk_prob (denominator + 1e-20), times
    routed_scaling_factor.  Plain torch on whatever device the module lives on: routing is not part of the GEMM path.
    """

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.top_k = config.num_experts_per_tok
        self.n_routed_experts = config.n_routed_experts
        self.routed_scaling_factor = config.routed_scaling_factor
        self.scoring_func = config.scoring_func
        self.topk_method = config.topk_method
        self.n_group = config.n_group
        self.topk_group = config.topk_group
        self.norm_topk_prob = config.norm_topk_prob
        self.gating_dim = config.hidden_size
        self.weight = nn.Parameter(torch.empty((self.n_routed_experts, self.gating_dim)))
        if self.topk_method == "noaux_tc":
            self.e_score_correction_bias = nn.Parameter(torch.zeros((self.n_routed_experts,)))
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))

    def forward(self, hidden_states):
        if self.scoring_func != "sigmoid":
            raise NotImplementedError(f"insupportable scoring function for MoE gating: {self.scoring_func}")
        if self.topk_method != "noaux_tc":
            raise NotImplementedError(f"insupportable TopK function for MoE gating: {self.topk_method}")
        assert not self.training
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        n, E, G = x.shape[0], self.n_routed_experts, self.n_group
        scores = torch.sigmoid(x.float() @ self.weight.float().t())
        biased = scores + self.e_score_correction_bias.float()[None, :]
        per_group = biased.view(n, G, E // G)
        group_rank = per_group.topk(2, dim=-1).values.sum(dim=-1)                  # [n, G]
        keep = torch.zeros_like(group_rank, dtype=torch.bool)
        keep.scatter_(1, group_rank.topk(self.topk_group, dim=-1, sorted=False).indices, True)
        candidates = torch.where(keep[:, :, None], per_group, torch.zeros((), device=x.device)).reshape(n, E)
        topk_idx = candidates.topk(self.top_k, dim=-1, sorted=False).indices
        topk_weight = scores.gather(1, topk_idx)
        if self.top_k > 1 and self.norm_topk_prob:
            topk_weight = topk_weight / (topk_weight.sum(dim=-1, keepdim=True) + 1e-20)
        return topk_idx, topk_weight * self.routed_scaling_factor


class EPMoE(nn.Module):
    """The reference's module (moe/sglang_moe_all_gather_all_reduce.py:162-446): a MoEGate, the stacked expert
    weights w13_weight [E, 2I, H] / w2_weight [E, H, I] in config.w_dtype (or the default dtype when
    config.quantize_method is None) and, with block quantisation, their fp16 scales w13_weight_scale
    [E, 2 ceil(I / bn), ceil(H / bk)] / w2_weight_scale [E, ceil(H / bn), ceil(I / bk)], all initialised to ones
    as there (the weight-init recipe of sglang_moe_all_gather_all_reduce_test.py:29-69 fills them).

    forward(hidden_states [B, S, H]) -> [B, S, H].  One GPU holds every expert here: config.ep_size must be 1, the
    reference's closing all-reduce over the expert-parallel ranks (:442-443) has nothing to add and is not issued.
    """

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.tp_size = config.ep_size or 1
        if self.tp_size != 1:
            raise NotImplementedError("EPMoE: this build runs every expert on one GPU (config.ep_size must be 1)")
        self.tp_rank = 0
        self.num_experts = config.n_routed_experts
        self.num_experts_per_partition = self.num_experts
        self.start_expert_id = 0
        self.end_expert_id = self.num_experts - 1
        self.top_k = config.num_experts_per_tok
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.moe_intermediate_size
        self.activation = config.hidden_act
        self.gate = MoEGate(config)
        quantised = config.quantize_method is not None
        params_dtype = config.w_dtype if quantised else torch.get_default_dtype()
        E, I, H = self.num_experts, self.intermediate_size, self.hidden_size

        def ones(*shape, dtype):
            # (torch.ones has no fp8 kernel: build in fp32 and cast)
            return nn.Parameter(torch.ones(*shape, dtype=torch.float32).to(dtype), requires_grad=False)

        self.w13_weight = ones(E, 2 * I, H, dtype=params_dtype)
        self.w2_weight = ones(E, H, I, dtype=params_dtype)
        self.w13_input_scale = None
        self.w2_input_scale = None
        self.use_fp8_w8a8 = False
        self.use_block_quant = config.use_block_quant
        if config.use_block_quant and quantised:
            bn, bk = config.w_quant_block_size
            self.w13_weight_scale = ones(E, 2 * ((I + bn - 1) // bn), (H + bk - 1) // bk, dtype=torch.float16)
            self.w2_weight_scale = ones(E, (H + bn - 1) // bn, (I + bk - 1) // bk, dtype=torch.float16)
            self.block_shape = list(config.w_quant_block_size)
        else:
            self.w13_weight_scale = None
            self.w2_weight_scale = None
            self.block_shape = None

    def forward(self, hidden_states: torch.Tensor, router_logits: Optional[torch.Tensor] = None):
        batch_size, seq_len, _ = hidden_states.shape
        topk_ids, topk_weights = self.gate(hidden_states)
        out = ep_moe_forward(hidden_states.reshape(-1, self.hidden_size), topk_ids.reshape(-1, self.top_k),
                             topk_weights.reshape(-1, self.top_k), self.w13_weight, self.w2_weight,
                             self.w13_weight_scale, self.w2_weight_scale, self.block_shape, self.activation,
                             self.start_expert_id, self.end_expert_id)
        return out.reshape(batch_size, seq_len, self.hidden_size)
