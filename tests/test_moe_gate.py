"""The router and module shell around the expert forward (CPU): MoEGate against the loop oracle, the oracle against
hand-computed cases, and the parameter shapes / dtypes of EPMoE against the reference's
(moe/sglang_moe_all_gather_all_reduce.py:218-259)."""
import math

import pytest
import torch

from oracle import moe_ref as m
from llm_kernels_amd.moe.config import Config
from llm_kernels_amd.moe.ep_moe import EPMoE, MoEGate


def _logit(p):
    return math.log(p / (1 - p))


def test_gate_oracle_hand_cases():
    """scores 0.9 0.1 | 0.5 0.6 in two groups: the group sums are 1.0 and 1.1, so with one group allowed the token goes
    to experts 2 and 3 although expert 0 has the best score; a bias of 0.3 on expert 1 lifts the first group to 1.3
    and the token goes to experts 0 and 1, weighted by the scores without the bias."""
    x = torch.tensor([[_logit(0.9), _logit(0.1), _logit(0.5), _logit(0.6)]])
    w = torch.eye(4)
    ids, wt = m.deepseek_gate(x, w, torch.zeros(4), top_k=2, n_group=2, topk_group=1, routed_scaling_factor=2.5)
    assert ids == [{2, 3}]
    assert wt[0][2] == pytest.approx(2.5 * 0.5 / 1.1) and wt[0][3] == pytest.approx(2.5 * 0.6 / 1.1)
    ids, wt = m.deepseek_gate(x, w, torch.tensor([0.0, 0.3, 0.0, 0.0]), top_k=2, n_group=2, topk_group=1)
    assert ids == [{0, 1}]
    assert wt[0][0] == pytest.approx(0.9) and wt[0][1] == pytest.approx(0.1)
    # without normalisation the weights are the raw scores times the factor
    ids, wt = m.deepseek_gate(x, w, torch.zeros(4), top_k=2, n_group=2, topk_group=2, norm_topk_prob=False,
                              routed_scaling_factor=2.0)
    assert ids == [{0, 3}] and wt[0][0] == pytest.approx(1.8) and wt[0][3] == pytest.approx(1.2)


@pytest.mark.parametrize("E,G,TG,K", [(16, 4, 2, 4), (8, 1, 1, 2), (256, 8, 4, 8), (12, 3, 3, 1)])
def test_gate_module_equals_oracle(E, G, TG, K):
    torch.manual_seed(E + K)
    cfg = Config(hidden_size=32, n_routed_experts=E, num_experts_per_tok=K, n_group=G, topk_group=TG,
                 routed_scaling_factor=2.5)
    gate = MoEGate(cfg).eval()
    with torch.no_grad():
        gate.weight.normal_(0, 0.5)
        gate.e_score_correction_bias.uniform_(-0.1, 0.1)
        x = torch.randn(2, 9, 32)
        ids, w = gate(x)
    assert ids.shape == (18, K) and w.shape == (18, K) and w.dtype == torch.float32
    oids, ow = m.deepseek_gate(x, gate.weight.detach(), gate.e_score_correction_bias.detach(), K, G, TG, True, 2.5)
    for t in range(18):
        assert set(ids[t].tolist()) == oids[t]
        for j in range(K):
            assert float(w[t, j]) == pytest.approx(ow[t][int(ids[t, j])], rel=1e-5)


def test_gate_rejects_other_methods():
    with pytest.raises(NotImplementedError):
        MoEGate(Config(hidden_size=8, n_routed_experts=4, n_group=1, topk_group=1, scoring_func="softmax")).eval()(torch.zeros(1, 1, 8))
    with pytest.raises(NotImplementedError):
        MoEGate(Config(hidden_size=8, n_routed_experts=4, n_group=1, topk_group=1, topk_method="greedy")).eval()(torch.zeros(1, 1, 8))


def test_epmoe_parameters():
    cfg = Config(hidden_size=256, moe_intermediate_size=384, n_routed_experts=8, num_experts_per_tok=2, n_group=2, topk_group=1)
    mod = EPMoE(cfg)
    assert mod.w13_weight.shape == (8, 768, 256) and mod.w13_weight.dtype == torch.int8
    assert mod.w2_weight.shape == (8, 256, 384) and mod.w2_weight.dtype == torch.int8
    assert mod.w13_weight_scale.shape == (8, 6, 2) and mod.w13_weight_scale.dtype == torch.float16
    assert mod.w2_weight_scale.shape == (8, 2, 3) and mod.block_shape == [128, 128]
    assert (mod.start_expert_id, mod.end_expert_id, mod.num_experts_per_partition) == (0, 7, 8)
    assert not any(p.requires_grad for n, p in mod.named_parameters() if not n.startswith("gate."))
    plain = EPMoE(Config(hidden_size=64, moe_intermediate_size=128, n_routed_experts=4, num_experts_per_tok=2, n_group=1,
                         topk_group=1, quantize_method=None))
    assert plain.w13_weight.dtype == torch.get_default_dtype() and plain.w13_weight_scale is None and plain.block_shape is None
    fp8 = EPMoE(Config(hidden_size=128, moe_intermediate_size=128, n_routed_experts=2, num_experts_per_tok=1, n_group=1,
                       topk_group=1, quantize_method="blockwise_w8a8_fp8_gemm", w_dtype=torch.float8_e4m3fn))
    assert fp8.w2_weight.dtype == torch.float8_e4m3fn
    with pytest.raises(NotImplementedError):
        EPMoE(Config(ep_size=2))
