"""Attribute bag read by MoEGate and EPMoE: the field names of the reference's Config (moe/config.py:3-30).

The defaults are the reference's (DeepSeek-V3 routed experts, block-wise int8 weights); every field can be
overridden by keyword, e.g. Config(hidden_size=4096, n_routed_experts=8, num_experts_per_tok=2, n_group=1,
topk_group=1, moe_intermediate_size=14336, quantize_method="blockwise_w8a8_fp8_gemm",
w_dtype=torch.float8_e4m3fn) for the Mixtral expert layer of the benchmark.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass
class Config:
    # model
    hidden_size: int = 7168
    intermediate_size: int = 18432
    moe_intermediate_size: int = 2048
    n_routed_experts: int = 256
    n_shared_experts: int = 0
    num_experts_per_tok: int = 8
    hidden_act: str = "silu"
    # gate
    scoring_func: str = "sigmoid"
    topk_method: str = "noaux_tc"
    n_group: int = 8
    topk_group: int = 4
    norm_topk_prob: bool = True
    routed_scaling_factor: float = 2.5
    seq_aux: bool = True
    # deployment
    ep_size: int = 1
    use_triton_group_gemm: bool = False
    # quantisation (quantize_method None: 16-bit weights)
    quantize_method: Optional[str] = "blockwise_w8a8_int8_gemm"
    use_block_quant: bool = True
    w_quant_block_size: Tuple[int, int] = (128, 128)
    a_quant_block_size: Tuple[int, int] = (1, 128)
    w_bit: int = 8
    a_bit: int = 8
    w_dtype: torch.dtype = torch.int8
    a_dtype: torch.dtype = torch.int8
