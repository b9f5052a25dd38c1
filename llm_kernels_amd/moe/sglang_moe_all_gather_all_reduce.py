"""Module path of the reference's EPMoE (moe/sglang_moe_all_gather_all_reduce.py:162): the class lives in ep_moe.py."""
from .config import Config
from .ep_moe import EPMoE, MoEGate, ep_moe_forward

__all__ = ["EPMoE", "MoEGate", "Config", "ep_moe_forward"]
