"""bench.py's table of streaming-operator workloads: names and oracle passes (host side only, no GPU)."""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench
from oracle import quant_ref as q, bitpack_ref as bp


def test_stream_workload_table_is_complete():
    ops = bench._stream_ops()
    assert set(ops) == set(bench.STREAM_WORKLOADS) and len(bench.STREAM_WORKLOADS) == len(set(bench.STREAM_WORKLOADS))
    assert all(name.startswith("stream_") for name in ops)
    assert not set(ops) & (set(bench.WORKLOADS) | set(bench.MOE_WORKLOADS))


def test_stream_workload_oracle_passes_run_on_host_inputs():
    """Every oracle pass of the table accepts host tensors shaped like its operator's device inputs (2048 rows
    here; the pass itself takes the first 1024)."""
    torch.manual_seed(0)
    ops = bench._stream_ops()
    N, K = 2048, 512
    x, w = torch.randn(N, K).bfloat16(), torch.randn(N, K) * 0.02
    nib = torch.randint(0, 16, (N, K), dtype=torch.uint8)
    yf, sf = q.weight_quant_fp8(w)
    yi, si = q.weight_quant_int8(w)
    qq, s, s4, z4 = q.w4a8_weight_quant_levels(w.half())
    as_t = lambda a: torch.from_numpy(a)
    host = {
        "stream_act_quant_fp8": (x,), "stream_act_quant_int8": (x,), "stream_act_quant_int8_per_token": (x,),
        "stream_weight_quant_fp8": (w,), "stream_weight_quant_int8": (w,),
        "stream_weight_dequant_fp8": (yf, sf), "stream_weight_dequant_int8": (yi, si),
        "stream_weight_dequant_w4a8": (as_t(bp.pack_rows(qq.numpy(), 4, 32)[0]), s, s4, z4),
        "stream_quantize_w4a16_nk": (w.half(),),
        "stream_pack_rows_4in32": (nib,), "stream_pack_cols_4in32": (nib,),
        "stream_unpack_rows_4in32": (as_t(bp.pack_rows(nib.numpy(), 4, 32)[0]),),
        "stream_unpack_cols_4in32": (as_t(bp.pack_cols(nib.numpy(), 4, 32)[0]),),
        "stream_silu_and_mul": (torch.randn(N, 256).bfloat16(), torch.sort(torch.randint(0, 8, (N,)))[0]),
    }
    assert set(host) == set(ops)
    for name, args in host.items():
        assert ops[name][2](*args) is not None, name
