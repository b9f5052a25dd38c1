"""The package directory works as a drop-in for the reference's top-level module layout.

The reference is imported as `quantization.fp8_kernel`, `moe.group_gemm_kernel`, ... with the repository
root on sys.path (e.g. moe/group_gemm_kernel.py:463 `from quantization.int8_kernel import act_quant`,
quantization/w4a8_kernel.py:10 `from quantization.bitpack import pack_weights_over_rows`).  Putting
llm_kernels_amd/ first on sys.path must resolve the same names here.
"""
import os
import subprocess
import sys
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "llm_kernels_amd")

IMPORTS = textwrap.dedent("""
    import sys; sys.path.insert(0, %r)
    from quantization.fp8_kernel import act_quant, weight_dequant, fp8_gemm
    from quantization.int8_kernel import act_quant, weight_quant, weight_dequant, int8_gemm
    from quantization.w4a8_kernel import act_quant, weight_quant, weight_dequant, w4a8_gemm
    from quantization.bitpack import pack_weights_over_rows, pack_weights_over_cols, unpack_over_rows, unpack_over_cols
    from quantization.quant_utils import Int4QuantUtils
    from fast_dequant.simple_marlin.utils import QuantUtils
    from fast_dequant.simple_marlin.marlin import mul
    from fast_dequant.w4a16 import w4a16_gemm, quantize_nk
    from moe.group_gemm_kernel import (run_moe_ep_preproess, grouped_gemm_triton, pre_reorder_triton_kernel,
                                       silu_and_mul_triton_kernel, gelu_and_mul_triton_kernel, post_reorder_triton_kernel)
    from moe.ep_moe import ep_moe_forward
    from moe.sglang_moe_all_gather_all_reduce import EPMoE
    from moe.config import Config
    from quant_communication.quant_utils import int8_quant, int8_dequant, fp8_quant, fp8_dequant
    from fast_dequant.fast_dtype_convert import uint4_to_fp16, uint8_to_fp16, uint8_to_bf16, mma_fp16
    import quantization.fp8_kernel as m
    assert m.__file__.startswith(%r), m.__file__
""") % (PKG, PKG)


def _run(code):
    # a fresh interpreter started outside the repository: nothing but the inserted path can resolve the names
    return subprocess.run([sys.executable, "-c", code], cwd="/tmp", capture_output=True, text=True, timeout=300)


def test_top_level_module_layout_imports_in_a_fresh_process():
    r = _run(IMPORTS + "print('imports ok')")
    assert r.returncode == 0 and "imports ok" in r.stdout, r.stderr


@pytest.mark.gpu
def test_ops_run_through_the_top_level_module_layout(dev):
    code = IMPORTS + textwrap.dedent("""
        import torch
        torch.manual_seed(0)
        torch.set_default_dtype(torch.bfloat16)
        x = torch.randn(16, 512, device="cuda").bfloat16()
        a, a_s = m.act_quant(x)
        w = torch.randn(256, 512, device="cuda", dtype=torch.float32) * 0.02
        b, b_s = m.weight_quant(w)
        c = fp8_gemm(a, a_s, b, b_s)
        ref = x.float() @ w.t()
        cos = torch.nn.functional.cosine_similarity(c.float().flatten(), ref.flatten(), dim=0).item()
        assert c.dtype == torch.bfloat16 and cos > 0.998, cos
        # the grouped GEMM quantises through `quantization.int8_kernel` exactly as the reference's import does
        wi = torch.randint(-127, 128, (2, 256, 512), device="cuda", dtype=torch.int8)
        ws = torch.full((2, 2, 4), 0.01, device="cuda", dtype=torch.float16)
        out = torch.zeros(16, 256, device="cuda", dtype=torch.bfloat16)
        seg = torch.tensor([0, 10, 16], device="cuda", dtype=torch.int64)
        grouped_gemm_triton(x, wi, out, 2, True, seg, torch.arange(2, device="cuda"), False, None, ws, [128, 128])
        want = torch.cat([x[:10].float() @ (wi[0].float() * 0.01).t(), x[10:].float() @ (wi[1].float() * 0.01).t()])
        cos = torch.nn.functional.cosine_similarity(out.float().flatten(), want.flatten(), dim=0).item()
        assert cos > 0.999, cos
        print('ops ok')
    """)
    r = _run(code)
    assert r.returncode == 0 and "ops ok" in r.stdout, r.stderr[-2000:]
