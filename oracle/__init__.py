"""CPU oracle for the quantized-GEMM hot path.  TEST INFRASTRUCTURE ONLY.

Everything under ``oracle/`` is a CPU restatement (numpy / torch-CPU) of the
algorithms in Jzz24/LLM_Kernels.  It exists so that the HIP kernels can be
checked on identical inputs.  It is imported only by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``;
the product package ``llm_kernels_amd`` never imports it and has no CPU
fallback.

How each function is pinned (the reference ships no stored golden vectors, so
closed forms, invariants, hand-worked vectors and an independent emulation of
the reference CUDA kernel are used; see ``tests/test_oracle_*.py``):

* bitpack_ref      - closed form sum(nibble_i << i*nbits), hand vectors
                     (1..8 -> 0x87654321), sign-bit word, round trips over
                     every nbits x width x direction.
* quant_ref        - rounding-mode tables (half-away / half-up / half-even),
                     hand-computed groups, |q| bounds, |x - q*s| <= s/2.
* marlin_ref       - the pack permutation is checked against an independent
                     lane-by-lane emulation of the reference kernel's
                     mma.m16n8k16 fragment consumption (marlin_emulate).
* gemm_ref         - blockwise form == dequantize-then-matmul form,
                     unit-scale case == plain integer matmul, brute-force
                     triple loops on tiny shapes.
* moe_ref          - the worked 6-token example in the reference comment
                     (src2dst = [0,6,3,9,1,4,7,10,5,8,2,11]), bincount/cumsum.

Parity unpinned (bit level only; irrelevant at the stated tolerances): the
fp32->e4m3 rounding and the fp32 summation order inside Triton's ``tl.dot``
(the reference has no test for ``fp8_gemm`` and only prints cosine similarity
for ``int8_gemm`` / ``w4a8_gemm``), and whether the reference's compiler
rounds an fp32 product once or twice on its way into an fp16 tensor and which
sign a zero product keeps.  The oracle assumes IEEE round-to-nearest-even
casts, exact fp32 division, every product rounded to fp32 before a cast and
signed zeros kept, which is what torch-CPU does.
"""
