#!/usr/bin/env python3
"""Throughput of the quantized-GEMM path on one MI355X, against its roofline, with a CPU baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--headline-only] [--no-cpu] [--eager]

A "step" is one GEMM call over one batch of synthetic input already resident in HBM.  Small-M
(HBM-bound) workloads rotate through enough distinct weight copies to exceed the 256 MB on-die cache,
so the figure is an HBM figure and not a cache figure.  Rank 0 prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import re
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# published MI355X peaks (dense)
PEAK_HBM_GBS = 8000.0
PEAK_TFLOPS = {"fp8": 5000.0, "int8": 5000.0, "fp16": 2500.0, "bf16": 2500.0}
CACHE_DEFEAT_BYTES = 512 << 20


def _bytes_fp8(M, N, K):
    kb, nb = K // 128, (N + 127) // 128
    return M * K + N * K + 4 * M * kb + 4 * nb * kb + 2 * M * N


def _bytes_i8(M, N, K):
    kb, nb = K // 128, (N + 127) // 128
    return M * K + N * K + 2 * M * kb + 2 * nb * kb + 2 * M * N


def _bytes_i8_pt(M, N, K):
    return M * K + N * K + 4 * M + 4 * N + 2 * M * N


def _bytes_w4a16(M, N, K, g=128):
    return 2 * M * K + N * K // 2 + 2 * N * K // g + 2 * M * N


def _bytes_w4a8(M, N, K):
    kb, nb = K // 128, (N + 127) // 128
    return M * K + N * K // 2 + 2 * M * kb + 2 * nb * kb + 2 * N * kb + 2 * M * N


class CopyCase:
    """Plain device-to-device copy of a known size: the calibration point for the HBM traffic counters."""

    def __init__(self, name, nbytes):
        self.name, self.op, self.M, self.N, self.K = name, "copy", 0, 0, 0
        self.nbytes = nbytes
        self.flops = 0.0
        self.bytes = 2 * nbytes
        self.bound, self.mfma_dtype, self.dtype, self.nbuf = "hbm", "fp8", "u8", 1

    def setup(self, dev):
        src = torch.empty(self.nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        self.launch = lambda i: dst.copy_(src)

    def cpu_seconds(self, max_rows):
        a = torch.empty(self.nbytes, dtype=torch.uint8).random_(0, 255)
        b = torch.empty_like(a)
        b.copy_(a)
        t0 = time.perf_counter()
        b.copy_(a)
        return time.perf_counter() - t0, 0


def _stream_ops():
    """name -> (inputs(dev), device launch(*inputs), oracle pass(*host inputs)) of the streaming operators beside
    the GEMMs: quantisers, dequantisers, the bit packers and the gated activation, at the sizes of the benchmark
    configurations (14336 x 4096 weights, 8192 tokens).  The oracle pass takes the first rows of the host copies."""
    import numpy as np
    from llm_kernels_amd.quantization import fp8_kernel, int8_kernel, w4a8_kernel, bitpack
    from llm_kernels_amd.fast_dequant import w4a16
    from llm_kernels_amd.moe import group_gemm_kernel as gk
    from oracle import quant_ref as q, bitpack_ref as bp, moe_ref
    N, K, T, I = 14336, 4096, 8192, 14336
    act = lambda dev: (torch.randn(T, K, device=dev).bfloat16(),)
    wgt = lambda dev: (torch.randn(N, K, device=dev) * 0.02,)
    nib = lambda dev: (torch.randint(0, 16, (N, K), dtype=torch.uint8, device=dev),)

    def quantised(kernel):
        def make(dev):
            y, s = kernel.weight_quant(torch.randn(N, K, device=dev) * 0.02)
            return y, s
        return make

    def w4a8_packed(dev):
        return w4a8_kernel.weight_quant((torch.randn(N, K, device=dev) * 0.02).half())

    def gate_up(dev):
        ids = torch.sort(torch.randint(0, 8, (T,), dtype=torch.int64, device=dev))[0]
        return torch.randn(T, 2 * I, device=dev).bfloat16(), ids

    def silu(gu, ids):
        out = torch.empty(gu.size(0), gu.size(1) // 2, dtype=gu.dtype, device=gu.device)
        return gk.silu_and_mul(gu, out, gu.size(1), ids, None, 0, 7)

    R = 1024                                           # oracle sample: the first R rows
    return {
        "stream_act_quant_fp8": (act, fp8_kernel.act_quant, lambda x: q.act_quant_fp8(x[:R])),
        "stream_act_quant_int8": (act, int8_kernel.act_quant, lambda x: q.act_quant_int8(x[:R])),
        "stream_act_quant_int8_per_token": (act, int8_kernel.act_quant_per_token, lambda x: q.int8_quant_rowwise(x[:R])),
        "stream_weight_quant_fp8": (wgt, fp8_kernel.weight_quant, lambda w: q.weight_quant_fp8(w[:R])),
        "stream_weight_quant_int8": (wgt, int8_kernel.weight_quant, lambda w: q.weight_quant_int8(w[:R])),
        "stream_weight_dequant_fp8": (quantised(fp8_kernel), fp8_kernel.weight_dequant,
                                      lambda y, s: q.weight_dequant_block(y[:R], s[:R // 128])),
        "stream_weight_dequant_int8": (quantised(int8_kernel), int8_kernel.weight_dequant,
                                       lambda y, s: q.weight_dequant_block(y[:R], s[:R // 128])),
        "stream_weight_dequant_w4a8": (w4a8_packed, w4a8_kernel.weight_dequant,
                                       lambda y, s, s4, z4: q.w4a8_weight_dequant(
                                           torch.from_numpy(bp.unpack_rows(y[:R // 8].numpy(), 4, R)), s[:R // 128], s4[:R], z4[:R])),
        "stream_quantize_w4a16_nk": (lambda dev: (wgt(dev)[0].half(),), lambda w: w4a16.quantize_nk(w, 128),
                                     lambda w: (q.w4a16_quant_nk(w[:R], 128), bp.pack_cols(q.w4a16_quant_nk(w[:R], 128)[0].numpy(), 4, 32))),
        "stream_pack_rows_4in32": (nib, lambda w: bitpack.pack_weights_over_rows(w, 4, 32, False)[0],
                                   lambda w: bp.pack_rows(w[:R].numpy(), 4, 32)),
        "stream_pack_cols_4in32": (nib, lambda w: bitpack.pack_weights_over_cols(w, 4, 32, False)[0],
                                   lambda w: bp.pack_cols(w[:R].numpy(), 4, 32)),
        "stream_unpack_rows_4in32": (lambda dev: (bitpack.pack_weights_over_rows(nib(dev)[0], 4, 32, False)[0],),
                                     lambda p: bitpack.unpack_over_rows(p, 4, N), lambda p: bp.unpack_rows(p[:R // 8].numpy(), 4, R)),
        "stream_unpack_cols_4in32": (lambda dev: (bitpack.pack_weights_over_cols(nib(dev)[0], 4, 32, False)[0],),
                                     lambda p: bitpack.unpack_over_cols(p, 4, K), lambda p: bp.unpack_cols(p[:R].numpy(), 4, K)),
        "stream_silu_and_mul": (gate_up, silu, lambda gu, ids: moe_ref.silu_and_mul(gu[:R], ids[:R], None, 0, 7)),
    }


STREAM_WORKLOADS = ("stream_act_quant_fp8", "stream_act_quant_int8", "stream_act_quant_int8_per_token",
                    "stream_weight_quant_fp8", "stream_weight_quant_int8", "stream_weight_dequant_fp8",
                    "stream_weight_dequant_int8", "stream_weight_dequant_w4a8", "stream_quantize_w4a16_nk",
                    "stream_pack_rows_4in32", "stream_pack_cols_4in32", "stream_unpack_rows_4in32",
                    "stream_unpack_cols_4in32", "stream_silu_and_mul")


def _tensors(v):
    if isinstance(v, torch.Tensor):
        return [v]
    return [t for x in v for t in _tensors(x)] if isinstance(v, (tuple, list)) else []


class StreamCase:
    """One streaming operator (a quantiser, dequantiser, bit packer or the gated activation): every byte is read
    or written once, so the algorithmic bytes are the sizes of the operator's inputs and outputs."""

    def __init__(self, name):
        self.name, self.op, self.M, self.N, self.K, self.flops = name, "stream", 0, 0, 0, 0.0
        self.bound, self.mfma_dtype, self.dtype, self.nbuf, self.bytes = "hbm", "fp8", "u8", 1, 0

    def setup(self, dev):
        make, self.fn, self.oracle = _stream_ops()[self.name]
        torch.manual_seed(0)
        prev = torch.get_default_dtype()
        torch.set_default_dtype(torch.float32)        # the dequantisers return the default dtype: fp32, as the reference's tests run them
        self.inputs = make(dev)
        outs = self.fn(*self.inputs)
        torch.set_default_dtype(prev)
        self.bytes = sum(t.numel() * t.element_size() for t in _tensors(self.inputs) + _tensors(outs))
        del outs

        def launch(i):
            torch.set_default_dtype(torch.float32)
            self.fn(*self.inputs)
            torch.set_default_dtype(prev)
        self.launch = launch

    def cpu_seconds(self, max_rows):
        host = [t.cpu() for t in self.inputs]
        torch.set_default_dtype(torch.float32)
        dt, self.cpu_passes = _timed_passes(lambda: self.oracle(*host), min(CPU_BUDGET_S, 3.0))
        torch.set_default_dtype(torch.bfloat16)
        # the sample is the first 1024 of the operator's rows: scale its bytes by the rows' share
        rows = {"stream_silu_and_mul": 8192, "stream_act_quant_fp8": 8192, "stream_act_quant_int8": 8192,
                "stream_act_quant_int8_per_token": 8192}.get(self.name, 14336)
        self.cpu_bytes = self.bytes * 1024.0 / rows
        return dt, 1024


class MoECase:
    """Mixtral-8x7B shaped expert set on one GPU: permute -> grouped GEMM -> SwiGLU -> grouped GEMM -> un-permute.

    8 experts, hidden 4096, intermediate 14336, fp8 128x128 block-scaled weights, 4096 bf16 tokens,
    softmax top-2 routing.  A step is the whole forward of moe/ep_moe.py (activation quantisation included).
    """

    def __init__(self, name, kind="fp8", T=4096, H=4096, I=14336, E=8, topk=2):
        self.name, self.op, self.kind = name, "moe", kind
        self.T, self.H, self.I, self.E, self.topk = T, H, I, E, topk
        self.M, self.N, self.K = T * topk, 2 * I, H
        rows = T * topk
        self.flops = 2.0 * rows * (2 * I) * H + 2.0 * rows * H * I
        kb1, kb2 = H // 128, I // 128
        self.bytes = (rows * H + E * 2 * I * H + 4 * rows * kb1 + 4 * E * (2 * I // 128) * kb1 + 2 * rows * 2 * I) + \
                     (rows * I + E * H * I + 4 * rows * kb2 + 4 * E * (H // 128) * kb2 + 2 * rows * H)
        # a few tokens per expert: the forward streams every routed expert's weights once (HBM bound)
        self.bound, self.mfma_dtype, self.nbuf = ("hbm" if rows <= 64 * E else "mfma"), ("fp8" if kind == "fp8" else "int8"), 1
        self.dtype = "fp8_e4m3" if kind == "fp8" else "int8"

    def setup(self, dev):
        from llm_kernels_amd.moe.ep_moe import ep_moe_forward, softmax_topk_router
        from llm_kernels_amd.quantization import fp8_kernel, int8_kernel
        torch.manual_seed(0)
        T, H, I, E = self.T, self.H, self.I, self.E
        wq = fp8_kernel.weight_quant if self.kind == "fp8" else int8_kernel.weight_quant
        qdt = torch.float8_e4m3fn if self.kind == "fp8" else torch.int8
        sdt = torch.float32 if self.kind == "fp8" else torch.float16
        w13 = torch.empty(E, 2 * I, H, dtype=qdt, device=dev)
        w13s = torch.empty(E, 2 * I // 128, H // 128, dtype=sdt, device=dev)
        w2 = torch.empty(E, H, I, dtype=qdt, device=dev)
        w2s = torch.empty(E, H // 128, I // 128, dtype=sdt, device=dev)
        for e in range(E):                                    # per expert: bounds the fp32 staging memory
            w13[e], w13s[e] = wq(torch.randn(2 * I, H, device=dev) * 0.02)
            w2[e], w2s[e] = wq(torch.randn(H, I, device=dev) * 0.02)
        x = torch.randn(T, H, device=dev).bfloat16()
        ids, wts = softmax_topk_router(torch.randn(T, E, device=dev), self.topk)
        self.tensors = (x, ids, wts, w13, w2, w13s, w2s)
        self.counts = torch.bincount(ids.flatten(), minlength=E).tolist()
        # experts that no token is routed to are not read: count the weights of the routed ones only
        idle = sum(1 for c in self.counts if c == 0)
        self.bytes -= idle * (2 * I * H + 4 * (2 * I // 128) * (H // 128) + H * I + 4 * (H // 128) * (I // 128))
        self.launch = lambda i: ep_moe_forward(x, ids, wts, w13, w2, w13s, w2s, block_shape=[128, 128])

    def cpu_seconds(self, max_rows):
        """Dense per-expert SwiGLU loop in fp32 on dequantised weights, for the first `max_rows` tokens."""
        import torch.nn.functional as F
        x, ids, wts, w13, w2, w13s, w2s = [t.cpu() for t in self.tensors]
        rows = min(self.T, max_rows)
        x, ids, wts = x[:rows].float(), ids[:rows], wts[:rows].float()

        def deq(w, s):
            wf = w.float() if w.dtype == torch.int8 else w.to(torch.float32)
            return wf * s.float().repeat_interleave(128, 0).repeat_interleave(128, 1)

        def run():
            out = torch.zeros(rows, self.H, dtype=torch.float32)
            for e in range(self.E):
                tok, slot = torch.where(ids == e)
                if tok.numel() == 0:
                    continue
                h = x[tok] @ deq(w13[e], w13s[e]).T
                y = (F.silu(h[:, :self.I]) * h[:, self.I:]) @ deq(w2[e], w2s[e]).T
                out.index_add_(0, tok, y * wts[tok, slot][:, None])
            return out
        dt, self.cpu_passes = _timed_passes(run, CPU_BUDGET_S)
        return dt, rows


CPU_BUDGET_S = 10.0       # the CPU baseline repeats its pass until this much time has gone by
CPU_BUDGET_HEADLINE_S, CPU_BUDGET_OTHER_S = 10.0, 1.5


def _timed_passes(run, budget):
    """One untimed pass, then timed passes until `budget` seconds are used: (seconds per pass, passes)."""
    run()
    total, n = 0.0, 0
    while n == 0 or (total < budget and n < 10000):
        t0 = time.perf_counter()
        run()
        total += time.perf_counter() - t0
        n += 1
    return total / n, n


class Case:
    """One GEMM workload: device buffers (rotated), a launcher, algorithmic cost and a CPU restatement."""

    def __init__(self, name, op, M, N, K):
        self.name, self.op, self.M, self.N, self.K = name, op, M, N, K
        self.flops = 2.0 * M * N * K
        self.bytes = {"fp8": _bytes_fp8, "int8": _bytes_i8, "int8_pt": _bytes_i8_pt, "w4a8": _bytes_w4a8}.get(op, None)
        self.bytes = self.bytes(M, N, K) if self.bytes else _bytes_w4a16(M, N, K)
        self.mfma_dtype = {"fp8": "fp8", "int8": "int8", "int8_pt": "int8", "w4a8": "int8", "w4a16": "fp16", "w4a16_nk": "fp16", "w4a16_nk_bf16": "bf16"}[op]
        intensity = self.flops / self.bytes
        ridge = PEAK_TFLOPS[self.mfma_dtype] * 1e12 / (PEAK_HBM_GBS * 1e9)
        self.bound = "hbm" if intensity < ridge else "mfma"
        self.dtype = {"fp8": "fp8_e4m3", "int8": "int8", "int8_pt": "int8", "w4a8": "int8", "w4a16": "fp16", "w4a16_nk": "fp16", "w4a16_nk_bf16": "bf16"}[op]

    # ---- device side
    def setup(self, dev):
        from llm_kernels_amd.quantization import fp8_kernel, int8_kernel, w4a8_kernel
        from llm_kernels_amd.fast_dequant.simple_marlin.utils import QuantUtils
        from llm_kernels_amd.fast_dequant.simple_marlin.marlin import mul
        from llm_kernels_amd.fast_dequant import w4a16
        M, N, K, op = self.M, self.N, self.K, self.op
        torch.manual_seed(0)
        wbytes = {"fp8": N * K, "int8": N * K, "int8_pt": N * K}.get(op, N * K // 2)
        nbuf = 1 if self.bound == "mfma" else max(2, min(64, -(-CACHE_DEFEAT_BYTES // wbytes)))
        self.nbuf = nbuf
        x = torch.randn(M, K, device=dev)
        w = torch.randn(N, K, device=dev) * 0.02
        self.host = (x.cpu(), w.cpu())
        if op == "fp8":
            a, a_s = fp8_kernel.act_quant(x.bfloat16())
            b, b_s = fp8_kernel.weight_quant(w)
            bs = [b.clone() for _ in range(nbuf)]
            self.launch = lambda i: fp8_kernel.fp8_gemm(a, a_s, bs[i % nbuf], b_s)
        elif op == "int8":
            a, a_s = int8_kernel.act_quant(x.bfloat16())
            b, b_s = int8_kernel.weight_quant(w)
            bs = [b.clone() for _ in range(nbuf)]
            self.launch = lambda i: int8_kernel.int8_gemm(a, a_s, bs[i % nbuf], b_s)
        elif op == "int8_pt":               # per-token x per-channel scales, one int32 accumulation over K
            a, a_s = int8_kernel.act_quant_per_token(x.bfloat16())
            b, b_s = int8_kernel.weight_quant_per_channel(w)
            bs = [b.clone() for _ in range(nbuf)]
            self.launch = lambda i: int8_kernel.int8_gemm_per_token(a, a_s, bs[i % nbuf], b_s)
        elif op == "w4a8":
            a, a_s = w4a8_kernel.act_quant(x.bfloat16())
            b, b_s, s4, z4 = w4a8_kernel.weight_quant(w.half())
            bs = [b.clone() for _ in range(nbuf)]
            self.launch = lambda i: w4a8_kernel.w4a8_gemm(a, a_s, bs[i % nbuf], b_s, s4, z4)
        elif op == "w4a16":
            A = x.half()
            _, q, s = QuantUtils.fake_quantize(w.t().contiguous().half(), 128)
            B, sp = QuantUtils.pack(q, s, 128)
            Bs = [B.clone() for _ in range(nbuf)]
            C = torch.empty(M, N, dtype=torch.half, device=dev)
            ws = torch.zeros(max(16, N // 128 * 16), dtype=torch.int32, device=dev)
            self.launch = lambda i: mul(A, Bs[i % nbuf], C, sp, ws)
        elif op in ("w4a16_nk", "w4a16_nk_bf16"):
            A = x.half() if op == "w4a16_nk" else x.bfloat16()
            packed, s, _ = w4a16.quantize_nk(w, 128)
            Ps = [packed.clone() for _ in range(nbuf)]
            self.launch = lambda i: w4a16.w4a16_gemm(A, Ps[i % nbuf], s, 128)
        else:
            raise ValueError(op)

    # ---- host side: the repo's torch reference semantics (dequantize, then matmul in fp32) on CPU cores
    def cpu_seconds(self, max_rows):
        from oracle import quant_ref, marlin_ref, gemm_ref
        x, w = self.host
        rows = min(self.M, max_rows)
        x = x[:rows]
        op = self.op
        if op == "fp8":
            a, a_s = quant_ref.act_quant_fp8(x.bfloat16())
            b, b_s = quant_ref.weight_quant_fp8(w)

            def run():
                ad = a.float() * a_s.repeat_interleave(128, 1)
                bd = quant_ref.weight_dequant_block(b, b_s)
                return ad @ bd.T
        elif op == "int8_pt":
            xf, wf = x.bfloat16().float(), w.float()
            sa, sb = xf.abs().amax(1) / 127.0, wf.abs().amax(1) / 127.0
            a, b = torch.round(xf / sa[:, None]).to(torch.int8), torch.round(wf / sb[:, None]).to(torch.int8)

            def run():
                return (a.float() * sa[:, None]) @ (b.float() * sb[:, None]).T
        elif op in ("int8", "w4a8"):
            a, a_s = quant_ref.act_quant_int8(x.bfloat16(), rounding="away" if op == "int8" else "up")
            if op == "int8":
                b, b_s = quant_ref.weight_quant_int8(w)
                deq = lambda: quant_ref.weight_dequant_block(b, b_s)
            else:
                qq, s, s4, z4 = quant_ref.w4a8_weight_quant_levels(w)
                deq = lambda: quant_ref.w4a8_weight_dequant(qq, s, s4, z4).float()

            def run():
                ad = a.float() * a_s.float().repeat_interleave(128, 1)
                return ad @ deq().T
        else:
            wk = w.t().contiguous().half()
            _, q, s = marlin_ref.fake_quantize(wk, 128)

            def run():
                return x.half().float() @ gemm_ref.w4a16_dequant_kn(q, s, 128).float()
        dt, self.cpu_passes = _timed_passes(run, CPU_BUDGET_S)
        # the matmul alone, on weights dequantised beforehand (what a CPU deployment that keeps an fp32 copy pays)
        xd, wd = self._cpu_dense(op, x, w)
        self.cpu_matmul_s, _ = _timed_passes(lambda: xd @ wd, min(CPU_BUDGET_S, 1.5))
        return dt, rows

    def _cpu_dense(self, op, x, w):
        """(activations, dequantised weights^T) in fp32 for the matmul-only CPU figure (same operands)."""
        from oracle import quant_ref, marlin_ref, gemm_ref
        if op == "fp8":
            a, a_s = quant_ref.act_quant_fp8(x.bfloat16())
            b, b_s = quant_ref.weight_quant_fp8(w)
            return a.float() * a_s.repeat_interleave(128, 1), quant_ref.weight_dequant_block(b, b_s).T.contiguous()
        if op == "int8_pt":
            xf, wf = x.bfloat16().float(), w.float()
            sa, sb = xf.abs().amax(1) / 127.0, wf.abs().amax(1) / 127.0
            return torch.round(xf / sa[:, None]) * sa[:, None], (torch.round(wf / sb[:, None]) * sb[:, None]).T.contiguous()
        if op in ("int8", "w4a8"):
            a, a_s = quant_ref.act_quant_int8(x.bfloat16(), rounding="away" if op == "int8" else "up")
            ad = a.float() * a_s.float().repeat_interleave(128, 1)
            if op == "int8":
                b, b_s = quant_ref.weight_quant_int8(w)
                return ad, quant_ref.weight_dequant_block(b, b_s).T.contiguous()
            qq, s, s4, z4 = quant_ref.w4a8_weight_quant_levels(w)
            return ad, quant_ref.w4a8_weight_dequant(qq, s, s4, z4).float().T.contiguous()
        _, q, s = marlin_ref.fake_quantize(w.t().contiguous().half(), 128)
        return x.half().float(), gemm_ref.w4a16_dequant_kn(q, s, 128).float()


WORKLOADS = {}
for _op in ("fp8", "w4a16_nk"):                 # Llama-3 lm_head at decode size
    WORKLOADS["%s_m16_n128256_k4096" % _op] = (_op, 16, 128256, 4096)
for _op in ("fp8", "int8", "int8_pt", "w4a8", "w4a16", "w4a16_nk"):
    for _M in (1, 16, 128, 256, 1024, 4096):
        for _N, _K in ((4096, 4096), (6144, 4096), (14336, 4096), (28672, 4096), (4096, 14336)):
            WORKLOADS["%s_m%d_n%d_k%d" % (_op, _M, _N, _K)] = (_op, _M, _N, _K)

# name -> (weight kind, tokens).  16 tokens: the decode-sized forward, bound by streaming the experts' weights.
MOE_WORKLOADS = {"moe_mixtral_fp8_t4096": ("fp8", 4096), "moe_mixtral_int8_t4096": ("int8", 4096),
                 "moe_mixtral_fp8_t16": ("fp8", 16)}
DEFAULT_WORKLOAD = "fp8_m4096_n4096_k4096"
HEADLINE_SET = ["w4a16_m16_n4096_k4096", "w4a16_nk_m16_n4096_k4096", "w4a16_nk_m16_n28672_k4096", "fp8_m16_n4096_k4096", "fp8_m16_n28672_k4096", "fp8_m16_n4096_k14336",
                "fp8_m16_n128256_k4096", "w4a16_nk_m16_n128256_k4096",
                "w4a16_m4096_n4096_k4096", "w4a16_nk_m4096_n4096_k4096", "fp8_m4096_n4096_k4096", "fp8_m4096_n28672_k4096",
                "int8_m4096_n14336_k4096", "int8_pt_m4096_n14336_k4096",
                # the mid-size rows of the benchmark grids (few tiles, cold weights): the weakest points
                "fp8_m256_n4096_k4096", "fp8_m256_n4096_k14336", "int8_pt_m128_n4096_k4096", "w4a16_nk_m128_n4096_k4096",
                "w4a8_m16_n4096_k4096", "w4a8_m128_n4096_k4096", "w4a8_m4096_n4096_k4096",
                "moe_mixtral_fp8_t4096", "moe_mixtral_fp8_t16"]


PREROLL_MS = 150.0        # untimed replays of the captured steps before anything is timed (clock and cache state settle)
TIMED_REPLAYS = 7         # every replay times exactly `steps` steps; the median replay is reported
_flush_buf = None


def _flush_caches(dev):
    """Read and write 1 GiB on the current stream: afterwards neither the L2s nor the 256 MB memory-side cache
    hold any operand of the case, whatever --steps is.  (It also keeps the GPU busy while the host queues the
    timed replay, so the events bracket GPU work only.)"""
    global _flush_buf
    if _flush_buf is None:
        _flush_buf = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
    _flush_buf.add_(1)


def run_case(case, dev, steps, warmup, eager=False):
    """Times exactly `steps` steps, TIMED_REPLAYS times over; returns a dict of timings.

    The steps are captured once into a HIP graph and replayed, so that the timed region is bound by the
    GPU and not by the Python launch path (decode-sized kernels last a few microseconds).  Events are
    recorded on the stream the replay runs on.  Before anything is timed the captured steps are replayed
    for PREROLL_MS, so the first case of a process is not measured on idle clocks.  HBM-bound cases give every
    step of a replay its own copy of the weights where that is possible (steps <= copies; otherwise a copy
    returns only after 512 MB of other copies went by) and every timed replay starts behind a 1 GiB
    read-modify-write, so no step finds its weights in a cache.
    """
    case.setup(dev)
    for i in range(warmup):
        case.launch(i)
    torch.cuda.synchronize()
    graph = None

    def replay():
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                case.launch(warmup + i)

    if not eager:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(steps):
                case.launch(warmup + i)
        graph.replay()                   # first replay uploads the graph
        torch.cuda.synchronize()
    # pre-roll
    t0 = time.perf_counter()
    n_pre = 0
    while n_pre < 2 or (time.perf_counter() - t0) * 1e3 < PREROLL_MS:
        replay()
        n_pre += 1
        if n_pre % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    preroll_ms = (time.perf_counter() - t0) * 1e3
    # wall clock: exactly `steps` steps between two host synchronisations (includes the host-side cost of
    # launching the graph, about 0.2 ms per replay)
    t0 = time.perf_counter()
    replay()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    # HIP events around each timed replay.  The replay is queued behind GPU work that is not waited for (the
    # cache flush for HBM-bound cases, an untimed replay otherwise), so its launch cost hides behind that work.
    cold = case.bound == "hbm"
    ev = []
    for _ in range(TIMED_REPLAYS):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if cold:
            _flush_caches(dev)
        else:
            replay()
        e0.record()
        replay()
        e1.record()
        torch.cuda.synchronize()
        ev.append(e0.elapsed_time(e1))
    ev.sort()
    # HBM-bound cases also without the flush (a replay queued right behind another): what a caller sees whose weights
    # are still in the 256 MB memory-side cache; reported beside the cold figure, never instead of it
    warm = None
    if cold:
        wv = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            replay()
            e0.record()
            replay()
            e1.record()
            torch.cuda.synchronize()
            wv.append(e0.elapsed_time(e1))
        warm = sorted(wv)[1]
    return {"wall": wall, "ev_ms": ev[len(ev) // 2], "ev_ms_min": ev[0], "ev_ms_max": ev[-1],
            "preroll_ms": preroll_ms, "preroll_replays": n_pre, "cold": cold, "warm_ms": warm}


def measured_traffic(workload):
    """HBM bytes per launch from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE runs (profiles/traffic.json)."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(workload, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def record(case, t, steps):
    dur = t["ev_ms"] / 1e3 / steps                  # average launch-to-launch duration from HIP events, median replay
    tflops = case.flops / dur / 1e12
    gbs = case.bytes / dur / 1e9
    if case.bound == "hbm":
        roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": measured_traffic(case.name)}
    else:
        pk = PEAK_TFLOPS[case.mfma_dtype]
        roof = {"bound": "mfma", "achieved": round(tflops, 1), "peak": pk, "unit": "TFLOP/s",
                "frac": round(tflops / pk, 4), "traffic": measured_traffic(case.name)}
    return {"workload": case.name, "M": case.M, "N": case.N, "K": case.K, "us_per_launch": round(dur * 1e6, 2),
            "us_per_launch_min": round(t["ev_ms_min"] * 1e3 / steps, 2), "us_per_launch_max": round(t["ev_ms_max"] * 1e3 / steps, 2),
            "timed_replays": TIMED_REPLAYS, "preroll_ms": round(t["preroll_ms"], 1), "preroll_replays": t["preroll_replays"],
            "cache_flushed_before_each_replay": t["cold"],
            "us_per_launch_without_flush": None if t.get("warm_ms") is None else round(t["warm_ms"] * 1e3 / steps, 2),
            "tflops": round(tflops, 2), "gbs": round(gbs, 1), "alg_bytes": case.bytes, "flops": case.flops,
            "weight_copies_rotated": case.nbuf, "wall_ms_per_step": round(t["wall"] * 1e3 / steps, 4), "roofline": roof}


def cpu_baseline(case, budget):
    """The oracle's dequantize-then-matmul on the host cores for a bounded sample of the case."""
    global CPU_BUDGET_S
    CPU_BUDGET_S = budget
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    max_rows = 512 if case.op == "moe" else 4096       # bounded sample of the same workload
    dt, rows = case.cpu_seconds(max_rows)
    if case.op == "copy":
        return {"value": round(case.bytes / dt / 1e9, 2), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "host memcpy of the same size"}
    if case.op == "stream":
        return {"value": round(case.cpu_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                "cpu_model": _cpu_model(),
                "sample": "the oracle's restatement of the operator on the first %d rows of the same inputs, 1 warm-up + "
                          "%d timed passes of %.4f s each" % (rows, case.cpu_passes, dt)}
    cpu_flops = case.flops * rows / case.T if case.op == "moe" else 2.0 * rows * case.N * case.K
    out = {"value": round(cpu_flops / dt / 1e12, 4), "unit": "TFLOP/s",
           "cores": torch.get_num_threads(), "kind": "port", "cpu_model": _cpu_model(),
           "sample": "torch-CPU dequantize-then-matmul (fp32) of the same operands, first %d of %d rows, "
                     "1 warm-up + %d timed passes of %.3f s each, weight dequantisation included in every pass"
                     % (rows, case.T if case.op == "moe" else case.M, getattr(case, "cpu_passes", 1), dt)}
    mm = getattr(case, "cpu_matmul_s", None)
    if mm:
        out["matmul_only_value"] = round(cpu_flops / mm / 1e12, 4)      # same unit; weights dequantised beforehand
    return out


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or platform.machine()


def calibration(dev):
    """What this box sustains on the two resources the roofline prices against, from the library's calibration
    kernels (llmk_calib_mfma: nothing but matrix instructions on random register operands, eight waves per CU;
    llmk_calib_read: a read without arithmetic, linear and with the decode kernels' addresses, of 1 GiB, four
    times the memory-side cache).  Reported beside the published peaks, never instead of them."""
    from llm_kernels_amd import _lib
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    st = _lib.stream(torch.empty(1, device=dev))
    out = torch.empty(cus * 512, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    res = {"cus": cus}

    def timed(launch, reps=5):
        launch()
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            launch()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e-3)
        return sorted(ts)[len(ts) // 2]

    torch.manual_seed(0)
    iters = 2000
    kinds = (("fp8", _lib.KIND_FP8, 2 * 16 * 16 * 128, (torch.randn(65536, device=dev) * 0.5).to(torch.float8_e4m3fn)),
             ("int8", _lib.KIND_I8, 2 * 16 * 16 * 64, torch.randint(-127, 128, (65536,), dtype=torch.int8, device=dev)),
             ("f16", _lib.KIND_F16, 2 * 16 * 16 * 32, torch.randn(32768, device=dev).half()),
             ("bf16", _lib.KIND_BF16, 2 * 16 * 16 * 32, torch.randn(32768, device=dev).bfloat16()))
    for name, kind, flops_per_mfma, ops in kinds:
        dt_s = timed(lambda: _lib.call("llmk_calib_mfma", kind, iters, _lib.ptr(ops), _lib.ptr(out), cus, _lib.ptr(clocks), st))
        res["mfma_%s_sustained_tflops" % name] = round(cus * 8 * iters * 32 * flops_per_mfma / dt_s / 1e12, 1)
        ck = clocks.tolist()
        if ck[1] > 0:            # s_memtime counts the shader clock, s_memrealtime a constant 100 MHz
            res["shader_clock_mhz_in_mfma_%s_loop" % name] = round(100.0 * ck[0] / ck[1], 0)
    # the shader clock the headline GEMM itself runs at (fp8 4096^3 on random operands, first workgroup's lifetime)
    from llm_kernels_amd.quantization import fp8_kernel
    M = N = K = 4096
    a, a_s = fp8_kernel.act_quant(torch.randn(M, K, device=dev).bfloat16())
    b, b_s = fp8_kernel.weight_quant(torch.randn(N, K, device=dev) * 0.02)
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    wsp, wsn = _lib.gemm_workspace(dev, M, N, K)
    clocks.zero_()
    gemm = lambda: _lib.call("llmk_calib_gemm_fp8_clock", _lib.ptr(a), _lib.ptr(a_s), _lib.ptr(b), _lib.ptr(b_s), _lib.ptr(c),
                             _lib.BF16, M, N, K, wsp, wsn, _lib.ptr(clocks), st)
    for _ in range(50):
        gemm()
    dt_s = timed(gemm, reps=9)
    ck = clocks.tolist()
    if ck[1] > 0:
        res["shader_clock_mhz_in_fp8_gemm_4096"] = round(100.0 * ck[0] / ck[1], 0)
        res["fp8_gemm_4096_workgroup_lifetime_us"] = round(ck[1] / 100.0, 2)
        res["fp8_gemm_4096_eager_us"] = round(dt_s * 1e6, 2)
    del a, a_s, b, b_s, c
    global _flush_buf
    if _flush_buf is None:
        _flush_buf = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    for name, pattern, wgs in (("hbm_read_linear_gbs", 0, cus * 8), ("hbm_read_decode_tiles_gbs", 1, cus)):
        dt_s = timed(lambda: _lib.call("llmk_calib_read", _lib.ptr(_flush_buf), _flush_buf.numel(), pattern, _lib.ptr(sink), wgs, st))
        res[name] = round(_flush_buf.numel() / dt_s / 1e9, 1)
    res["note"] = ("sustained rates of this box by the library's calibration kernels; roofline.peak stays the published "
                   "figure (HBM 8000 GB/s; fp8 / int8 5000, fp16 / bf16 2500 TFLOP/s, which assume the 2400 MHz peak "
                   "engine clock: the shader clocks above are what the chip holds under each load)")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD)
    ap.add_argument("--headline-only", action="store_true", help="skip the other headline shapes (reported under 'cases')")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-calibration", action="store_true", help="skip the sustained-MFMA / HBM-read calibration kernels")
    ap.add_argument("--eager", action="store_true", help="launch every step from Python instead of replaying a HIP graph")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    from llm_kernels_amd import _lib
    _lib.load()                                      # fails loudly if the HIP library is not built
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.set_default_dtype(torch.bfloat16)

    if args.workload == "copy_256m":
        op, M, N, K = "copy", 0, 0, 0
        case = CopyCase(args.workload, 256 << 20)
    elif args.workload in STREAM_WORKLOADS:
        op, M, N, K = "stream", 0, 0, 0
        case = StreamCase(args.workload)
    elif args.workload in MOE_WORKLOADS or re.fullmatch(r"moe_mixtral_(fp8|int8)_t(\d+)", args.workload):
        if args.workload not in MOE_WORKLOADS:          # any other token count of the registered expert layer
            mm = re.fullmatch(r"moe_mixtral_(fp8|int8)_t(\d+)", args.workload)
            MOE_WORKLOADS[args.workload] = (mm.group(1), int(mm.group(2)))
        case = MoECase(args.workload, *MOE_WORKLOADS[args.workload])
        op, M, N, K = "moe", case.M, case.N, case.K
    else:
        if args.workload not in WORKLOADS:
            # any other shape of a known operator, spelt like the registered names: <op>_m<M>_n<N>_k<K>
            m = re.fullmatch(r"(fp8|int8|int8_pt|w4a8|w4a16|w4a16_nk|w4a16_nk_bf16)_m(\d+)_n(\d+)_k(\d+)", args.workload)
            if not m:
                raise SystemExit("unknown workload %r" % args.workload)
            WORKLOADS[args.workload] = (m.group(1), int(m.group(2)), int(m.group(3)), int(m.group(4)))
        op, M, N, K = WORKLOADS[args.workload]
        case = Case(args.workload, op, M, N, K)
    t = run_case(case, dev, args.steps, args.warmup, args.eager)
    rec = record(case, t, args.steps)

    cases = []
    if not args.headline_only and args.workload in WORKLOADS:
        for name in HEADLINE_SET:
            if name == args.workload:
                continue
            c = MoECase(name, *MOE_WORKLOADS[name]) if name in MOE_WORKLOADS else Case(name, *WORKLOADS[name])
            r2 = record(c, run_case(c, dev, args.steps, args.warmup, args.eager), args.steps)
            if not args.no_cpu:
                r2["cpu_baseline"] = cpu_baseline(c, CPU_BUDGET_OTHER_S)
            cases.append(r2)
            del c
            torch.cuda.empty_cache()

    if not args.headline_only and args.workload in STREAM_WORKLOADS:      # the other streaming operators, same method
        for name in STREAM_WORKLOADS:
            if name == args.workload:
                continue
            c = StreamCase(name)
            r2 = record(c, run_case(c, dev, args.steps, args.warmup, args.eager), args.steps)
            if not args.no_cpu:
                r2["cpu_baseline"] = cpu_baseline(c, CPU_BUDGET_OTHER_S)
            cases.append(r2)
            del c
            torch.cuda.empty_cache()

    cpu = None if args.no_cpu else cpu_baseline(case, CPU_BUDGET_HEADLINE_S)
    calib = None if args.no_calibration else calibration(dev)

    out = {
        "metric": "w4a16/fp8 GEMM TFLOPS & % roofline (HBM at M=16, MFMA at M=4096)",
        "value": rec["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(rec["us_per_launch"] / 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": case.dtype, "data": "synthetic",
        "config": {"workload": args.workload, "M": M, "N": N, "K": K, "weight_copies_rotated": case.nbuf,
                   "us_per_launch_hip_events": rec["us_per_launch"], "us_per_launch_min": rec["us_per_launch_min"],
                   "us_per_launch_max": rec["us_per_launch_max"], "timed_replays": TIMED_REPLAYS,
                   "preroll_ms": rec["preroll_ms"], "preroll_replays": rec["preroll_replays"],
                   "cache_flushed_before_each_replay": rec["cache_flushed_before_each_replay"],
                   "wall_ms_per_step": rec["wall_ms_per_step"], "alg_bytes": rec["alg_bytes"],
                   "flops": rec["flops"], "launch": "eager" if args.eager else "hip_graph"},
        "roofline": rec["roofline"], "cpu_baseline": cpu, "calibration": calib,
    }
    if cases:
        out["cases"] = cases
    print(json.dumps(out))


if __name__ == "__main__":
    main()
