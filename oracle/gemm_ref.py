"""GEMM oracles on CPU (test infrastructure).

Two independent statements of every GEMM are given:
  *_blockwise : the kernel's own formula  C = sum_kb dot_kb * a_s[m,kb] * b_s[n//128,kb]
  *_dequant   : dequantize both operands to fp32/fp64, then one matmul (what the
                reference repo compares against, e.g. int8_kernel.py:286-295)
They must agree (tests/test_oracle_gemm.py); the HIP kernels are checked against
the float64 blockwise form.
"""
import torch

from . import quant_ref


def _expand_a_scale(a_s, K, block=128):
    return a_s.double().repeat_interleave(block, dim=-1)[..., :K]


def _expand_b_scale(b_s, N, K, block=128):
    return b_s.double().repeat_interleave(block, 0)[:N].repeat_interleave(block, 1)[:, :K]


def block_dots(a, b, block=128):
    """Exact per-128-K partial products, float64 [kb, M, N] (exact for int8 and for fp8 blocks)."""
    K = a.shape[-1]
    a2 = a.reshape(-1, K).double()
    b2 = b.double()
    kb = K // block
    return torch.stack([a2[:, i * block:(i + 1) * block] @ b2[:, i * block:(i + 1) * block].T
                        for i in range(kb)])


def gemm_blockwise(a, a_s, b, b_s, block=128):
    """fp8_kernel.py:140-167 / int8_kernel.py:201-230 in float64.

    a [..,K] (int8 or e4m3fn), a_s [..,K/128], b [N,K], b_s [ceil(N/128), K/128].
    """
    K = a.shape[-1]
    N = b.shape[0]
    af = a.float() if a.dtype != torch.int8 else a
    bf = b.float() if b.dtype != torch.int8 else b
    d = block_dots(af, bf, block)                                   # [kb, M, N]
    kb = d.shape[0]
    as2 = a_s.reshape(-1, kb).double()                              # [M, kb]
    bs2 = b_s.double().repeat_interleave(block, 0)[:N]              # [N, kb]
    c = torch.einsum('kmn,mk,nk->mn', d, as2, bs2)
    return c.reshape(*a.shape[:-1], N)


def gemm_dequant(a, a_s, b, b_s, block=128):
    """dequantize-then-matmul in float64."""
    K = a.shape[-1]
    N = b.shape[0]
    ad = a.reshape(-1, K).double() * _expand_a_scale(a_s.reshape(-1, a_s.shape[-1]), K, block)
    bd = b.double() * _expand_b_scale(b_s, N, K, block)
    return (ad @ bd.T).reshape(*a.shape[:-1], N)


def int8_gemm_int32(a, b):
    """Exact int8 x int8 -> int32 full-K product (float64 matmul is exact below 2^53)."""
    K = a.shape[-1]
    return (a.reshape(-1, K).double() @ b.double().T).to(torch.int64).to(torch.int32)


def int8_gemm_rowcol(a, a_s, b, b_s):
    """per-token x per-channel W8A8: C = int32(a b^T) * a_s[m] * b_s[n]."""
    acc = int8_gemm_int32(a, b).double()
    return acc * a_s.double()[:, None] * b_s.double()[None, :]


def w4a8_gemm(a, a_s, q, b_s, b_s4, b_z4, group_size_int4=128, block=128):
    """w4a8_kernel.py:334-404.  q is the unpacked [N,K] 0..15 matrix."""
    b8 = quant_ref.w4a8_dequant_int8(q, b_s4, b_z4, group_size_int4)
    return gemm_blockwise(a, a_s, b8, b_s, block)


def w4a16_dequant_kn(q_kn, s_kn_groups, group_size):
    """(q - 8).half() * s in fp16, [K,N] (simple_marlin/utils.py:125; marlin_w4a16_gemm.cu:44-70)."""
    K, N = q_kn.shape
    if group_size == -1:
        group_size = K
    se = s_kn_groups.repeat_interleave(group_size, 0)[:K]
    return (q_kn.to(torch.int32) - 8).half() * se


def w4a16_gemm(a, q_kn, s, group_size):
    """C = A @ dequant(W) with fp16 weights and float64 accumulation; a [M,K] fp16, q [K,N]."""
    w = w4a16_dequant_kn(q_kn, s, group_size)
    return a.double() @ w.double()


def brute_gemm_blockwise(a, a_s, b, b_s, block=128):
    """Triple python loop; only for tiny shapes (<= 16 x 16 x 256)."""
    M, K = a.shape
    N = b.shape[0]
    out = [[0.0] * N for _ in range(M)]
    al, bl = a.double().tolist(), b.double().tolist()
    asl, bsl = a_s.double().tolist(), b_s.double().tolist()
    for m in range(M):
        for n in range(N):
            tot = 0.0
            for kb in range(K // block):
                d = 0.0
                for k in range(kb * block, (kb + 1) * block):
                    d += al[m][k] * bl[n][k]
                tot += d * asl[m][kb] * bsl[n // block][kb]
            out[m][n] = tot
    return torch.tensor(out, dtype=torch.float64)
