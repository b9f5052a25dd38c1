"""W4A16 GEMM entry point `mul` (reference fast_dequant/simple_marlin/test.py:25 ->
marlin_w4a16_gemm.cpp:23-111).  Same argument list and error behaviour (RuntimeError)."""
import torch

try:
    from ... import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib


def mul(A, B, C, s, workspace, thread_k=-1, thread_n=-1, sms=-1, max_par=16):
    """C[M,N] (fp16, written in place) = A[M,K] (fp16) x dequant(B, s).

    B is the int32 [K/16, 2N] tensor and s the permuted fp16 [K/g, N] tensor from QuantUtils.pack;
    groupsize is inferred as K / s.size(0).  `workspace`, `thread_k`, `thread_n`, `sms` and `max_par`
    are accepted and ignored, as in the reference.
    """
    prob_m, prob_k = A.size(0), A.size(1)
    prob_n = C.size(1)
    if prob_m % 16 != 0 or prob_n % 16 != 0 or prob_k % 16 != 0:
        raise RuntimeError(f"Matrix dimensions must be divisible by 16. Got M={prob_m}, N={prob_n}, K={prob_k}")
    if not (A.is_cuda and B.device == A.device and C.device == A.device and s.device == A.device):
        raise RuntimeError("All tensors must be on the same CUDA device")
    if A.dtype != torch.float16 or C.dtype != torch.float16:
        raise RuntimeError("A and C matrices must be of type torch.float16")
    if s.dtype != torch.float16:
        raise RuntimeError("Scale tensor must be of type torch.float16")
    if B.dtype != torch.int32:
        raise RuntimeError("B matrix must be packed INT4 data (torch.int32)")
    if not C.is_contiguous():
        raise RuntimeError("C must be contiguous (the result is written in place)")
    if C.size(0) != prob_m:
        raise RuntimeError("C must have as many rows as A")
    A_c, B_c, s_c = A.contiguous(), B.contiguous(), s.contiguous()
    groupsize = -1
    if s.dim() == 2:
        if s.size(1) != prob_n:
            raise RuntimeError(f"Scale tensor N dimension mismatch: expected {prob_n} but got {s.size(1)}")
        groupsize = prob_k // s.size(0)
        if groupsize == 0 or prob_k % groupsize != 0:
            raise RuntimeError(f"K dimension not divisible by groupsize: K={prob_k}, groupsize={groupsize}")
    if B_c.numel() * 8 != prob_k * prob_n:
        raise RuntimeError("B does not hold K*N packed 4-bit values")
    ws_bytes = _lib.load().llmk_gemm_w4a16_marlin_workspace_bytes(prob_m, prob_n, prob_k)
    ws = _lib.workspace(A.device, ws_bytes) if ws_bytes else None
    _lib.call("llmk_gemm_w4a16_marlin", _lib.ptr(A_c), _lib.ptr(B_c), _lib.ptr(C), _lib.ptr(s_c),
              prob_m, prob_n, prob_k, groupsize, _lib.ptr(ws), ws.numel() if ws is not None else 0,
              _lib.stream(A), exc=RuntimeError)
