"""W4A16 GEMM for weights kept in the plain [N, K] bit-packed layout.

W [N, K] is quantised symmetrically along K in groups (s = absmax / 7, q = clamp(rne(w / s), -8, 7) + 8)
and stored with quantization.bitpack.pack_weights_over_cols as int32 [N, K/8] (nibble i of a word is
k = 8*word + i).  The simple-Marlin layout has its own entry point (simple_marlin.marlin.mul).
"""
import torch

try:
    from .. import _lib
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib


def quantize_nk(w: torch.Tensor, group_size: int = 128):
    """W [N, K] float -> (packed int32 [N, K/8], scales fp16 [N, K/group_size], q uint8 [N, K]).

    One pass over W on the GPU: s = absmax / 7 rounded to fp16, q = clamp(rne(w / s), -8, 7) + 8 with the
    quotient by the rounded scale in fp32, nibble i of a packed word is k = 8 * word + i (the layout of
    quantization.bitpack.pack_weights_over_cols(q, 4, 32, transpose=False))."""
    assert w.dim() == 2 and w.shape[1] % group_size == 0
    assert w.dtype in (torch.float32, torch.float16, torch.bfloat16), 'weights must be fp32, fp16 or bf16'
    _lib.require_gpu(w)
    w = w.contiguous()
    N, K = w.shape
    packed = torch.empty(N, K // 8, dtype=torch.int32, device=w.device)
    s = torch.empty(N, K // group_size, dtype=torch.float16, device=w.device)
    q = torch.empty(N, K, dtype=torch.uint8, device=w.device)
    _lib.call("llmk_quant_w4_nk", _lib.ptr(w), _lib.dt(w.dtype), _lib.ptr(packed), _lib.ptr(s), _lib.ptr(q),
              N, K, group_size, _lib.stream(w), exc=AssertionError)
    return packed, s, q


def w4a16_gemm(x: torch.Tensor, w_packed: torch.Tensor, scales: torch.Tensor, group_size: int = 128):
    """y[..., n] = sum_k x[..., k] * (nibble(n, k) - 8) * scales[n, k // group_size]; fp16 or bf16 in / out
    (the dtype of x), fp16 scales."""
    assert x.is_contiguous() and w_packed.is_contiguous() and scales.is_contiguous(), 'Input tensors must be contiguous'
    assert w_packed.dtype == torch.int32 and scales.dtype == torch.float16
    _lib.require_gpu(x, w_packed, scales)
    K = x.size(-1)
    M = x.numel() // K
    N = w_packed.size(0)
    assert w_packed.size(1) * 8 == K, 'packed weight must be [N, K/8]'
    y = x.new_empty(*x.size()[:-1], N)
    assert x.dtype in (torch.float16, torch.bfloat16), 'activations must be fp16 or bf16'
    # bf16 at decode size runs on the weight-streaming ring kernel under exactly the conditions the library
    # checks (128-wide groups, K ranges of at most 32 steps in whole four-step shares, 8-byte aligned scale rows
    # and outputs, 32-bit lane offsets, and with more than one K range M * N % 4 == 0 for the summing pass);
    # every other bf16 call goes through the bf16 copy of W and needs room for it
    steps = K // 128
    nz = max(1, -(-steps // 32))
    per = -(-steps // nz)
    ring_ok = (group_size == 128 and per <= 32 and steps % 4 == 0 and per % 4 == 0 and scales.data_ptr() % 8 == 0
               and N * (K // 2) < (1 << 32) and M * K * 2 < (1 << 32))
    bf_decode = (x.dtype == torch.bfloat16 and M <= 64 and ring_ok and y.data_ptr() % 8 == 0
                 and (nz == 1 or (M * N) % 4 == 0))
    if M > 64 or (x.dtype == torch.bfloat16 and not bf_decode):
        # fp16 / bf16 copy of W for the compute-bound path, split-K partials behind it for mid-size M
        ws = _lib.workspace(x.device, ((N * K * 2 + 255) // 256) * 256 + (8 * M * N * 4 if M <= 512 else 0))
    elif K > 4096 or M > 16:
        ws = _lib.workspace(x.device, max(8, -(-K // 4096)) * M * N * 4)   # fp32 partial sums of K ranges / K slices
    else:
        ws = None
    _lib.call("llmk_gemm_w4a16_nk", _lib.ptr(x), _lib.ptr(w_packed), _lib.ptr(y), _lib.ptr(scales),
              _lib.dt(x.dtype), M, N, K, group_size, _lib.ptr(ws), ws.numel() if ws is not None else 0,
              _lib.stream(x), exc=AssertionError)
    return y
