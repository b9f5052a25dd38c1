"""ctypes binding of libllmk_gfx950.so (the C ABI declared in include/llmk.h).

There is no CPU or PyTorch fallback: if the library is missing, or a tensor is
not on a HIP device, the call raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("LLMK_LIB", os.path.join(_HERE, "libllmk_gfx950.so"))

F32, F16, BF16 = 0, 1, 2
ROUND_HALF_AWAY, ROUND_HALF_UP = 0, 1
KIND_I8, KIND_FP8, KIND_F16, KIND_BF16 = 0, 1, 2, 3

_DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

_c = ctypes
_p, _i, _l, _f = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float

# name -> argument types (return type is int unless listed in _RESTYPE)
SIGNATURES = {
    "llmk_version": [],
    "llmk_last_error": [],
    "llmk_gemm_workspace_bytes": [_l, _l, _l],
    "llmk_pack_rows": [_p, _i, _p, _l, _l, _i, _i, _p],
    "llmk_pack_cols": [_p, _i, _p, _l, _l, _i, _i, _p],
    "llmk_unpack_rows": [_p, _i, _p, _i, _l, _l, _i, _i, _p],
    "llmk_unpack_cols": [_p, _i, _p, _i, _l, _l, _i, _i, _p],
    "llmk_act_quant_fp8": [_p, _i, _p, _p, _l, _i, _p],
    "llmk_act_quant_i8": [_p, _i, _p, _p, _l, _i, _i, _p],
    "llmk_quant_i8_rowwise": [_p, _i, _p, _p, _l, _l, _p],
    "llmk_weight_quant_i8_block": [_p, _i, _p, _p, _l, _l, _i, _f, _i, _i, _p],
    "llmk_weight_quant_fp8_block": [_p, _i, _p, _p, _l, _l, _i, _p],
    "llmk_quant_w4_nk": [_p, _i, _p, _p, _p, _l, _l, _i, _p],
    "llmk_weight_quant_w4a8_level2": [_p, _p, _p, _l, _l, _i, _p],
    "llmk_weight_dequant_fp8_block": [_p, _p, _p, _i, _l, _l, _i, _p],
    "llmk_weight_dequant_i8_block": [_p, _p, _i, _p, _i, _l, _l, _i, _p],
    "llmk_weight_dequant_w4a8": [_p, _p, _p, _p, _p, _l, _l, _i, _i, _p],
    "llmk_gemm_fp8_block": [_p, _p, _p, _p, _p, _i, _l, _l, _l, _p, _l, _p],
    "llmk_gemm_fp8_block_static": [_p, _p, _p, _p, _p, _i, _l, _l, _l, _p],
    "llmk_gemm_i8_block": [_p, _p, _p, _p, _i, _p, _i, _l, _l, _l, _p, _l, _p],
    "llmk_gemm_i8_rowcol": [_p, _p, _p, _p, _p, _i, _p, _l, _l, _l, _p, _l, _p],
    "llmk_gemm_w4a8": [_p, _p, _p, _p, _i, _p, _p, _p, _i, _l, _l, _l, _i, _p, _l, _p],
    "llmk_gemm_w4a8_workspace_bytes": [_l, _l, _l, _i],
    "llmk_gemm_w4a16_marlin_workspace_bytes": [_l, _l, _l],
    "llmk_gemm_w4a16_marlin": [_p, _p, _p, _p, _l, _l, _l, _i, _p, _l, _p],
    "llmk_gemm_w4a16_nk": [_p, _p, _p, _p, _i, _l, _l, _l, _i, _p, _l, _p],
    "llmk_convert_u4_to_f16": [_p, _p, _l, _p],
    "llmk_convert_u8_to_f16": [_p, _p, _l, _p],
    "llmk_convert_u8_to_bf16": [_p, _p, _l, _p],
    "llmk_gemm_f16_simple": [_p, _p, _p, _l, _l, _l, _p],
    "llmk_comm_quant_fp8": [_p, _i, _p, _p, _i, _l, _i, _p],
    "llmk_comm_dequant": [_p, _i, _p, _i, _p, _i, _l, _i, _p],
    "llmk_moe_seg_indptr": [_p, _p, _l, _i, _p],
    "llmk_moe_src2dst": [_p, _p, _l, _p],
    "llmk_moe_ep_preprocess": [_p, _i, _l, _i, _p, _p, _p, _p],
    "llmk_moe_pre_reorder": [_p, _i, _p, _i, _p, _p, _i, _p, _i, _i, _i, _l, _l, _p],
    "llmk_moe_act_and_mul": [_p, _i, _p, _i, _p, _i, _p, _i, _i, _l, _l, _i, _p],
    "llmk_moe_act_and_mul_quant": [_p, _i, _p, _p, _i, _i, _p, _i, _p, _i, _i, _l, _l, _i, _p],
    "llmk_grouped_gemm_swiglu_quant_fused": [_i, _i, _l, _l, _l],
    "llmk_grouped_gemm_swiglu_quant": [_p, _p, _p, _p, _i, _i, _i, _i, _l, _l, _l, _p, _p, _p, _p, _i, _i, _p, _l, _p],
    "llmk_moe_pre_reorder_quant": [_p, _i, _p, _p, _i, _i, _p, _p, _i, _p, _i, _i, _i, _l, _l, _p],
    "llmk_moe_post_reorder": [_p, _p, _i, _p, _p, _i, _p, _i, _i, _i, _i, _l, _l, _p],
    "llmk_moe_expert_scales": [_p, _p, _p, _i, _i, _l, _l, _l, _p, _p, _i, _p],
    "llmk_calib_mfma": [_i, _i, _p, _p, _i, _p, _p],
    "llmk_calib_read": [_p, _l, _i, _p, _i, _p],
    "llmk_calib_gemm_fp8_clock": [_p, _p, _p, _p, _p, _i, _l, _l, _l, _p, _l, _p, _p],
    "llmk_grouped_gemm": [_p, _p, _p, _i, _i, _i, _l, _l, _l, _p, _p, _p, _p, _i, _p, _l, _p],
}
_RESTYPE = {"llmk_last_error": _c.c_char_p, "llmk_gemm_workspace_bytes": _l, "llmk_gemm_w4a8_workspace_bytes": _l,
            "llmk_gemm_w4a16_marlin_workspace_bytes": _l}

_lib = None


class LlmkError(RuntimeError):
    pass


def load():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LlmkError(
            "libllmk_gfx950.so is not built (%s). Run `python -m llm_kernels_amd.build`; "
            "there is no fallback implementation." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is missing
        fn.argtypes = args
        fn.restype = _RESTYPE.get(name, _i)
    _lib = lib
    return lib


def dt(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise TypeError("unsupported floating dtype %s (need float32/float16/bfloat16)" % dtype)


def ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def stream(t: torch.Tensor):
    require_gpu(t)
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise LlmkError("llm_kernels_amd kernels run on a HIP device only; got a %s tensor "
                            "(no CPU fallback exists)" % t.device)


def call(name, *args, exc=LlmkError):
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.llmk_last_error()
        raise exc("%s failed (rc=%d): %s" % (name, rc, msg.decode() if msg else ""))
    return rc


def gemm_workspace(device, M, N, K):
    """(pointer, nbytes) of the optional GEMM scratch for this shape, (None, 0) when none is needed."""
    n = load().llmk_gemm_workspace_bytes(M, N, K)
    if n <= 0:
        return None, 0
    buf = workspace(device, n)
    # the size asked for, not the size of the cached buffer: what a kernel does with its scratch (K splits) then
    # depends on the shape alone, never on what an earlier call left behind
    return ptr(buf), int(n)


_ws = {}


def workspace(device, nbytes):
    """Per (device, stream) scratch buffer, grown on demand.  Calls issued on one stream are
    ordered, so sharing the buffer between consecutive launches on that stream is safe."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _ws.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _ws[key] = buf
    return buf


def release_workspaces(device=None):
    """Drops the cached scratch buffers (of one device, or of all): the next call that needs scratch allocates
    again.  The memory goes back to torch's allocator once the launches that use it have run (stream-ordered)."""
    index = None
    if device is not None:
        index = torch.device(device).index
        if index is None:                      # "cuda" without an ordinal: the current device
            index = torch.cuda.current_device()
    for key in [k for k in _ws if index is None or k[0] == index]:
        del _ws[key]
