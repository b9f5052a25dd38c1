"""EP-MoE device ops on MI355X (reference moe/group_gemm_kernel.py).

run_moe_ep_preproess (:48), grouped_gemm_triton (:442) keep their names and signatures.  The four
Triton kernels of the reference (pre_reorder :81, silu_and_mul :120, gelu_and_mul :176,
post_reorder :238) are exposed twice: as plain functions, and as `*_triton_kernel` objects that
accept the reference's `kernel[grid](args..., BLOCK_SIZE=...)` call form, so that a caller written
against the reference runs unchanged.
"""
from typing import List, Optional

import torch

try:
    from .. import _lib
    from ..quantization import fp8_kernel as _fp8_kernel, int8_kernel as _int8_kernel
except ImportError:  # this directory itself is on sys.path (the reference's top-level module layout)
    import _lib
    from quantization import fp8_kernel as _fp8_kernel, int8_kernel as _int8_kernel


def _cdiv(a, b):
    return (a + b - 1) // b


# limits of the one-workgroup sort behind llmk_moe_ep_preprocess (LLMK_MOE_PREPROCESS_MAX_* of the C header)
PREPROCESS_MAX_IDS = 32768
PREPROCESS_MAX_EXPERTS = 512


def run_moe_ep_preproess(topk_ids: torch.Tensor, num_experts: int):
    """Stable sort of the flattened expert ids -> (sorted ids, src2dst int32 [T*topk], seg_indptr int64 [E+1])."""
    _lib.require_gpu(topk_ids)
    n = topk_ids.numel()
    st = _lib.stream(topk_ids)
    if (n <= PREPROCESS_MAX_IDS and num_experts <= PREPROCESS_MAX_EXPERTS and topk_ids.is_contiguous()
            and topk_ids.dtype in (torch.int32, torch.int64)):
        # the id counts of one forward pass: one launch instead of the eight of sort + pointers + map
        reorder_topk_ids = torch.empty(n, device=topk_ids.device, dtype=topk_ids.dtype)
        seg_indptr = torch.empty(num_experts + 1, device=topk_ids.device, dtype=torch.int64)
        src2dst = torch.empty(n, device=topk_ids.device, dtype=torch.int32)
        _lib.call("llmk_moe_ep_preprocess", _lib.ptr(topk_ids), _ids_bytes(topk_ids), n, int(num_experts),
                  _lib.ptr(reorder_topk_ids), _lib.ptr(src2dst), _lib.ptr(seg_indptr), st)
        return reorder_topk_ids, src2dst, seg_indptr
    reorder_topk_ids, reorder_ids = torch.sort(topk_ids.view(-1), stable=True)
    seg_indptr = torch.zeros(num_experts + 1, device=topk_ids.device, dtype=torch.int64)
    src2dst = torch.empty(n, device=topk_ids.device, dtype=torch.int32)
    sorted64 = reorder_topk_ids if reorder_topk_ids.dtype == torch.int64 else reorder_topk_ids.to(torch.int64)
    _lib.call("llmk_moe_seg_indptr", _lib.ptr(sorted64), _lib.ptr(seg_indptr), n, num_experts, st)
    _lib.call("llmk_moe_src2dst", _lib.ptr(reorder_ids), _lib.ptr(src2dst), n, st)
    return reorder_topk_ids, src2dst, seg_indptr


def _ids_bytes(t):
    if t.dtype == torch.int64:
        return 8
    if t.dtype == torch.int32:
        return 4
    raise TypeError("expert id tensors must be int32 or int64, got %s" % t.dtype)


def _f32_or_none(t):
    return None if t is None else t.float().contiguous()


def pre_reorder(input, gateup_input, src2dst, topk_ids, a1_scales, start_expert_id, end_expert_id, topk,
                hidden_size):
    """gateup_input[src2dst[t, j]] = input[t] * (1 / a1_scales[e] or 1) for every local expert e of token t."""
    _lib.require_gpu(input, gateup_input, src2dst, topk_ids)
    assert input.is_contiguous() and gateup_input.is_contiguous() and src2dst.is_contiguous() and topk_ids.is_contiguous()
    sc = _f32_or_none(a1_scales)
    T = input.numel() // hidden_size
    _lib.call("llmk_moe_pre_reorder", _lib.ptr(input), _lib.dt(input.dtype), _lib.ptr(gateup_input),
              _lib.dt(gateup_input.dtype), _lib.ptr(src2dst), _lib.ptr(topk_ids), _ids_bytes(topk_ids), _lib.ptr(sc),
              int(start_expert_id), int(end_expert_id), int(topk), T, int(hidden_size), _lib.stream(input))
    return gateup_input


def _act_and_mul(act, gateup_output, down_input, hidden_size, reorder_topk_ids, scales, start_expert_id,
                 end_expert_id):
    _lib.require_gpu(gateup_output, down_input, reorder_topk_ids)
    assert gateup_output.is_contiguous() and down_input.is_contiguous() and reorder_topk_ids.is_contiguous()
    sc = _f32_or_none(scales)
    M = gateup_output.numel() // hidden_size
    _lib.call("llmk_moe_act_and_mul", _lib.ptr(gateup_output), _lib.dt(gateup_output.dtype), _lib.ptr(down_input),
              _lib.dt(down_input.dtype), _lib.ptr(reorder_topk_ids), _ids_bytes(reorder_topk_ids), _lib.ptr(sc),
              int(start_expert_id), int(end_expert_id), M, int(hidden_size), act, _lib.stream(gateup_output))
    return down_input


def silu_and_mul(gateup_output, down_input, hidden_size, reorder_topk_ids, scales, start_expert_id, end_expert_id):
    """down_input[r] = dtype(silu_fp32(gate)) * up * (1/scale[e]); gate = cols [0, I), up = [I, 2I)."""
    return _act_and_mul(0, gateup_output, down_input, hidden_size, reorder_topk_ids, scales, start_expert_id,
                        end_expert_id)


def gelu_and_mul(gateup_output, down_input, hidden_size, reorder_topk_ids, scales, start_expert_id, end_expert_id):
    return _act_and_mul(1, gateup_output, down_input, hidden_size, reorder_topk_ids, scales, start_expert_id,
                        end_expert_id)


def post_reorder(down_output, output, src2dst, topk_ids, topk_weights, start_expert_id, end_expert_id, topk,
                 hidden_size):
    """output[t] = sum_j down_output[src2dst[t, j]] * dtype(topk_weights[t, j]), summed in the tensor dtype."""
    _lib.require_gpu(down_output, output, src2dst, topk_ids, topk_weights)
    assert down_output.is_contiguous() and output.is_contiguous() and topk_weights.is_contiguous()
    assert down_output.dtype == output.dtype
    T = output.numel() // hidden_size
    _lib.call("llmk_moe_post_reorder", _lib.ptr(down_output), _lib.ptr(output), _lib.dt(output.dtype),
              _lib.ptr(src2dst), _lib.ptr(topk_ids), _ids_bytes(topk_ids), _lib.ptr(topk_weights),
              _lib.dt(topk_weights.dtype), int(start_expert_id), int(end_expert_id), int(topk), T,
              int(hidden_size), _lib.stream(output))
    return output


def _quant_buffers(rows, cols, quant_dtype, device):
    """(q, s, kind, round_mode) for the 1 x 128 activation format that goes with a weight dtype."""
    assert cols % 128 == 0, 'row length must be a multiple of 128'
    if quant_dtype == torch.float8_e4m3fn:
        return (torch.empty(rows, cols, device=device, dtype=torch.float8_e4m3fn),
                torch.empty(rows, cols // 128, device=device, dtype=torch.float32), _lib.KIND_FP8, 0)
    assert quant_dtype == torch.int8, 'quant_dtype must be torch.int8 or torch.float8_e4m3fn'
    return (torch.empty(rows, cols, device=device, dtype=torch.int8),
            torch.empty(rows, cols // 128, device=device, dtype=torch.float16), _lib.KIND_I8, 0)


def pre_reorder_quant(input, src2dst, topk_ids, a1_scales, start_expert_id, end_expert_id, topk, hidden_size,
                      quant_dtype):
    """pre_reorder followed by the 1 x 128 activation quantizer, in one pass (the reference's TODO at
    sglang_moe_all_gather_all_reduce.py:295-296).  Returns (q [T*topk, hidden], s [T*topk, hidden/128]); equal
    bit for bit to act_quant(pre_reorder(...)).  Rows of non-local experts are left unwritten."""
    _lib.require_gpu(input, src2dst, topk_ids)
    assert input.is_contiguous() and src2dst.is_contiguous() and topk_ids.is_contiguous()
    assert input.dtype in (torch.float16, torch.bfloat16)
    T = input.numel() // hidden_size
    q, s, kind, mode = _quant_buffers(T * topk, hidden_size, quant_dtype, input.device)
    sc = _f32_or_none(a1_scales)
    _lib.call("llmk_moe_pre_reorder_quant", _lib.ptr(input), _lib.dt(input.dtype), _lib.ptr(q), _lib.ptr(s), kind, mode,
              _lib.ptr(src2dst), _lib.ptr(topk_ids), _ids_bytes(topk_ids), _lib.ptr(sc), int(start_expert_id),
              int(end_expert_id), int(topk), T, int(hidden_size), _lib.stream(input))
    return q, s


def act_and_mul_quant(gateup_output, hidden_size, reorder_topk_ids, scales, start_expert_id, end_expert_id, quant_dtype,
                      activation="silu"):
    """silu_and_mul / gelu_and_mul followed by the 1 x 128 activation quantizer, in one pass (the reference's TODO
    at sglang_moe_all_gather_all_reduce.py:365,407-408).  `hidden_size` is the gate+up width 2I as in
    silu_and_mul.  Returns (q [M, I], s [M, I/128]); equal bit for bit to act_quant(silu_and_mul(...))."""
    _lib.require_gpu(gateup_output, reorder_topk_ids)
    assert gateup_output.is_contiguous() and reorder_topk_ids.is_contiguous()
    assert gateup_output.dtype in (torch.float16, torch.bfloat16)
    M = gateup_output.numel() // hidden_size
    q, s, kind, mode = _quant_buffers(M, hidden_size // 2, quant_dtype, gateup_output.device)
    sc = _f32_or_none(scales)
    _lib.call("llmk_moe_act_and_mul_quant", _lib.ptr(gateup_output), _lib.dt(gateup_output.dtype), _lib.ptr(q),
              _lib.ptr(s), kind, mode, _lib.ptr(reorder_topk_ids), _ids_bytes(reorder_topk_ids), _lib.ptr(sc),
              int(start_expert_id), int(end_expert_id), M, int(hidden_size), {"silu": 0, "gelu": 1}[activation],
              _lib.stream(gateup_output))
    return q, s


def grouped_gemm_swiglu_quant_fused(a, b, batch_size):
    """True when `grouped_gemm_swiglu_quant` runs this gate / up projection in one kernel (shapes that the 256-column
    tile kernel takes); otherwise run grouped_gemm_triton and act_and_mul_quant."""
    kind = {torch.int8: _lib.KIND_I8, torch.float8_e4m3fn: _lib.KIND_FP8}.get(b.dtype)
    if kind is None or a.dtype != b.dtype or b.dim() != 3:
        return False
    return bool(_lib.load().llmk_grouped_gemm_swiglu_quant_fused(kind, int(batch_size), a.shape[0], b.shape[1], b.shape[2]))


def grouped_gemm_swiglu_quant(a, scale_a, b, scale_b, batch_size, seg_indptr, weight_indices, mid_dtype, activation="silu"):
    """Gate / up projection of a gated MLP over expert segments with the gated activation and the 1 x 128 quantiser of
    the down projection in the GEMM's epilogue: equal bit for bit to
    act_and_mul_quant(grouped_gemm_triton(a, b, c of `mid_dtype`, ...)), without the [M, 2I] tensor (the reference runs
    the three kernels one after the other, sglang_moe_all_gather_all_reduce.py:330-408).  a [M, K] and b [E, 2I, K]
    int8 or float8_e4m3fn with 1 x 128 / 128 x 128 block scales.  Returns (q [M, I], s [M, I/128]); rows outside every
    segment are left unwritten.  Only for shapes for which grouped_gemm_swiglu_quant_fused() is true."""
    _lib.require_gpu(a, b, scale_a, scale_b, seg_indptr)
    assert a.is_contiguous() and b.is_contiguous() and a.dtype == b.dtype and b.dim() == 3 and a.shape[-1] == b.shape[-1]
    assert mid_dtype in (torch.float16, torch.bfloat16)
    M, two_i, K = a.shape[0], b.shape[1], b.shape[2]
    q, s, kind, mode = _quant_buffers(M, two_i // 2, b.dtype, a.device)
    scale_a, scale_b = scale_a.contiguous(), scale_b.contiguous()
    if scale_b.dtype != scale_a.dtype:
        scale_b = scale_b.to(scale_a.dtype)
    seg = (seg_indptr if seg_indptr.dtype == torch.int64 else seg_indptr.to(torch.int64)).contiguous()
    wi = None
    if weight_indices is not None:
        wi = (weight_indices if weight_indices.dtype == torch.int64 else weight_indices.to(torch.int64)).contiguous()
    ws, ws_bytes = None, 0
    if scale_a.dtype != torch.float32:
        ws_bytes = M * (K // 128) * 4
        ws = _lib.ptr(_lib.workspace(a.device, ws_bytes))
    _lib.call("llmk_grouped_gemm_swiglu_quant", _lib.ptr(a), _lib.ptr(b), _lib.ptr(q), _lib.ptr(s), kind, _lib.dt(mid_dtype),
              mode, int(batch_size), M, two_i, K, _lib.ptr(seg), _lib.ptr(wi), _lib.ptr(scale_a), _lib.ptr(scale_b),
              _lib.dt(scale_a.dtype), {"silu": 0, "gelu": 1}[activation], ws, ws_bytes, _lib.stream(a), exc=AssertionError)
    return q, s


class _GridCall:
    """Accepts `obj[grid](*args, BLOCK_SIZE=...)`; the grid and the tile size are chosen by the HIP launcher."""

    def __init__(self, fn):
        self._fn = fn
        self.__doc__ = fn.__doc__

    def __getitem__(self, grid):
        def launch(*args, BLOCK_SIZE=None, **kw):
            return self._fn(*args, **kw)
        return launch

    def __call__(self, *args, BLOCK_SIZE=None, **kw):
        return self._fn(*args, **kw)


pre_reorder_triton_kernel = _GridCall(pre_reorder)
silu_and_mul_triton_kernel = _GridCall(silu_and_mul)
gelu_and_mul_triton_kernel = _GridCall(gelu_and_mul)
post_reorder_triton_kernel = _GridCall(post_reorder)


def grouped_gemm_triton(
    a: torch.Tensor,
    b: torch.Tensor,
    c: torch.Tensor,
    batch_size: int,
    weight_column_major: bool,
    seg_indptr: Optional[torch.Tensor] = None,
    weight_indices: Optional[torch.Tensor] = None,
    use_fp8_w8a8: bool = False,
    scale_a: torch.Tensor = None,
    scale_b: torch.Tensor = None,
    block_shape: Optional[List[int]] = None,
):
    """c[seg[e]:seg[e+1]] = a[seg[e]:seg[e+1]] @ b[weight_indices[e]]^T for e < batch_size; c is written in place.

    With `block_shape` and quantised weights the activations are quantised here per 1 x block_k group:
    int8 weights -> int8 activations (the reference behaviour), float8_e4m3fn weights -> e4m3 activations.
    """
    assert weight_column_major == True  # noqa: E712  (same precondition as the reference)
    if use_fp8_w8a8 and block_shape is None:
        assert scale_a is not None and scale_b is not None
    _lib.require_gpu(a, b, c)
    assert seg_indptr is not None, 'seg_indptr is required'
    quantised_w = b.dtype in (torch.int8, torch.float8_e4m3fn)
    if block_shape is not None and quantised_w:
        assert len(block_shape) == 2
        block_n, block_k = block_shape[0], block_shape[1]
        assert block_n == 128 and block_k == 128, 'block-scaled grouped GEMM uses 128 x 128 weight blocks'
        if a.dtype == b.dtype:
            # extension: activations already in the 1 x block_k format of the weights (from pre_reorder_quant /
            # act_and_mul_quant); scale_a is theirs
            assert scale_a is not None, 'quantised activations need scale_a'
            scale_a = scale_a.contiguous()
        else:
            per_token_group_quant = (_int8_kernel if b.dtype == torch.int8 else _fp8_kernel).act_quant
            a, scale_a = per_token_group_quant(a.contiguous(), block_k)
        assert _cdiv(a.shape[-1], block_k) == scale_a.shape[-1]
        assert _cdiv(b.shape[-2], block_n) == scale_b.shape[-2]
        assert _cdiv(b.shape[-1], block_k) == scale_b.shape[-1]
    elif quantised_w and use_fp8_w8a8:
        # per-expert scalar scales (the branch the reference keeps commented out, group_gemm_kernel.py:417-420):
        # c = (a . b^T) * scale_a[e] * scale_b[e] with operands already quantised.  Run as block scales that are
        # constant per expert: a scalar factor commutes with the per-block accumulation.
        assert a.dtype == b.dtype, 'per-expert scaling takes activations already in the weight dtype'
        assert a.shape[-1] % 128 == 0, 'K must be a multiple of 128'
        kb = a.shape[-1] // 128
        nb = _cdiv(b.shape[1], 128)
        sdt = torch.float32 if b.dtype == torch.float8_e4m3fn else torch.float16
        seg64 = (seg_indptr if seg_indptr.dtype == torch.int64 else seg_indptr.to(torch.int64)).contiguous()
        sa = scale_a.to(torch.float32).flatten().contiguous()
        sb = scale_b.to(torch.float32).flatten().contiguous()
        assert sa.numel() >= batch_size and sb.numel() >= b.shape[0], 'one activation scale per segment, one weight scale per expert'
        scale_a = torch.empty(a.shape[0], kb, device=a.device, dtype=sdt)
        scale_b = torch.empty(b.shape[0], nb, kb, device=a.device, dtype=sdt)
        # one launch, nothing read back (usable under graph capture)
        _lib.call("llmk_moe_expert_scales", _lib.ptr(sa), _lib.ptr(sb), _lib.ptr(seg64), int(batch_size), b.shape[0],
                  a.shape[0], b.shape[1], b.shape[2], _lib.ptr(scale_a), _lib.ptr(scale_b), _lib.dt(sdt), _lib.stream(a))
    elif quantised_w:
        raise AssertionError('quantised weights need block_shape=[128, 128] and scale_b, or use_fp8_w8a8 with per-expert scales')
    assert a.is_contiguous() and b.is_contiguous() and c.is_contiguous(), 'Input tensors must be contiguous'
    assert b.dim() == 3 and a.shape[-1] == b.shape[-1] and c.shape[-1] == b.shape[1] and c.shape[0] == a.shape[0]
    assert a.dtype == b.dtype, 'a and b must share a dtype after activation quantisation'
    kind = {torch.int8: _lib.KIND_I8, torch.float8_e4m3fn: _lib.KIND_FP8,
            torch.float16: _lib.KIND_F16, torch.bfloat16: _lib.KIND_BF16}.get(b.dtype)
    assert kind is not None, 'unsupported operand dtype %s' % b.dtype
    s_dt = 0
    if kind in (_lib.KIND_I8, _lib.KIND_FP8):
        scale_b = scale_b.contiguous()
        if scale_b.dtype != scale_a.dtype:
            scale_b = scale_b.to(scale_a.dtype)
        s_dt = _lib.dt(scale_a.dtype)
    else:
        scale_a = scale_b = None
    seg = seg_indptr if seg_indptr.dtype == torch.int64 else seg_indptr.to(torch.int64)
    seg = seg.contiguous()
    wi = None
    if weight_indices is not None:
        wi = (weight_indices if weight_indices.dtype == torch.int64 else weight_indices.to(torch.int64)).contiguous()
    _lib.call("llmk_grouped_gemm", _lib.ptr(a), _lib.ptr(b), _lib.ptr(c), kind, _lib.dt(c.dtype), int(batch_size),
              a.shape[0], b.shape[1], b.shape[2], _lib.ptr(seg), _lib.ptr(wi), _lib.ptr(scale_a), _lib.ptr(scale_b),
              s_dt, *_lib.gemm_workspace(a.device, a.shape[0], b.shape[1], b.shape[2]), _lib.stream(a),
              exc=AssertionError)
    return c
