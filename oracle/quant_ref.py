"""Activation / weight quantizers and dequantizers restated in torch-CPU fp32 (test oracle).

Each function cites the reference lines it restates.  All arithmetic is fp32
with IEEE division, exactly as the reference kernels state it; the three
rounding rules used by the reference are explicit functions here.
"""
import torch

FP8_MAX = 448.0


# ----------------------------------------------------------------- rounding
def round_half_away(v: torch.Tensor) -> torch.Tensor:
    """libdevice.round (quantization/int8_kernel.py:27,84): ties away from zero, exact.

    Written through trunc/frac so that it is exact for every fp32 input
    (floor(|v|+0.5) is not: 0.49999997+0.5 rounds up to 1.0 in fp32).
    """
    t = torch.trunc(v)
    frac = v - t                      # exact in fp32
    return t + torch.sign(v) * (frac.abs() >= 0.5).to(v.dtype)


def round_half_up(v: torch.Tensor) -> torch.Tensor:
    """tl.floor(v + 0.5) (quantization/w4a8_kernel.py:164,222,248-252); the fp32 add is part of the rule."""
    return torch.floor(v + 0.5)


# ----------------------------------------------------------------- int8, 1x128 / 128x128
def _groups(x, block):
    assert x.shape[-1] % block == 0
    return x.contiguous().float().reshape(-1, block)


def act_quant_int8(x, block_size=128, rounding="away"):
    """int8_kernel.py:23-31 (rounding='away') and w4a8_kernel.py:159-168 (rounding='up').

    s = max|x| / 127 in fp32; y = round(x / s_fp32) -> int8; s stored as fp16.
    """
    g = _groups(x, block_size)
    s = g.abs().amax(dim=1) / 127.0
    v = g / s[:, None]
    r = round_half_away(v) if rounding == "away" else round_half_up(v)
    y = r.to(torch.int8).reshape(x.shape)
    return y, s.to(torch.float16).reshape(*x.shape[:-1], x.shape[-1] // block_size)


def _blocks2d(x, block):
    """[M,N] -> padded [mb, nb, block, block] fp32 view with zeros outside (mask other=0)."""
    M, N = x.shape
    mb, nb = (M + block - 1) // block, (N + block - 1) // block
    xp = torch.zeros(mb * block, nb * block, dtype=torch.float32)
    xp[:M, :N] = x.float()
    return xp.reshape(mb, block, nb, block).permute(0, 2, 1, 3), mb, nb


def _unblocks2d(b, M, N):
    mb, nb, block, _ = b.shape
    return b.permute(0, 2, 1, 3).reshape(mb * block, nb * block)[:M, :N].contiguous()


def weight_quant_int8(x, block_size=128):
    """int8_kernel.py:75-88: 128x128 block, s = absmax/127, half-away rounding, fp16 stored scale."""
    M, N = x.shape
    b, mb, nb = _blocks2d(x, block_size)
    s = b.abs().amax(dim=(2, 3)) / 127.0
    y = round_half_away(b / s[:, :, None, None]).to(torch.int8)
    return _unblocks2d(y, M, N), s.to(torch.float16)


def weight_dequant_block(x, s, block_size=128, out_dtype=torch.float32):
    """fp8_kernel.py:71-81, int8_kernel.py:132-142, w4a8_kernel.py:32-42: y = fp32(x) * fp32(s[block])."""
    M, N = x.shape
    se = s.float().repeat_interleave(block_size, 0)[:M].repeat_interleave(block_size, 1)[:, :N]
    return (x.float() * se).to(out_dtype)


# ----------------------------------------------------------------- fp8 e4m3fn
def act_quant_fp8(x, block_size=128):
    """fp8_kernel.py:23-30: s = max|x|/448 (fp32, stored fp32); y = (x/s) -> e4m3fn (RNE)."""
    g = _groups(x, block_size)
    s = g.abs().amax(dim=1) / FP8_MAX
    y = (g / s[:, None]).to(torch.float8_e4m3fn).reshape(x.shape)
    return y, s.reshape(*x.shape[:-1], x.shape[-1] // block_size)


def weight_quant_fp8(x, block_size=128):
    """128x128 block e4m3fn weight quantizer, s = blockmax/448 (fp32).

    The reference has no fp8 weight quantizer (fp8_kernel.py has only
    act_quant / weight_dequant / fp8_gemm); this is the analogue of
    int8_kernel.py:75-88 with the constant of fp8_kernel.py:26.
    """
    M, N = x.shape
    b, mb, nb = _blocks2d(x, block_size)
    s = b.abs().amax(dim=(2, 3)) / FP8_MAX
    y = (b / s[:, :, None, None]).to(torch.float8_e4m3fn)
    return _unblocks2d(y.view(torch.uint8), M, N).view(torch.float8_e4m3fn), s


# ----------------------------------------------------------------- w4a8 two-level weights
def w4a8_weight_quant_levels(x, block_size=128, group_size_int4=128):
    """w4a8_kernel.py:212-262 without the packing step.

    level 1: 128x128 blocks, s = absmax/119, y = clamp(floor(x/s+.5), -119, 119) int8, s fp16.
    level 2: per (row, 128-col group) of y: s4 = floor((max-min)/15+.5),
             z4 = floor(-min/s4+.5), q = clamp(floor(y/s4+.5)+z4, 0, 15).
    Returns (q uint8 [M,N] in 0..15, s fp16 [mb,nb], s4 int8 [M,ng], z4 int8 [M,ng]).
    """
    M, N = x.shape
    assert N % block_size == 0 and block_size % group_size_int4 == 0
    b, mb, nb = _blocks2d(x, block_size)
    s = b.abs().amax(dim=(2, 3)) / 119.0
    y = torch.clamp(round_half_up(b / s[:, :, None, None]), -119.0, 119.0)
    y = _unblocks2d(y, M, N)                       # fp32 holding int8 values
    g = y.reshape(M, N // group_size_int4, group_size_int4)
    mx, mn = g.amax(dim=2), g.amin(dim=2)
    s4 = round_half_up((mx - mn) / 15.0)
    z4 = round_half_up(-mn / s4)
    q = torch.clamp(round_half_up(g / s4[:, :, None]) + z4[:, :, None], 0, 15)
    return (q.reshape(M, N).to(torch.uint8), s.to(torch.float16),
            s4.to(torch.int8), z4.to(torch.int8))


def w4a8_dequant_int8(q, s4, z4, group_size_int4=128):
    """w4a8_kernel.py:64-101 / :382: (q - z4) * s4 evaluated in int8 (two's-complement wrap)."""
    M, N = q.shape
    s4e = s4.to(torch.int32).repeat_interleave(group_size_int4, 1)[:, :N]
    z4e = z4.to(torch.int32).repeat_interleave(group_size_int4, 1)[:, :N]
    d = (q.to(torch.int32) - z4e)
    d = ((d + 128) % 256) - 128                    # int8 wrap of the subtraction
    d = d * s4e
    d = ((d + 128) % 256) - 128                    # int8 wrap of the product
    return d.to(torch.int8)


def w4a8_weight_dequant(q, s, s4, z4, block_size=128, group_size_int4=128):
    """w4a8_kernel.py:104-142: int4 -> int8 -> fp16 (q is the *unpacked* 0..15 matrix [N,K])."""
    d8 = w4a8_dequant_int8(q, s4, z4, group_size_int4)
    return weight_dequant_block(d8, s, block_size, torch.float16)


# ----------------------------------------------------------------- config-variant quantizers
def w4a16_quant_nk(w, group_size=128):
    """Symmetric int4 along K for W [N,K]: s = absmax/7 (fp16), q = clamp(rne(w/s), -8, 7) + 8.

    This is the absmax/7 rule (not the Marlin 2*absmax/15 rule).
    """
    N, K = w.shape
    g = w.float().reshape(N, K // group_size, group_size)
    s = (g.abs().amax(dim=2) / 7.0).to(torch.float16)
    q = torch.clamp(torch.round(g / s.float()[:, :, None]), -8, 7) + 8
    return q.reshape(N, K).to(torch.uint8), s


def int8_quant_rowwise(x):
    """Per-row symmetric int8 with fp32 scale (per-token activations / per-channel weights)."""
    xf = x.float()
    s = xf.abs().amax(dim=1) / 127.0
    y = round_half_away(xf / s[:, None]).to(torch.int8)
    return y, s
