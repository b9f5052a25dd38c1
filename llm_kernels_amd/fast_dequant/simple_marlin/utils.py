"""Offline W4A16 quantisation and simple-Marlin packing (reference fast_dequant/simple_marlin/utils.py).

QuantUtils.fake_quantize (:98-137) and QuantUtils.pack (:53-95) with identical outputs; the permutation
tables are built from the fragment-ownership rule directly and everything stays on the tensor's device
(no host round trip).
"""
import torch


def _weight_perm() -> torch.Tensor:
    """Gather index over one (16 K x 64 N) chunk laid out as four row-major 16x16 tiles.

    Output position p = 32*lane + 8*j + t holds, for fragment lane `lane` and 16-column tile j, nibble t:
    t = h + 2*b + 4*odd  ->  row = 2*(lane % 4) + odd + 8*h,  col = lane // 4 + 8*b.
    """
    p = torch.arange(1024)
    lane, j, t = p // 32, (p // 8) % 4, p % 8
    odd, b, h = t // 4, (t // 2) % 2, t % 2
    row = 2 * (lane % 4) + odd + 8 * h
    col = lane // 4 + 8 * b
    return 256 * j + 16 * row + col


def _scale_perm(grouped: bool) -> torch.Tensor:
    p = torch.arange(64 if grouped else 32)
    if grouped:
        return (p // 8) + 8 * (p % 8)
    off = torch.tensor([0, 1, 8, 9, 16, 17, 24, 25])
    return 2 * (p // 8) + off[p % 8]


_perm = _weight_perm()
_scale_perm_grouped = _scale_perm(True)
_scale_perm_single = _scale_perm(False)


class QuantUtils():

    @staticmethod
    def pack(weight: torch.Tensor, scale: torch.Tensor, groupsize: int = -1) -> tuple:
        """weight int32 [K, N] in 0..15, scale [K/g, N] -> (packed int32 [K/16, 2N], permuted scale [K/g, N])."""
        assert weight.dtype == torch.int, f"weight dtype {weight.dtype} != torch.int"
        assert weight.shape[0] % groupsize == 0, "Weight shape must be divisible by groupsize"
        tile = 16
        k, n = weight.shape
        dev = weight.device
        sp = (_scale_perm_grouped if groupsize != -1 else _scale_perm_single).to(scale.device)
        scale = scale.reshape(-1, sp.numel())[:, sp].reshape(-1, n).contiguous()

        w = weight.reshape(k // tile, tile, n // tile, tile).permute(0, 2, 1, 3).reshape(k // tile, n * tile)
        w = w.reshape(-1, _perm.numel())[:, _perm.to(dev)].reshape(k // tile, n * tile // 8, 8)
        shifts = torch.arange(0, 32, 4, device=dev, dtype=torch.int64)
        packed = ((w.to(torch.int64) & 0xF) << shifts).sum(dim=-1)
        packed = torch.where(packed >= 2 ** 31, packed - 2 ** 32, packed).to(torch.int32)
        return packed, scale

    @staticmethod
    def fake_quantize(weight: torch.Tensor, groupsize: int = -1) -> tuple:
        """W [K, N] fp16 -> (dequantised fp16 reference, q int32 in 0..15, scale fp16 [K/g, N]).

        scale = max|w| * 2/15 per (group, column) in fp16; q = clamp(round(w / scale) + 8, 0, 15)."""
        assert weight.dtype == torch.half, f"weight dtype {weight.dtype} != torch.half"
        assert weight.shape[0] % groupsize == 0, "Weight shape must be divisible by groupsize"
        maxq = 2 ** 4 - 1
        k, n = weight.shape
        g = k if groupsize == -1 else groupsize
        w = weight.reshape(k // g, g, n)
        scale = w.abs().amax(dim=1, keepdim=True)
        scale = scale * (2 / maxq)
        q = torch.round(w / scale).int() + (maxq + 1) // 2
        q = torch.clamp(q, 0, maxq)
        ref = (q - (maxq + 1) // 2).half() * scale
        return ref.reshape(k, n).contiguous(), q.reshape(k, n).contiguous(), scale.reshape(-1, n).contiguous()
