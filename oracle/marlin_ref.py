"""simple-Marlin W4A16 offline quantize / pack, and an emulation of the reference kernel (test oracle).

fake_quantize  follows fast_dequant/simple_marlin/utils.py:98-137
pack           follows fast_dequant/simple_marlin/utils.py:20-46,53-95
emulate_*      follows fast_dequant/simple_marlin/marlin_w4a16_gemm.cu:44-64 (dequant),
               :152-163 (B tile addressing), :166-176,:198-213 (scale addressing),
               :215-236 (fragment use) and :244-279 (write-back), with the
               mma.sync.m16n8k16 fragment ownership of the PTX ISA manual
               (B: lane owns k in {2(l%4), +1, +8, +9}, n = l/4; C: rows l/4, l/4+8,
               cols 2(l%4), +1).  The emulation reads the packed words the way the
               kernel does, so pack() and the kernel's consumption pin each other.
"""
import numpy as np
import torch


def fake_quantize(weight: torch.Tensor, groupsize: int = -1):
    """W [K,N] fp16 -> (ref fp16 [K,N], q int32 [K,N] in 0..15, scale fp16 [K/g, N]).

    scale = max|w| * (2/15) computed in fp16, q = clamp(rne(w / scale) + 8, 0, 15),
    ref = (q - 8).half() * scale.
    """
    assert weight.dtype == torch.half
    K, N = weight.shape
    g = K if groupsize == -1 else groupsize
    assert K % g == 0
    w = weight.reshape(K // g, g, N)
    scale = w.abs().amax(dim=1, keepdim=True)            # fp16 [K/g,1,N]
    scale = scale * (2 / 15)                             # python scalar * fp16 tensor -> fp16
    q = torch.round(w / scale).int() + 8
    q = torch.clamp(q, 0, 15)
    ref = (q - 8).half() * scale
    return ref.reshape(K, N).contiguous(), q.reshape(K, N).contiguous(), scale.reshape(K // g, N).contiguous()


def weight_perm():
    """The 1024-entry gather index applied to each (16 K x 64 N) chunk of the tiled matrix.

    Tiled position index inside a chunk: 256*j + 16*row + col for 16x16 tile j (N direction).
    For mma lane i, sub-tile j, the 8 values (block in {0,1}) x (rows 2(i%4), +1, +8, +9) at
    col i//4 + 8*block are gathered, then reordered [0,2,4,6,1,3,5,7] so that nibble pairs
    (t, t+4) of a word hold consecutive k.
    """
    perm = np.empty(1024, dtype=np.int64)
    inter = (0, 2, 4, 6, 1, 3, 5, 7)
    p = 0
    for i in range(32):
        col = i // 4
        base = []
        for block in (0, 1):
            for row in (2 * (i % 4), 2 * (i % 4) + 1, 2 * (i % 4 + 4), 2 * (i % 4 + 4) + 1):
                base.append(16 * row + col + 8 * block)
        for j in range(4):
            grp = [b + 256 * j for b in base]
            for t in range(8):
                perm[p] = grp[inter[t]]
                p += 1
    return perm


def scale_perm(grouped=True):
    if grouped:
        return np.array([i + 8 * j for i in range(8) for j in range(8)], dtype=np.int64)
    return np.array([2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)], dtype=np.int64)


def pack(q: torch.Tensor, scale: torch.Tensor, groupsize: int = -1):
    """q int32 [K,N] (0..15), scale [K/g,N] -> (B int32 [K/16, 2N], permuted scale [K/g,N])."""
    assert q.dtype == torch.int32
    K, N = q.shape
    sp = scale_perm(groupsize != -1)
    s = scale.reshape(-1, len(sp))[:, torch.from_numpy(sp)].reshape(-1, N).contiguous()
    t = q.reshape(K // 16, 16, N // 16, 16).permute(0, 2, 1, 3).reshape(K // 16, N * 16)
    wp = torch.from_numpy(weight_perm())
    t = t.reshape(-1, 1024)[:, wp].reshape(K // 16, N * 16)
    u = t.numpy().astype(np.uint32)
    out = np.zeros((K // 16, N * 16 // 8), dtype=np.uint32)
    for i in range(8):
        out |= u[:, i::8] << np.uint32(4 * i)
    return torch.from_numpy(out.view(np.int32).copy()), s


def emulate_unpack(B: torch.Tensor, s_perm: torch.Tensor, K: int, N: int, groupsize: int):
    """Recover (q [K,N], scale [K/g,N]) from packed tensors by walking the reference kernel.

    For every 16-K strip, 64-N chunk, mma lane l (0..31), sub-tile j (0..3): the kernel reads
    int4 word `l` of the chunk, component j; dequant() takes nibbles at bits 0,16 (k0,k0+1)
    and 4,20 (k0+8,k0+9) for column block 0, the same of (word >> 8) for column block 1.
    """
    Bu = B.numpy().view(np.uint32).reshape(K // 16, N // 64, 32, 4)
    q = np.zeros((K, N), dtype=np.int32)
    for l in range(32):
        k0 = 2 * (l % 4)
        c = l // 4
        for j in range(4):
            w = Bu[:, :, l, j]                            # [K/16, N/64]
            for blk in (0, 1):
                ww = w >> np.uint32(8 * blk)
                n_in = 16 * j + 8 * blk + c
                vals = {k0: ww & 0xF, k0 + 1: (ww >> 16) & 0xF, k0 + 8: (ww >> 4) & 0xF, k0 + 9: (ww >> 20) & 0xF}
                for kk, v in vals.items():
                    q[kk::16, n_in::64] = v
    g = K if groupsize == -1 else groupsize
    sp = s_perm.reshape(K // g, N // 64, 8, 8)             # [.., chunk, lane/4, 2j+blk]
    s = torch.zeros(K // g, N, dtype=s_perm.dtype)
    if groupsize != -1:
        for c in range(8):
            for j in range(4):
                for blk in (0, 1):
                    s[:, (16 * j + 8 * blk + c)::64] = sp[:, :, c, 2 * j + blk]
    return torch.from_numpy(q), s
