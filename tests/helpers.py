import sys

import torch


def announce(*a):
    """Name the case on stderr before a GPU step so that a faulting run still says what it was doing."""
    print("[case]", *a, file=sys.stderr, flush=True)


def assert_close_scaled(out, ref, rtol=1e-2, atol=1e-2, what=""):
    """|out - ref| <= atol * rms(ref) + rtol * |ref| elementwise (tolerance relative to the output scale)."""
    out = out.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert out.shape == ref.shape, (out.shape, ref.shape)
    assert torch.isfinite(out).all(), "%s: non-finite output" % what
    scale = ref.pow(2).mean().sqrt().item() if ref.numel() else 1.0
    err = (out - ref).abs()
    bound = atol * scale + rtol * ref.abs()
    bad = err > bound
    assert not bad.any(), "%s: %d/%d outside tolerance, max err %.3e (scale %.3e), worst ratio %.2f" % (
        what, int(bad.sum()), bad.numel(), err.max().item(), scale, (err / bound).max().item())


def default_dtype(dt):
    class _Ctx:
        def __enter__(self):
            self.prev = torch.get_default_dtype()
            torch.set_default_dtype(dt)

        def __exit__(self, *exc):
            torch.set_default_dtype(self.prev)
    return _Ctx()
