"""Comparison helpers for fp16 results."""
import torch


def ulp_diff(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in fp16 units-in-the-last-place between two fp16 tensors (finite values)."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return (key(a.half().cpu()) - key(b.half().cpu())).abs()


def assert_fp16_close(got, want, max_ulp=1, max_frac=5e-3, atol=2e-5, what=""):
    """Both sides accumulate in fp32 and round once, so they may differ only where an fp32
    sum-order difference straddles an fp16 rounding boundary: at most `max_ulp` ulp (or `atol`
    absolute, for results that cancel to nearly zero), on at most `max_frac` of the elements."""
    got, want = got.detach().cpu(), want.detach().cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert torch.isfinite(got.float()).all(), what + ": non-finite output"
    if got.numel() == 0:
        return 0, 0.0
    d = ulp_diff(got, want)
    ad = (got.float() - want.float()).abs()
    bad = (d > max_ulp) & (ad > atol)
    frac = float((d > 0).float().mean())
    assert not bool(bad.any()), "%s: %d elements off by up to %d ulp / %g abs" % (
        what, int(bad.sum()), int(d[bad].max()), float(ad[bad].max()))
    assert frac <= max_frac, "%s: %.4f of elements differ" % (what, frac)
    return int(d.max()), frac
