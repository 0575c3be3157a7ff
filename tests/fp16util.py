"""Comparison helpers for fp16 results."""
import torch


def _key(t):
    """fp16 bit patterns mapped to integers that are monotone in the value."""
    i = t.contiguous().view(torch.int16).to(torch.int32)
    return torch.where(i < 0, -(i & 0x7FFF), i)


def ulp_diff(a: torch.Tensor, b: torch.Tensor, on_device=False) -> torch.Tensor:
    """Distance in fp16 units-in-the-last-place between two fp16 tensors (finite values).  The
    comparison runs on the CPU unless ``on_device`` (then on ``a``'s device: large tensors)."""
    a, b = a.half(), b.half()
    if on_device:
        b = b.to(a.device)
    else:
        a, b = a.cpu(), b.cpu()
    return (_key(a) - _key(b)).abs()


def fp16_stats(got, want, max_ulp=1, atol=2e-5, mag=None, rel=1.01 * 2.0 ** -10,
               floor=2.0 ** -24, chunk=1 << 26):
    """On ``got``'s device, in chunks (tensors of a billion elements): (largest ulp distance,
    fraction of elements that differ at all, number of elements further apart than ``max_ulp``
    ulp AND than the absolute bound, the largest absolute difference among those, the largest
    difference as a fraction of what the element is allowed).  The absolute
    bound is ``atol``, or per element ``rel * mag + floor`` for a tensor ``mag`` of ``got``'s shape
    (one fp16 ulp, relatively, of a magnitude that bounds the op's rounding points; ``floor``:
    the spacing of fp16 subnormals, where an ulp is no longer relative)."""
    assert got.shape == want.shape, (got.shape, want.shape)
    got = got.detach().half().reshape(-1)
    want = want.detach().half().to(got.device).reshape(-1)
    if mag is not None:
        mag = mag.reshape(-1)
        assert mag.shape == got.shape
    worst_ulp, differ, n_bad, worst_abs, worst_rel = 0, 0, 0, 0.0, 0.0
    for i in range(0, got.numel(), chunk):
        g, w = got[i:i + chunk], want[i:i + chunk]
        assert bool(torch.isfinite(g).all()), "non-finite output"
        d = ulp_diff(g, w, on_device=True)
        ad = (g.float() - w.float()).abs()
        bound = atol if mag is None else mag[i:i + chunk].float() * rel + floor
        bad = (d > max_ulp) & (ad > bound)
        # allowed: max_ulp ulps or the absolute bound, whichever is larger for the element
        ulp = torch.ldexp(torch.ones_like(ad), torch.frexp(w.float().abs().clamp_min(
            2.0 ** -14))[1] - 11)
        worst_rel = max(worst_rel, float((ad / torch.maximum(ulp * max_ulp, bound + 0 * ad)).max()))
        worst_ulp = max(worst_ulp, int(d.max()))
        differ += int((d > 0).sum())
        nb = int(bad.sum())
        if nb:
            n_bad += nb
            worst_abs = max(worst_abs, float(ad[bad].max()))
    return worst_ulp, differ / max(1, got.numel()), n_bad, worst_abs, worst_rel


def assert_fp16_close(got, want, max_ulp=1, max_frac=5e-3, atol=2e-5, what="", on_device=False):
    """Both sides accumulate in fp32 and round once, so they may differ only where an fp32
    sum-order difference straddles an fp16 rounding boundary: at most `max_ulp` ulp (or `atol`
    absolute, for results that cancel to nearly zero), on at most `max_frac` of the elements."""
    got, want = got.detach(), want.detach()
    if not on_device:
        got, want = got.cpu(), want.cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert torch.isfinite(got.float()).all(), what + ": non-finite output"
    if got.numel() == 0:
        return 0, 0.0
    d = ulp_diff(got, want, on_device=on_device)
    ad = (got.float() - want.float().to(got.device)).abs()
    bad = (d > max_ulp) & (ad > atol)
    frac = float((d > 0).float().mean())
    assert not bool(bad.any()), "%s: %d elements off by up to %d ulp / %g abs" % (
        what, int(bad.sum()), int(d[bad].max()), float(ad[bad].max()))
    assert frac <= max_frac, "%s: %.4f of elements differ" % (what, frac)
    return int(d.max()), frac
