"""Shared helpers of the parity tests."""
import torch


def run_region(backend, region, *args):
    """Run `region` on CPU tensors through the chosen backend; results on CPU."""
    if backend == "emul":
        from tests.support import emul
        return emul.run(region, *args)
    dev = torch.device("cuda:0")

    def g(x):
        if isinstance(x, torch.Tensor):
            return x.to(dev)
        if isinstance(x, (list, tuple)) and x and isinstance(x[0], torch.Tensor):
            return [t.to(dev) for t in x]
        return x

    outs = region(*[g(a) for a in args])
    torch.cuda.synchronize()

    def c(x):
        return [c(t) for t in x] if isinstance(x, (list, tuple)) else x.cpu()

    return c(outs)


def assert_exact(got, ref, what=""):
    if isinstance(ref, (list, tuple)):
        assert len(got) == len(ref), "%s: %d vs %d entries" % (what, len(got), len(ref))
        for i, (g, r) in enumerate(zip(got, ref)):
            assert_exact(g, r, "%s[%d]" % (what, i))
        return
    assert got.dtype == ref.dtype, "%s: dtype %s vs %s" % (what, got.dtype, ref.dtype)
    assert tuple(got.shape) == tuple(ref.shape), "%s: shape %s vs %s" % (what, tuple(got.shape), tuple(ref.shape))
    assert torch.equal(got, ref), "%s: not bit-exact (max abs diff %g)" % (
        what, (got.double() - ref.double()).abs().max().item() if ref.numel() else 0.0)


# fp32 elementwise tolerance of the build: 1e-5 relative
RTOL = 1e-5


def assert_close(got, ref, what="", rtol=RTOL, atol=1e-7):
    if isinstance(ref, (list, tuple)):
        assert len(got) == len(ref), "%s: %d vs %d entries" % (what, len(got), len(ref))
        for i, (g, r) in enumerate(zip(got, ref)):
            assert_close(g, r, "%s[%d]" % (what, i), rtol, atol)
        return
    assert got.dtype == ref.dtype, "%s: dtype %s vs %s" % (what, got.dtype, ref.dtype)
    assert tuple(got.shape) == tuple(ref.shape), "%s: shape %s vs %s" % (what, tuple(got.shape), tuple(ref.shape))
    if not ref.dtype.is_floating_point:
        assert torch.equal(got, ref), "%s: integer result differs" % what
        return
    err = (got.double() - ref.double()).abs()
    bound = atol + rtol * ref.double().abs()
    bad = err > bound
    assert not bool(bad.any()), "%s: %d elements beyond rtol %g (max err %g)" % (what, int(bad.sum()), rtol, err.max().item())


def assert_boxes_close(got, ref, what="", rtol=RTOL):
    """Boxes are x1 = c - h, x2 = c + h: the two results of one pair share the
    rounding error of c and h, so the 1e-5 relative bound is taken against
    |c| + |h| = max(|x1|, |x2|) (same for y), not against a difference that may
    cancel to nearly zero."""
    if isinstance(ref, (list, tuple)):
        assert len(got) == len(ref)
        for i, (g, r) in enumerate(zip(got, ref)):
            assert_boxes_close(g, r, "%s[%d]" % (what, i), rtol)
        return
    assert tuple(got.shape) == tuple(ref.shape), "%s: shape %s vs %s" % (what, tuple(got.shape), tuple(ref.shape))
    if ref.numel() == 0:
        return
    r = ref.double()
    scale = torch.maximum(r[:, :2].abs(), r[:, 2:].abs())
    scale = torch.cat([scale, scale], dim=1)
    err = (got.double() - r).abs()
    bad = err > (1e-7 + rtol * scale)
    assert not bool(bad.any()), "%s: %d box coordinates beyond rtol %g (max err %g)" % (
        what, int(bad.sum()), rtol, err.max().item())
