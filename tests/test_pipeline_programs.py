"""Small imperative programs (views, in-place writes, loops, branches) through the
whole route on the GPU: script -> build -> regions run by tssa::ParallelFunctor,
everything that is not a region by ATen on the device.  Reference: eager PyTorch on
the CPU.  The programs are the ones of tests/test_tensorssa.py."""
import pytest
import torch

import functs_amd.jit as fj
from tests.test_tensorssa import PROGRAMS, _IDS, _clone

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fn,make", PROGRAMS, ids=_IDS)
def test_program_on_gpu(fn, make):
    gen = torch.Generator().manual_seed(4321)
    args = make(gen)
    want = fn(*_clone(args))
    built = fj.build(fj.script(fn, add_clone=True), list(args))
    dev_args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
    got = built(*dev_args)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-6)
    # a second call reuses the compiled variants and must not see state of the first
    got2 = built(*dev_args)
    assert torch.equal(got2, got)


# Two more programs in the style of the reference's simple-op benchmarks
# (functs/benchmark/simpleops/bbox_expand/bbox_expand.py:9-17,
# offset2bbox/offset2bbox.py:8-44): row writes chosen by a list of labels, and a
# box transform written through strided slice assigns.
from typing import List  # noqa: E402


def expand_by_labels(targets: torch.Tensor, weights: torch.Tensor, labels: List[int]):
    t = targets.clone() * 0.5
    w = weights.clone() + 1.0
    for i in labels:
        t[i, :] = targets[i, :]
        w[i, :] = weights[i, :] * 2.0
    return t.clone(), w.clone()


def deltas_to_boxes(boxes: torch.Tensor, deltas: torch.Tensor):
    x1, y1, x2, y2 = boxes[:, 0], boxes[:, 1], boxes[:, 2], boxes[:, 3]
    widths = x2 - x1 + 1
    heights = y2 - y1 + 1
    cx = x1 + 0.5 * widths
    cy = y1 + 0.5 * heights
    dx = deltas[:, 0::4]
    dy = deltas[:, 1::4]
    dw = torch.clamp(deltas[:, 2::4], max=4.135)
    dh = torch.clamp(deltas[:, 3::4], max=4.135)
    pcx = dx * widths[:, None] + cx[:, None]
    pcy = dy * heights[:, None] + cy[:, None]
    pw = torch.exp(dw) * widths[:, None]
    ph = torch.exp(dh) * heights[:, None]
    out = deltas.clone()
    out[:, 0::4] = pcx - 0.5 * pw
    out[:, 1::4] = pcy - 0.5 * ph
    out[:, 2::4] = pcx + 0.5 * pw - 1
    out[:, 3::4] = pcy + 0.5 * ph - 1
    return out


def test_expand_by_labels_on_gpu():
    g = torch.Generator().manual_seed(5)
    targets, weights = torch.rand(300, 4, generator=g), torch.rand(300, 4, generator=g)
    labels = [1, 2, 3, 4, 250]
    want = expand_by_labels(targets, weights, labels)
    built = fj.build(fj.script(expand_by_labels), [targets, weights, labels])
    got = built(targets.cuda(), weights.cuda(), labels)
    for g_, w in zip(got, want):
        torch.testing.assert_close(g_.cpu(), w, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("n,classes", [(3000, 1), (500, 21)])
def test_deltas_to_boxes_on_gpu(n, classes):
    g = torch.Generator().manual_seed(6)
    xy = torch.rand(n, 2, generator=g) * 200
    boxes = torch.cat([xy, xy + torch.rand(n, 2, generator=g) * 100 + 1], dim=1)
    deltas = torch.randn(n, 4 * classes, generator=g)
    want = deltas_to_boxes(boxes, deltas)
    f = fj.script(deltas_to_boxes)
    assert torch.equal(f(boxes, deltas), want)  # functionalized graph on the CPU
    built = fj.build(f, [boxes, deltas])
    assert str(built.graph).count("= tssa::ParallelFunctor") == 1  # the whole transform is one region
    got = built(boxes.cuda(), deltas.cuda())
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-3)
