"""prim::ParallelMap regions: every loop iteration of a parallelised loop runs
as one task of a single launch (reference: fait/passes/parallelize_loops.cpp:59-126,
te_op.cpp:34-133; worked example examples/pmap.py, README.md:611-663)."""
import torch

from functs_amd import Region
from tests.util import assert_close, assert_exact, run_region


def _decode(bboxes, pred, stride):
    xy = (bboxes[..., :2] + bboxes[..., 2:]) * 0.5 + (pred[..., :2] - 0.5) * stride
    wh = (bboxes[..., 2:] - bboxes[..., :2]) * 0.5 * pred[..., 2:].exp()
    return torch.stack((xy[..., 0] - wh[..., 0], xy[..., 1] - wh[..., 1],
                        xy[..., 0] + wh[..., 0], xy[..., 1] + wh[..., 1]), dim=-1)


def build_pmap(degree):
    """examples/pmap.py:101-136: lists of boxes / predictions / strides, one
    element per task (is_parallel_args = [1, 1, 1])."""
    r = Region(parallel_degree=degree, is_parallel_map=True)
    b = r.tensor_input(torch.float32, 2, per_task=True)
    p = r.tensor_input(torch.float32, 2, per_task=True)
    s = r.scalar_input("float", per_task=True)
    xy = (b.slice(1, 0, 2) + b.slice(1, 2, None)) * 0.5 + (p.slice(1, 0, 2) - 0.5) * s
    wh = (b.slice(1, 2, None) - b.slice(1, 0, 2)) * 0.5 * p.slice(1, 2, None).exp()
    out = r.stack([xy.select(1, 0) - wh.select(1, 0), xy.select(1, 1) - wh.select(1, 1),
                   xy.select(1, 0) + wh.select(1, 0), xy.select(1, 1) + wh.select(1, 1)], -1)
    r.output(out.clone())
    return r.finalize()


def test_pmap_example_three_levels(backend):
    g = torch.Generator().manual_seed(0)
    sizes = [128, 64, 32]
    boxes = [torch.rand(n, 4, generator=g) for n in sizes]
    preds = [torch.rand(n, 4, generator=g) for n in sizes]
    strides = [8.0, 16.0, 32.0]
    (got,) = run_region(backend, build_pmap(3), boxes, preds, strides)
    ref = [_decode(b, p, s) for b, p, s in zip(boxes, preds, strides)]
    assert len(got) == 3
    assert_close(got, ref, "pmap", rtol=1e-5, atol=1e-6)


def test_pmap_task_index_addressing(backend):
    """A shared tensor indexed by the task index (immut::select(x, 0, i))."""
    T = 5
    r = Region(parallel_degree=T, is_parallel_map=True)
    x = r.tensor_input(torch.float32, 3)
    i = r.task_index()
    r.output(x.select(0, i) * 2.0)
    r.output(x.select(0, r.op("INT_SUB", T - 1, i)))
    r.finalize()
    t = torch.rand(T, 9, 11, generator=torch.Generator().manual_seed(2))
    a, b = run_region(backend, r, t)
    assert_exact(a, [t[k] * 2.0 for k in range(T)])
    assert_exact(b, [t[T - 1 - k] for k in range(T)])
