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


# ---- maps of more tasks than the kernel argument block has room for ------------------------------
def _many_task_map(T):
    """Three per-task results and a per-task scalar: 3 T + pointers of the inputs, T scalars."""
    r = Region(parallel_degree=T, is_parallel_map=True)
    x = r.tensor_input(torch.float32, 3)
    w = r.tensor_input(torch.float32, 2, per_task=True)
    s = r.scalar_input("float", per_task=True)
    i = r.task_index()
    row = x.select(0, i)
    r.output(row * s + w)
    r.output((row - w).relu())
    r.output(x.select(0, r.op("INT_SUB", T - 1, i)) * 0.5)
    return r.finalize()


def test_a_map_of_many_tasks_uploads_its_tables(backend):
    """150 tasks x 4 per-task tensors = 600 pointers (the argument block holds 320) and 150 scalars:
    the tables travel through device memory, the results are those of the loop over the tasks."""
    import ctypes
    from functs_amd._lib import lib
    T = 150
    g = torch.Generator().manual_seed(5)
    x = torch.rand(T, 7, 33, generator=g)
    ws = [torch.rand(7, 33, generator=g) for _ in range(T)]
    ss = [0.25 * (k % 9) - 1.0 for k in range(T)]
    r = _many_task_map(T)
    a, b, c = run_region(backend, r, x, ws, ss)
    assert_exact(a, [x[k] * torch.tensor(ss[k], dtype=torch.float32) + ws[k] for k in range(T)], "scaled")
    assert_exact(b, [(x[k] - ws[k]).relu() for k in range(T)], "relu")
    assert_exact(c, [x[T - 1 - k] * 0.5 for k in range(T)], "mirrored")
    arr, n, keep = r._flatten((x, ws, ss))
    p = r.plan(arr, n)
    n_p, n_s, up = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_int()
    assert lib.fx_plan_table_sizes(p.handle, ctypes.byref(n_p), ctypes.byref(n_s), ctypes.byref(up)) == 0
    assert up.value == 1 and n_p.value >= 4 * T and n_s.value >= T
    assert p.scratch_bytes >= 8 * n_p.value + 4 * n_s.value     # a dense region, and still scratch: the tables
    # the same region over few tasks keeps the argument block
    small = _many_task_map(8)
    arr, n, keep = small._flatten((x[:8], ws[:8], ss[:8]))
    ps = small.plan(arr, n)
    assert lib.fx_plan_table_sizes(ps.handle, ctypes.byref(n_p), ctypes.byref(n_s), ctypes.byref(up)) == 0
    assert up.value == 0 and ps.scratch_bytes == 0


def test_a_compacting_map_of_many_tasks(backend):
    """A row filter over 200 tasks with two results each: both passes read the uploaded tables."""
    T = 200
    r = Region(parallel_degree=T, is_parallel_map=True)
    x = r.tensor_input(torch.float32, 2, per_task=True)
    thr = r.scalar_input("float", per_task=True)
    keep = x.select(1, 0) > thr
    r.compact_rows(keep)
    r.output(x * 2.0)
    r.output(x.select(1, 1))
    r.finalize()
    g = torch.Generator().manual_seed(6)
    xs = [torch.rand(5 + (k * 7) % 40, 6, generator=g) for k in range(T)]
    ts = [0.1 + 0.004 * k for k in range(T)]
    a, b = run_region(backend, r, xs, ts)
    masks = [x[:, 0] > torch.tensor(t, dtype=torch.float32) for x, t in zip(xs, ts)]
    assert_exact(a, [x[m] * 2.0 for x, m in zip(xs, masks)], "rows")
    assert_exact(b, [x[m][:, 1] for x, m in zip(xs, masks)], "column")


def test_tables_beyond_the_upload_limit_are_an_error():
    import pytest
    T = 1400   # 4 x 1400 pointers > 4096
    x = torch.rand(T, 2, 4)
    ws = [torch.rand(2, 4) for _ in range(T)]
    ss = [1.0] * T
    r = _many_task_map(T)
    arr, n, keep = r._flatten((x, ws, ss))
    with pytest.raises(RuntimeError, match="pointer slots"):
        r.plan(arr, n)
