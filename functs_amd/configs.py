"""Fused regions of the five benchmark configurations, written directly against
the region builder.  Each function states the functionalized graph (immut::
access / assign operators) that the pass pipeline produces for the matching
TorchScript program and hands it to the HIP backend as ONE region.

Graph shapes follow the reference's own worked examples: README.md:284-299
(get_started after functionalization), README.md:484-507 (slice/select assigns
inlined into one fused subgraph), README.md:611-659 (ParallelMap ->
tssa::ParallelFunctor with parallel_degree / is_parallel_args).
"""
import torch

from .region import Region


def build_c1():
    """get_started loop (examples/get_started.py:10-15) after functionalization:
        for i in range(n): b = immut::select_rev(b, immut::select(b, 0, i) + 1, 0, i)
    The carried tensor is read and written only through slab i, so the n
    iterations collapse into one region (FX_OP_FORALL_SELECT_REV)."""
    r = Region()
    b = r.tensor_input(torch.float32, 2)
    n = r.scalar_input("int")
    i = r.loop_var()
    body = b.select(0, i) + 1
    r.output(r.op("FORALL_SELECT_REV", b, body, 0, 0, n))
    return r.finalize()


def _yolo_body(r, pred, anchors, strides):
    """pred: [1, N, 85] value.  Returns (boxes [N,4], cls [N,80], obj [N], keep [N])."""
    # pred[..., :2].sigmoid_()  ->  slice_rev(pred, sigmoid(slice(pred)))
    pred1 = pred.slice_rev(pred.slice(2, 0, 2).sigmoid(), 2, 0, 2)
    obj = pred1.select(2, 4).sigmoid()           # [1, N]
    cls = pred1.slice(2, 5, None).sigmoid()      # [1, N, 80]
    p = pred1.select(0, 0)                       # [N, 85]
    xy = (anchors.slice(1, 0, 2) + anchors.slice(1, 2, None)) * 0.5 + (p.slice(1, 0, 2) - 0.5) * strides.unsqueeze(-1)
    wh = (anchors.slice(1, 2, None) - anchors.slice(1, 0, 2)) * 0.5 * p.slice(1, 2, 4).exp()
    boxes = r.op("FULL", r.int_list([r.op("SIZE", anchors, 0), 4]), 0.0, dtype=torch.float32)
    boxes = boxes.select_rev(xy.select(1, 0) - wh.select(1, 0), 1, 0)
    boxes = boxes.select_rev(xy.select(1, 1) - wh.select(1, 1), 1, 1)
    boxes = boxes.select_rev(xy.select(1, 0) + wh.select(1, 0), 1, 2)
    boxes = boxes.select_rev(xy.select(1, 1) + wh.select(1, 1), 1, 3)
    obj0 = obj.select(0, 0)
    keep = obj0 >= 0.3
    return boxes, cls.select(0, 0), obj0, keep


def build_c2():
    """YOLOv3-style post-processing of one image: decode + sigmoid + confidence
    mask select as one compacting region."""
    r = Region()
    pred = r.tensor_input(torch.float32, 3)
    anchors = r.tensor_input(torch.float32, 2)
    strides = r.tensor_input(torch.float32, 1)
    boxes, cls, obj, keep = _yolo_body(r, pred, anchors, strides)
    r.output(boxes)
    r.output(cls)
    r.output(obj)
    r.compact_rows(keep)
    return r.finalize()


def build_c5(batch=16):
    """The per-image loop over c2 as one ParallelMap launch: task i works on
    preds[i:i+1]; anchors and strides are shared (is_parallel_args = 0)."""
    r = Region(parallel_degree=batch, is_parallel_map=True)
    preds = r.tensor_input(torch.float32, 3)
    anchors = r.tensor_input(torch.float32, 2)
    strides = r.tensor_input(torch.float32, 1)
    i = r.task_index()
    pred = preds.slice(0, i, r.op("INT_ADD", i, 1))
    boxes, cls, obj, keep = _yolo_body(r, pred, anchors, strides)
    r.output(boxes)
    r.output(cls)
    r.output(obj)
    r.compact_rows(keep)
    return r.finalize()


def build_c3_decode():
    """SSD prior/variance decode (two slice assigns) + softmax: one dense region
    with two outputs (boxes [N,4], scores [N,C])."""
    r = Region()
    loc = r.tensor_input(torch.float32, 3)
    conf = r.tensor_input(torch.float32, 3)
    priors = r.tensor_input(torch.float32, 2)
    l0 = loc.select(0, 0)
    cxcy = priors.slice(1, 0, 2) + l0.slice(1, 0, 2) * 0.1 * priors.slice(1, 2, None)
    wh = priors.slice(1, 2, None) * (l0.slice(1, 2, None) * 0.2).exp()
    boxes = r.op("FULL", r.int_list([r.op("SIZE", priors, 0), 4]), 0.0, dtype=torch.float32)
    boxes = boxes.slice_rev(cxcy - wh / 2, 1, 0, 2)
    boxes = boxes.slice_rev(cxcy + wh / 2, 1, 2, None)
    scores = conf.select(0, 0).softmax(-1)
    r.output(boxes)
    r.output(scores)
    return r.finalize()


def build_c3_classes(n_fg=80):
    """The per-class loop `for c in range(1, C): m = scores[:, c] > 0.05;
    boxes[m], scores[:, c][m]` as one ParallelMap over the classes."""
    r = Region(parallel_degree=n_fg, is_parallel_map=True)
    boxes = r.tensor_input(torch.float32, 2)
    scores = r.tensor_input(torch.float32, 2)
    c = r.op("INT_ADD", r.task_index(), 1)
    sc = scores.select(1, c)
    r.output(boxes)
    r.output(sc)
    r.compact_rows(sc > 0.05)
    return r.finalize()


def build_c3_fused(n_fg=80, thr=0.05, var_xy=0.1, var_wh=0.2, first=1):
    """build_c3_decode and build_c3_classes as ONE ParallelMap over the classes whose body holds
    the decode and the softmax as well (what the TorchScript route makes of c3 when it sinks the
    dense producer into the class map).  The library runs it as one launch of its SSD head kernel;
    lowered generically every task redoes the softmax."""
    r = Region(parallel_degree=n_fg, is_parallel_map=True)
    loc = r.tensor_input(torch.float32, 3)
    conf = r.tensor_input(torch.float32, 3)
    priors = r.tensor_input(torch.float32, 2)
    l0 = loc.select(0, 0)
    cxcy = priors.slice(1, 0, 2) + l0.slice(1, 0, 2) * var_xy * priors.slice(1, 2, None)
    wh = priors.slice(1, 2, None) * (l0.slice(1, 2, None) * var_wh).exp()
    boxes = r.op("FULL", r.int_list([r.op("SIZE", priors, 0), 4]), 0.0, dtype=torch.float32)
    boxes = boxes.slice_rev(cxcy - wh / 2, 1, 0, 2)
    boxes = boxes.slice_rev(cxcy + wh / 2, 1, 2, None)
    scores = conf.select(0, 0).softmax(-1)
    sc = scores.select(1, r.op("INT_ADD", r.task_index(), first))
    r.output(boxes)
    r.output(sc)
    r.compact_rows(sc > thr)
    return r.finalize()


# shape for which `python -m functs_amd.aot` compiles the region below (its reduction extents are
# part of the programs, so the compiled kernels serve this shape only)
COLUMN_STANDARDIZE_SHAPE = (777, 12)


def build_column_standardize():
    """Not one of the five configurations: a region that exercises what they do not, used to
    keep the ahead-of-time compiled path honest (serial reduction loops, max over a dimension,
    `where`, `cat` branches, a row softmax in the same launch)::

        mean = x.sum(0) / n;  z = x - mean;  spread = z.abs().max(0)
        out0 = where(z > 0, z, 0.1 * z) / (spread + 1)
        out1 = cat([x[:, :2].exp(), x[:, 2:]], 1).softmax(1)
    """
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    n = r.op("SIZE", x, 0)
    mean = r.op("SUM_DIM", x, 0, False) / n
    z = x - mean.unsqueeze(0)
    spread = r.op("MAX_DIM", r.op("ABS", z), 0, False)
    r.output(r.where(z > 0.0, z, z * 0.1) / (spread.unsqueeze(0) + 1.0))
    r.output(r.cat([x.slice(1, 0, 2).exp(), x.slice(1, 2, None)], 1).softmax(1))
    return r.finalize()


# shapes for which `python -m functs_amd.aot` compiles the region below
ROW_FILTER_SHAPES = ((1000, 19), (1000, 2))


def build_row_filter():
    """Not one of the five configurations either: a row compaction that takes every route of the
    compaction kernel in one launch, used to check the compiled kernels against the interpreter.
    Rows of `x` [n, 19] with a positive first column are kept; of those rows it returns::

        wide   = sigmoid(x[:, 3:])              16 columns: whole groups of four, unaligned rows
        ragged = x[:, :7] * 2                   7 columns: a ragged last group
        narrow = cat([a * b + a, a * b - b], 1) with a = x[:, 1:2] * s[:, 0:1], b = x[:, 2:3] + s[:, 1:2]:
                 every column reads its inputs twice
        first  = x[:, 0]
    """
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    s = r.tensor_input(torch.float32, 2)
    a = x.slice(1, 1, 2) * s.slice(1, 0, 1)
    b = x.slice(1, 2, 3) + s.slice(1, 1, 2)
    r.output(x.slice(1, 3, None).sigmoid())
    r.output(x.slice(1, 0, 7) * 2.0)
    r.output(r.cat([a * b + a, a * b - b], 1))
    r.output(x.select(1, 0))
    r.compact_rows(x.select(1, 0) > 0.0)
    return r.finalize()


def _level_anchors(r, base, feat, stride):
    """Anchors of one feature level, generated inside the region the way the reference's
    model does it on the host (yolov3_bbox.py:78-101): base [A, 4] corner form + the grid shifts."""
    sx = r.arange(0, feat, dtype=torch.float32) * stride
    xx = sx.repeat(feat)
    yy = sx.view(-1, 1).repeat(1, feat).view(-1)
    shifts = r.stack([xx, yy, xx, yy], -1)
    return (base.unsqueeze(0) + shifts.unsqueeze(1)).view(-1, 4)


# the small instance of build_c5_generated_anchors that the tests run and kernels are linked for
GENERATED_ANCHOR_LEVELS = ((3, 32.0), (5, 16.0), (9, 8.0))
# ... and the benchmark's instance (YOLOv3 at 416 x 416: 10 647 rows)
GENERATED_ANCHOR_LEVELS_C5 = ((13, 32.0), (26, 16.0), (52, 8.0))


def build_c5_generated_anchors(batch, levels):
    """C5 with the anchor / stride tables generated inside the region (arange, repeat, view,
    stack, broadcast add, cat) instead of read from HBM: the step in front of the hot path
    (yolov3_bbox.py:78-101, 209-216).  `levels`: ((feature size, stride), ...); inputs:
    preds [B, N, 85] and one base-anchor tensor [A, 4] per level, N = sum(f * f * A).
    Every use of the anchor tensor inlines its generation, so the programs are long (about
    1 200 instructions for three levels): the interpreter's temporaries exceed a workgroup's
    LDS and the region runs with compiled kernels only."""
    r = Region(parallel_degree=batch, is_parallel_map=True)
    preds = r.tensor_input(torch.float32, 3)
    bases = [r.tensor_input(torch.float32, 2) for _ in levels]
    i = r.task_index()
    pred = preds.slice(0, i, r.op("INT_ADD", i, 1))
    anchors = r.cat([_level_anchors(r, b, f, s) for b, (f, s) in zip(bases, levels)], 0)
    strides = r.cat([r.full([f * f * 3], float(s)) for f, s in levels], 0)
    boxes, cls, obj, keep = _yolo_body(r, pred, anchors, strides)
    r.output(boxes)
    r.output(cls)
    r.output(obj)
    r.compact_rows(keep)
    return r.finalize()


# ---- other spellings of the detection head ------------------------------------------------
# Decode + score filter of a YOLO-style head as programs in the field write it: the reference's own
# model joins the four corners with torch.stack and pads the class scores with a zero column
# (yolov3_bbox.py:12-23, 227-228), others concatenate the two corner pairs, keep the objectness in
# another column, filter on a class score, or return one matrix per image.  None of them is the
# text of build_c2 / build_c5; all of them are row compactions over a row-major prediction matrix,
# which is what the generated row-stream kernels are for.  `python -m functs_amd.aot` generates
# the kernels of HEAD_VARIANTS (80 classes, the benchmark's row length).
HEAD_VARIANTS = {
    "stack": dict(decode="stack"),
    "cat": dict(decode="cat"),
    "stack_padded": dict(decode="stack", pad=True),
    "objectness_first": dict(obj_col=0),
    "quarter_size": dict(half=0.25),
    "class_score_mask": dict(mask_class=17),
    "one_matrix": dict(decode="cat", joined=True),
}


def build_head_variant(batch=None, thr=0.3, decode="assign", pad=False, obj_col=4, half=0.5, mask_class=None, joined=False):
    """A detection-head region.  pred [B, N, 5 + C] (columns: four box values, objectness at
    obj_col among the first five, C class scores from column 5), anchors [N, 4], strides [N].
    decode: how the corners are joined ("assign": four select assigns, "stack", "cat"); pad: the
    class scores get a zero column behind them; mask_class: rows are kept on sigmoid(class score)
    instead of the objectness; joined: one output [K, 4 + 1 + C] instead of three."""
    r = Region(parallel_degree=batch, is_parallel_map=True) if batch else Region()
    preds = r.tensor_input(torch.float32, 3)
    anchors = r.tensor_input(torch.float32, 2)
    strides = r.tensor_input(torch.float32, 1)
    if batch:
        i = r.task_index()
        pred = preds.slice(0, i, r.op("INT_ADD", i, 1))
    else:
        pred = preds
    box_cols = [c for c in range(5) if c != obj_col]
    p = pred.select(0, 0)
    pxy = r.stack([p.select(1, box_cols[0]), p.select(1, box_cols[1])], 1).sigmoid() if obj_col < 2 else p.slice(1, 0, 2).sigmoid()
    pwh = r.stack([p.select(1, box_cols[2]), p.select(1, box_cols[3])], 1) if obj_col < 4 else p.slice(1, 2, 4)
    obj = p.select(1, obj_col).sigmoid()
    cls = p.slice(1, 5, None).sigmoid()
    xy = (anchors.slice(1, 0, 2) + anchors.slice(1, 2, None)) * 0.5 + (pxy - 0.5) * strides.unsqueeze(-1)
    wh = (anchors.slice(1, 2, None) - anchors.slice(1, 0, 2)) * half * pwh.exp()
    if decode == "stack":
        boxes = r.stack([xy.select(1, 0) - wh.select(1, 0), xy.select(1, 1) - wh.select(1, 1),
                         xy.select(1, 0) + wh.select(1, 0), xy.select(1, 1) + wh.select(1, 1)], -1)
    elif decode == "cat":
        boxes = r.cat([xy - wh, xy + wh], 1)
    else:
        boxes = r.op("FULL", r.int_list([r.op("SIZE", anchors, 0), 4]), 0.0, dtype=torch.float32)
        boxes = boxes.select_rev(xy.select(1, 0) - wh.select(1, 0), 1, 0)
        boxes = boxes.select_rev(xy.select(1, 1) - wh.select(1, 1), 1, 1)
        boxes = boxes.select_rev(xy.select(1, 0) + wh.select(1, 0), 1, 2)
        boxes = boxes.select_rev(xy.select(1, 1) + wh.select(1, 1), 1, 3)
    if pad:
        cls = r.cat([cls, r.op("FULL", r.int_list([r.op("SIZE", anchors, 0), 1]), 0.0, dtype=torch.float32)], 1)
    keep = (cls.select(1, mask_class) if mask_class is not None else obj) >= thr
    if joined:
        r.output(r.cat([boxes, obj.unsqueeze(-1), cls], 1))
    else:
        r.output(boxes)
        r.output(cls)
        r.output(obj)
    r.compact_rows(keep)
    return r.finalize()
