"""Seeded synthetic inputs of the benchmark programs (CPU tensors; callers copy them to
the GPU).  Shapes follow the configurations the reference reports on: get_started
[1024,1024] (examples/get_started.py:29-33), YOLOv3 head outputs over the 13/26/52 grids
with three anchors each (functs/benchmark/ai_model/yolov3/yolov3_bbox.py:78-101, 190-193),
SSD300 priors (ssd_bbox.py:96-118), LSTM 2 x 512 over 64 steps (lstm.py:58-65)."""
from typing import Tuple

import torch
from torch import Tensor

YOLO_BASE_SIZES = (((116, 90), (156, 198), (373, 326)), ((30, 61), (62, 45), (59, 119)), ((10, 13), (16, 30), (33, 23)))
YOLO_STRIDES = (32, 16, 8)
YOLO_GRIDS = (13, 26, 52)


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def get_started(seed: int = 0, size: int = 1024, n: int = -1):
    g = _gen(seed)
    a = torch.randn(size, size, generator=g)
    b = torch.randn(size, size, generator=g)
    return a, b, (size if n < 0 else n)


def yolo_anchors(grids=YOLO_GRIDS) -> Tuple[Tensor, Tensor]:
    """anchors [N,4] as x1,y1,x2,y2 and strides [N]; per level cell-major, anchor-minor."""
    boxes, strides = [], []
    for level, cells in enumerate(grids):
        s = float(YOLO_STRIDES[level])
        half = torch.tensor(YOLO_BASE_SIZES[level], dtype=torch.float32) * 0.5            # [3,2] half w,h
        centre = torch.full((1, 2), s / 2.0)
        base = torch.cat([centre - half, centre + half], dim=1)                            # [3,4]
        step = torch.arange(cells, dtype=torch.float32) * s
        xs = step.repeat(cells)
        ys = step.repeat_interleave(cells)
        shift = torch.stack([xs, ys, xs, ys], dim=1)                                       # [cells^2,4]
        level_boxes = (shift[:, None, :] + base[None, :, :]).reshape(-1, 4)
        boxes.append(level_boxes)
        strides.append(torch.full((level_boxes.size(0),), s))
    return torch.cat(boxes).contiguous(), torch.cat(strides).contiguous()


def yolov3_postproc(seed: int = 0, grids=YOLO_GRIDS, batch: int = 1):
    anchors, strides = yolo_anchors(grids)
    pred = torch.randn(batch, anchors.size(0), 85, generator=_gen(seed))
    return pred, anchors, strides


def yolov3_batched(seed: int = 0, grids=YOLO_GRIDS, batch: int = 16):
    return yolov3_postproc(seed, grids, batch)


def yolov3_batched_nms(seed: int = 0, grids=YOLO_GRIDS, batch: int = 16, shift: float = 6.0):
    """The inputs of yolov3_batched with the class logits lowered by `shift`, so that about 1e-3 of
    the class scores pass the tail's 0.05, as behind a trained head (with N(0, 1) logits nearly all
    (row, class) pairs of an image would be candidates of the NMS)."""
    preds, anchors, strides = yolov3_postproc(seed, grids, batch)
    preds[..., 5:] -= shift
    return preds, anchors, strides


def ssd_postproc(seed: int = 0, n_priors: int = 8732, n_cls: int = 81):
    g = _gen(seed)
    loc = 0.5 * torch.randn(1, n_priors, 4, generator=g)
    conf = torch.randn(1, n_priors, n_cls, generator=g)
    priors = torch.rand(n_priors, 4, generator=g)
    return loc, conf, priors


def lstm(seed: int = 0, seq_len: int = 64, hidden: int = 512, layers: int = 2, batch: int = 1):
    g = _gen(seed)

    def uniform(*shape):
        return torch.rand(*shape, generator=g) * 0.2 - 0.1

    x = torch.randn(seq_len, batch, hidden, generator=g)
    wih = uniform(layers, 4, hidden, hidden)
    whh = uniform(layers, 4, hidden, hidden)
    bih = uniform(layers, 4, 1, hidden)
    bhh = uniform(layers, 4, 1, hidden)
    return x, wih, whh, bih, bhh


def yolov3_head(seed: int = 0, batch: int = 16, grids=YOLO_GRIDS, classes: int = 80):
    """Per level the NCHW map of the head [B, 3 * (5 + C), G, G] and its base anchors [3, 4]."""
    g = _gen(seed)
    maps = [torch.randn(batch, 3 * (5 + classes), cells, cells, generator=g) for cells in grids]
    bases = []
    for level in range(len(grids)):
        half = torch.tensor(YOLO_BASE_SIZES[level], dtype=torch.float32) * 0.5
        centre = torch.full((1, 2), YOLO_STRIDES[level] / 2.0)
        bases.append(torch.cat([centre - half, centre + half], dim=1))
    return maps, bases


def yolov3_head_nms(seed: int = 0, batch: int = 16, grids=YOLO_GRIDS, classes: int = 80, shift: float = 6.0):
    """The inputs of yolov3_head with the class logits of every anchor lowered by `shift` (see
    yolov3_batched_nms)."""
    maps, bases = yolov3_head(seed, batch, grids, classes)
    for m in maps:
        m.view(batch, 3, 5 + classes, m.size(2), m.size(3))[:, :, 5:] -= shift
    return maps, bases


def attention_steps(seed: int = 0, batch: int = 1, heads: int = 12, length: int = 50, depth: int = 64, start: int = 32):
    g = _gen(seed)
    x = torch.randn(batch, heads, 1, depth, generator=g)
    k = torch.zeros(batch, heads, length, depth)
    v = torch.zeros(batch, heads, length, depth)
    k[:, :, :start] = torch.randn(batch, heads, start, depth, generator=g)
    v[:, :, :start] = torch.randn(batch, heads, start, depth, generator=g)
    bound = (6.0 / (2 * depth)) ** 0.5
    ws = [(torch.rand(heads, depth, depth, generator=g) * 2 - 1) * bound for _ in range(4)]
    return (x, k, v) + tuple(ws) + (start,)


def delta2bbox(seed: int = 0, n: int = 8732, classes: int = 4):
    g = _gen(seed)
    rois = torch.rand(n, 4, generator=g) * 150
    rois[:, 2:] += rois[:, :2]
    deltas = torch.randn(n, 4 * classes, generator=g)
    return rois, deltas


INPUTS = {
    "c1": get_started,
    "c2": yolov3_postproc,
    "c3": ssd_postproc,
    "c4": lstm,
    "c5": yolov3_batched,
    "c5_nms": yolov3_batched_nms,
    "yolo_head": yolov3_head,
    "yolo_head_nms": yolov3_head_nms,
    "attention": attention_steps,
    "delta2bbox": delta2bbox,
}
