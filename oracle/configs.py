"""ORACLE - test infrastructure only.  Nothing under oracle/ is imported by the
product (functs_amd/); only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py use it.

The five benchmark configurations as plain TorchScript programs, run by STOCK
PyTorch on the CPU.  This is the "reference's unfused TorchScript CPU path":
the reference's own result for a graph is, by construction, what the
TorchScript interpreter computes for it (every reference test is differential
against it: test/test_basic.py:50-52, test/test_immut_tensorexpr.py:22,
fait/testing/test_lowering.cpp:221, fait/fait.cpp:74-77).

The programs imitate, at the shapes of the five benchmark configurations:
  c1  examples/get_started.py:10-15 (verbatim)
  c2  functs/benchmark/ai_model/yolov3/yolov3_bbox.py:12-23, 206-243
      (sigmoid_ slice assign, objectness / class sigmoid, box decode written
      through four select assigns, confidence mask select)
  c3  functs/benchmark/ai_model/ssd/ssd_bbox.py:121-154, 163-172, 268
      (prior/variance decode through slice assigns, softmax, per-class
      threshold index select)
  c4  functs/benchmark/ai_model/lstm/lstm.py:79-133 (cell + per-step out[t] = h)
  c5  c2 over 16 images in a per-image loop (yolov3_bbox.py:233-241)

Pinned by: closed forms checked in tests/test_oracle.py (c1: out = b, rows
[0, n) += 1; c2/c3: zero logits give anchor / prior boxes; softmax rows sum to
one; c4: equality with torch.nn.LSTM on re-packed weights; compaction:
count == mask.sum(), rows in increasing source order).
"""
from typing import List, Tuple

import torch
from torch import Tensor

# ---------------------------------------------------------------------------
# c1: get_started loop
# ---------------------------------------------------------------------------


def c1_fn(a: Tensor, b: Tensor, n: int):
    a = a.clone()
    b = b.clone()
    for i in range(n):
        b[i] = b[i] + 1
    return b


def c1_inputs(seed: int = 0, size: int = 1024, n: int = -1):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(size, size, generator=g)
    b = torch.randn(size, size, generator=g)
    return a, b, (size if n < 0 else n)


# ---------------------------------------------------------------------------
# c2: YOLOv3-style post-processing
# ---------------------------------------------------------------------------
YOLO_BASE_SIZES = [[(116, 90), (156, 198), (373, 326)], [(30, 61), (62, 45), (59, 119)], [(10, 13), (16, 30), (33, 23)]]
YOLO_STRIDES = [32, 16, 8]
YOLO_GRIDS = [13, 26, 52]


def yolo_anchors(grids=YOLO_GRIDS) -> Tuple[Tensor, Tensor]:
    """anchors [N,4] (x1,y1,x2,y2) and strides [N]; cell-major, anchor-minor per
    level (yolov3_bbox.py:78-101)."""
    all_a, all_s = [], []
    for lvl, g in enumerate(grids):
        s = YOLO_STRIDES[lvl]
        base = torch.tensor([[s / 2.0 - 0.5 * w, s / 2.0 - 0.5 * h, s / 2.0 + 0.5 * w, s / 2.0 + 0.5 * h]
                             for (w, h) in YOLO_BASE_SIZES[lvl]], dtype=torch.float32)
        sx = torch.arange(0, g, dtype=torch.float32) * s
        sy = torch.arange(0, g, dtype=torch.float32) * s
        xx = sx.repeat(g)
        yy = sy.reshape(-1, 1).repeat(1, g).reshape(-1)
        shifts = torch.stack([xx, yy, xx, yy], dim=-1)
        a = (base[None, :, :] + shifts[:, None, :]).reshape(-1, 4)
        all_a.append(a)
        all_s.append(torch.full((a.size(0),), float(s)))
    return torch.cat(all_a).contiguous(), torch.cat(all_s).contiguous()


def c2_fn(pred: Tensor, anchors: Tensor, strides: Tensor):
    pred = pred.clone()
    pred[..., :2].sigmoid_()
    obj = pred[..., 4].sigmoid()
    cls = pred[..., 5:].sigmoid()
    p = pred[0]
    xy = (anchors[:, :2] + anchors[:, 2:]) * 0.5 + (p[:, :2] - 0.5) * strides.unsqueeze(-1)
    wh = (anchors[:, 2:] - anchors[:, :2]) * 0.5 * p[:, 2:4].exp()
    boxes = torch.zeros_like(anchors)
    boxes[:, 0] = xy[:, 0] - wh[:, 0]
    boxes[:, 1] = xy[:, 1] - wh[:, 1]
    boxes[:, 2] = xy[:, 0] + wh[:, 0]
    boxes[:, 3] = xy[:, 1] + wh[:, 1]
    keep = obj[0] >= 0.3
    return boxes[keep], cls[0][keep], obj[0][keep]


def c2_inputs(seed: int = 0, grids=YOLO_GRIDS, batch: int = 1):
    anchors, strides = yolo_anchors(grids)
    g = torch.Generator().manual_seed(seed)
    pred = torch.randn(batch, anchors.size(0), 85, generator=g)
    return pred, anchors, strides


# ---------------------------------------------------------------------------
# c3: SSD300-style post-processing
# ---------------------------------------------------------------------------


def c3_fn(loc: Tensor, conf: Tensor, priors: Tensor):
    l0 = loc[0]
    cxcy = priors[:, :2] + l0[:, :2] * 0.1 * priors[:, 2:]
    wh = priors[:, 2:] * torch.exp(l0[:, 2:] * 0.2)
    boxes = torch.zeros_like(priors)
    boxes[:, :2] = cxcy - wh / 2
    boxes[:, 2:] = cxcy + wh / 2
    scores = conf[0].softmax(-1)
    out_b: List[Tensor] = []
    out_s: List[Tensor] = []
    for c in range(1, scores.size(1)):
        sc = scores[:, c]
        m = sc > 0.05
        out_b.append(boxes[m])
        out_s.append(sc[m])
    return out_b, out_s


def c3_inputs(seed: int = 0, n_priors: int = 8732, n_cls: int = 81):
    g = torch.Generator().manual_seed(seed)
    loc = 0.5 * torch.randn(1, n_priors, 4, generator=g)
    conf = torch.randn(1, n_priors, n_cls, generator=g)
    priors = torch.rand(n_priors, 4, generator=g)
    return loc, conf, priors


# ---------------------------------------------------------------------------
# c4: stacked LSTM loop (weights laid out like lstm.py:58-65: [4, in, hidden])
# ---------------------------------------------------------------------------


def c4_fn(x: Tensor, wih: Tensor, whh: Tensor, bih: Tensor, bhh: Tensor):
    # x [T,B,H]; wih/whh [L,4,H,H]; bih/bhh [L,4,1,H]
    seq_len = x.size(0)
    n_layers = wih.size(0)
    batch = x.size(1)
    hidden = x.size(2)
    out = torch.zeros(seq_len, batch, hidden)
    state_h = torch.zeros(n_layers, batch, hidden)
    state_c = torch.zeros(n_layers, batch, hidden)
    for t in range(seq_len):
        cur = x[t]
        for j in range(n_layers):
            h = state_h[j]
            c = state_c[j]
            ih = torch.matmul(cur, wih[j]) + bih[j]
            hh = torch.matmul(h, whh[j]) + bhh[j]
            ingate = torch.sigmoid(ih[0] + hh[0])
            forgetgate = torch.sigmoid(ih[1] + hh[1])
            cellgate = torch.tanh(ih[2] + hh[2])
            outgate = torch.sigmoid(ih[3] + hh[3])
            c2 = (forgetgate * c) + (ingate * cellgate)
            h2 = outgate * torch.tanh(c2)
            state_c[j] = c2
            state_h[j] = h2
            cur = h2
        out[t] = cur
    return out, state_h, state_c


def c4_inputs(seed: int = 0, seq_len: int = 64, hidden: int = 512, layers: int = 2, batch: int = 1):
    g = torch.Generator().manual_seed(seed)

    def u(*shape):
        return torch.rand(*shape, generator=g) * 0.2 - 0.1

    x = torch.randn(seq_len, batch, hidden, generator=g)
    wih = u(layers, 4, hidden, hidden)
    whh = u(layers, 4, hidden, hidden)
    bih = u(layers, 4, 1, hidden)
    bhh = u(layers, 4, 1, hidden)
    return x, wih, whh, bih, bhh


# ---------------------------------------------------------------------------
# c5: c2 over a batch in a per-image loop
# ---------------------------------------------------------------------------


def c5_fn(preds: Tensor, anchors: Tensor, strides: Tensor):
    out_b: List[Tensor] = []
    out_c: List[Tensor] = []
    out_o: List[Tensor] = []
    for i in range(preds.size(0)):
        b, c, o = c2_fn(preds[i:i + 1], anchors, strides)
        out_b.append(b)
        out_c.append(c)
        out_o.append(o)
    return out_b, out_c, out_o


def c5_inputs(seed: int = 0, grids=YOLO_GRIDS, batch: int = 16):
    return c2_inputs(seed, grids, batch)


CONFIGS = {
    "c1": (c1_fn, c1_inputs),
    "c2": (c2_fn, c2_inputs),
    "c3": (c3_fn, c3_inputs),
    "c4": (c4_fn, c4_inputs),
    "c5": (c5_fn, c5_inputs),
}

_scripted = {}


def scripted(name: str):
    """torch.jit.script of the config function (stock TorchScript, CPU)."""
    if name not in _scripted:
        _scripted[name] = torch.jit.script(CONFIGS[name][0])
    return _scripted[name]


def run(name: str, *inputs):
    return scripted(name)(*inputs)


def threshold_margin(values: Tensor, thr: float) -> float:
    """Smallest distance of any value to the threshold: a mask computed on the
    GPU can only differ from the oracle's where this is within rounding."""
    return float((values - thr).abs().min()) if values.numel() else float("inf")
