"""Imperative tensor programs in the style of the reference's examples and
benchmark models.  They are inputs to functs_amd.jit.script / build.

  get_started      examples/get_started.py:10-15
  yolov3_postproc  functs/benchmark/ai_model/yolov3/yolov3_bbox.py:12-23, 206-243
  yolov3_batched   the per-image loop of yolov3_bbox.py:233-241
  ssd_postproc     functs/benchmark/ai_model/ssd/ssd_bbox.py:121-154, 163-172, 268
  lstm             functs/benchmark/ai_model/lstm/lstm.py:79-133
"""
from typing import List

import torch
from torch import Tensor


def get_started(a: Tensor, b: Tensor, n: int):
    a = a.clone()
    b = b.clone()
    for i in range(n):
        b[i] = b[i] + 1
    return b


def yolov3_postproc(pred: Tensor, anchors: Tensor, strides: Tensor):
    """pred [1, N, 85]; anchors [N, 4] corner form; strides [N]."""
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


def yolov3_batched(preds: Tensor, anchors: Tensor, strides: Tensor):
    """preds [B, N, 85]: one image per loop iteration."""
    out_b: List[Tensor] = []
    out_c: List[Tensor] = []
    out_o: List[Tensor] = []
    for i in range(preds.size(0)):
        b, c, o = yolov3_postproc(preds[i:i + 1], anchors, strides)
        out_b.append(b)
        out_c.append(c)
        out_o.append(o)
    return out_b, out_c, out_o


def ssd_postproc(loc: Tensor, conf: Tensor, priors: Tensor):
    """loc [1, N, 4], conf [1, N, C], priors [N, 4] centre form; variances 0.1 / 0.2."""
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


def lstm(x: Tensor, wih: Tensor, whh: Tensor, bih: Tensor, bhh: Tensor):
    """x [T, B, H]; wih / whh [L, 4, H, H]; bih / bhh [L, 4, 1, H] (gate order i, f, g, o)."""
    seq_len = x.size(0)
    n_layers = wih.size(0)
    batch = x.size(1)
    hidden = x.size(2)
    out = torch.zeros(seq_len, batch, hidden, device=x.device)
    state_h = torch.zeros(n_layers, batch, hidden, device=x.device)
    state_c = torch.zeros(n_layers, batch, hidden, device=x.device)
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


PROGRAMS = {
    "c1": get_started,
    "c2": yolov3_postproc,
    "c3": ssd_postproc,
    "c4": lstm,
    "c5": yolov3_batched,
}
