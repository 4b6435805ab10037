"""Imperative tensor programs in the style of the reference's examples and
benchmark models.  They are inputs to functs_amd.jit.script / build.

  get_started      examples/get_started.py:10-15
  yolov3_postproc  functs/benchmark/ai_model/yolov3/yolov3_bbox.py:12-23, 206-243
  yolov3_batched   the per-image loop of yolov3_bbox.py:233-241
  yolov3_batched_nms  the same loop with its tail, multiclass_nms (yolov3_bbox.py:104-138, 233-243)
  ssd_postproc     functs/benchmark/ai_model/ssd/ssd_bbox.py:121-154, 163-172, 268
  lstm             functs/benchmark/ai_model/lstm/lstm.py:79-133
  yolov3_head      the whole detection head up to the NMS as the reference's model structures it,
                   functs/benchmark/ai_model/yolov3/yolov3_bbox.py:12-23, 78-101, 194-243
  yolov3_head_nms  the same with the NMS tail of yolov3_bbox.py:104-179 behind the per-image filter
  attention_steps  functs/benchmark/simpleops/attention/attention.py:38-58
  delta2bbox       functs/benchmark/ai_model/ssd/ssd_bbox.py:121-154
"""
from typing import List, Tuple

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


def yolov3_batched_nms(preds: Tensor, anchors: Tensor, strides: Tensor):
    """The per-image loop of the reference's forward with its tail (yolov3_bbox.py:233-243): decode,
    confidence filter, then multiclass_nms (:104-138) on the kept rows.  functs::multiclass_nms is
    the operator that stands where the reference calls its Python function of that name."""
    det_results: List[Tuple[Tensor, Tensor]] = []
    for i in range(preds.size(0)):
        b, c, o = yolov3_postproc(preds[i:i + 1], anchors, strides)
        det_results.append(torch.ops.functs.multiclass_nms(b, c, o, 0.05, 0.45, 100, False))
    return det_results


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


def _level_grid_anchors(base: Tensor, feat_h: int, feat_w: int, stride: int):
    """Anchors of one pyramid level: the level's base anchors [A, 4] shifted to every cell
    (yolov3_bbox.py:78-101), cell-major, anchor-minor."""
    shift_x = torch.arange(0, feat_w, device=base.device).to(base.dtype) * stride
    shift_y = torch.arange(0, feat_h, device=base.device).to(base.dtype) * stride
    xx = shift_x.repeat(feat_h)
    yy = shift_y.view(-1, 1).repeat(1, feat_w).view(-1)
    shifts = torch.stack([xx, yy, xx, yy], dim=-1)
    return (base[None, :, :] + shifts[:, None, :]).view(-1, 4)


def _decode_stack(anchors: Tensor, pred: Tensor, stride: Tensor):
    """Centre / size decode, the corners joined by torch.stack (yolov3_bbox.py:12-23)."""
    xy = (anchors[..., :2] + anchors[..., 2:]) * 0.5 + (pred[..., :2] - 0.5) * stride
    wh = (anchors[..., 2:] - anchors[..., :2]) * 0.5 * pred[..., 2:].exp()
    boxes = torch.stack((xy[..., 0] - wh[..., 0], xy[..., 1] - wh[..., 1], xy[..., 0] + wh[..., 0], xy[..., 1] + wh[..., 1]), dim=-1)
    return boxes.clone()


def _yolov3_head_scores(pred_maps: List[Tensor], base_anchors: List[Tensor]):
    """yolov3_bbox.py:194-238: per level the NCHW map is permuted, flattened and its centre offsets
    squashed in place, the levels are concatenated, anchors and strides are generated from the
    feature-map sizes, the boxes are decoded for the whole batch and the class scores get a zero
    column.  Returns boxes [B, N, 4], class scores [B, N, C + 1], objectness [B, N]."""
    featmap_strides = [32, 16, 8]
    num_imgs = pred_maps[0].size(0)
    num_attrib = pred_maps[0].size(1) // base_anchors[0].size(0)
    mlvl_anchors: List[Tensor] = []
    flatten_preds: List[Tensor] = []
    flatten_strides: List[Tensor] = []
    for lvl in range(3):
        pm = pred_maps[lvl]
        stride = featmap_strides[lvl]
        mlvl_anchors.append(_level_grid_anchors(base_anchors[lvl], pm.size(2), pm.size(3), stride))
        pred = pm.permute(0, 2, 3, 1).reshape(num_imgs, -1, num_attrib).clone()
        pred[..., :2].sigmoid_()
        flatten_preds.append(pred.clone())
        flatten_strides.append(torch.full([pred.size(1)], float(stride), device=pm.device))
    anchors = torch.cat(mlvl_anchors)
    preds = torch.cat(flatten_preds, dim=1)
    strides = torch.cat(flatten_strides)
    bbox_preds = preds[..., :4]
    objectness = preds[..., 4].sigmoid()
    cls_scores = preds[..., 5:].sigmoid()
    bboxes = _decode_stack(anchors, bbox_preds, strides.unsqueeze(-1))
    padding = bboxes.new_zeros(num_imgs, bboxes.size(1), 1)
    cls_scores = torch.cat([cls_scores, padding], dim=-1)
    return bboxes, cls_scores, objectness


def yolov3_head(pred_maps: List[Tensor], base_anchors: List[Tensor]):
    """The detection head as the reference's model structures it (yolov3_bbox.py:194-243), up to the
    NMS: the scores of _yolov3_head_scores, then a loop over the images that keeps the rows whose
    objectness passes the confidence threshold.
    pred_maps: per level [B, A * (5 + C), H, W]; base_anchors: per level [A, 4]."""
    bboxes, cls_scores, objectness = _yolov3_head_scores(pred_maps, base_anchors)
    out_b: List[Tensor] = []
    out_s: List[Tensor] = []
    out_o: List[Tensor] = []
    for i in range(bboxes.size(0)):
        o = objectness[i]
        keep = o >= 0.005
        out_b.append(bboxes[i][keep, :])
        out_s.append(cls_scores[i][keep, :])
        out_o.append(o[keep])
    return out_b, out_s, out_o


def yolov3_head_nms(pred_maps: List[Tensor], base_anchors: List[Tensor]):
    """The whole of the reference's forward (yolov3_bbox.py:194-243): the head, and per image the
    confidence filter followed by multiclass_nms (:104-138) on the kept rows, whose class scores
    carry the padding column that multiclass_nms cuts off again (:113)."""
    bboxes, cls_scores, objectness = _yolov3_head_scores(pred_maps, base_anchors)
    det_results: List[Tuple[Tensor, Tensor]] = []
    for i in range(bboxes.size(0)):
        o = objectness[i]
        keep = o >= 0.005
        det_results.append(torch.ops.functs.multiclass_nms(bboxes[i][keep, :], cls_scores[i][keep, :], o[keep], 0.05, 0.45, 100, True))
    return det_results


def attention_steps(x: Tensor, k: Tensor, v: Tensor, wq: Tensor, wk: Tensor, wv: Tensor, wo: Tensor, start_len: int):
    """Single-query attention over a growing key / value cache (attention.py:38-58): every step
    writes one row of both caches at a position that the loop carries, the products stay library
    GEMMs, scale and softmax fuse.  x [B, H, 1, D]; k, v [B, H, L, D], filled up to start_len;
    wq, wk, wv, wo [H, D, D]."""
    k = k + 0.0
    v = v + 0.0
    batch = x.size(0)
    heads = x.size(1)
    depth = x.size(3)
    gen_id = start_len
    for i in range(k.size(2) - start_len):
        q = torch.matmul(x, wq)
        k[:, :, gen_id, :] = torch.reshape(torch.matmul(x, wk), (batch, heads, depth))
        v[:, :, gen_id, :] = torch.reshape(torch.matmul(x, wv), (batch, heads, depth))
        attn = torch.matmul(k, q.transpose(2, 3)).transpose(2, 3)
        attn = attn * 0.125
        attn = torch.softmax(attn, dim=3)
        x = torch.matmul(attn, v)
        x = torch.matmul(x, wo)
        gen_id = gen_id + 1
    return k.clone(), v.clone(), x.clone()


def delta2bbox(rois: Tensor, deltas: Tensor):
    """Box regression of an SSD-style head (ssd_bbox.py:121-154): deltas [N, 4 * C] (dx, dy, dw, dh
    per class) applied to rois [N, 4] (corners), the size deltas clamped, the corners clamped to the
    image through in-place clamps on strided slices."""
    num_classes = deltas.size(1) // 4
    deltas = deltas.reshape(-1, 4)
    stds = torch.tensor([0.1, 0.1, 0.2, 0.2], dtype=deltas.dtype, device=deltas.device).view(1, -1)
    denorm = deltas * stds
    dxy = denorm[:, :2]
    dwh = denorm[:, 2:]
    rois_ = rois.repeat(1, num_classes).reshape(-1, 4)
    pxy = (rois_[:, :2] + rois_[:, 2:]) * 0.5
    pwh = rois_[:, 2:] - rois_[:, :2]
    dwh = dwh.clamp(min=-4.135, max=4.135)
    gxy = pxy + pwh * dxy
    gwh = pwh * dwh.exp()
    bboxes = torch.cat([gxy - gwh * 0.5, gxy + gwh * 0.5], dim=-1)
    bboxes[..., 0::2].clamp_(min=0, max=320)
    bboxes[..., 1::2].clamp_(min=0, max=320)
    return bboxes.clone()


PROGRAMS = {
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
