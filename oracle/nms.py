"""TEST INFRASTRUCTURE ONLY - CPU restatement of the detection tail that follows row compaction:
score sort, class-aware greedy NMS, top-k.  Never imported by the product.

The reference calls `torchvision.ops.nms` (functs/benchmark/ai_model/yolov3/yolov3_bbox.py:174-179,
functs/benchmark/ai_model/ssd/ssd_bbox.py:209-214).  torchvision is a third-party dependency that
the reference neither vendors nor pins (setup.py names no version) and that is not importable in
this image, so `nms` below restates its published algorithm (torchvision/csrc/ops/cpu/nms_kernel.cpp):
candidates in order of descending score (stable: equal scores keep their input order), a candidate
is kept unless an earlier kept one overlaps it with IoU > threshold, where
    inter = max(0, min(x2) - max(x1)) * max(0, min(y2) - max(y1));  iou = inter / (area_i + area_j - inter)
in float32.  PARITY UNPINNED against torchvision itself; pinned instead (tests/test_nms.py) by the
property that defines the greedy result uniquely (i is kept  <=>  no kept j ranked before i has
IoU(i, j) > threshold), by brute force over all subsets on tiny inputs, and by hand-computed cases
(ties, IoU exactly at the threshold, disjoint and nested boxes).

The functions around it follow the reference's own Python line by line in meaning:
  batched_nms      yolov3_bbox.py:141-171 / ssd_bbox.py:175-206, the `< split_thr` branch
  multiclass_nms   yolov3_bbox.py:104-138
  filter_scores_and_topk   ssd_bbox.py:163-172
"""
from typing import Tuple

import torch
from torch import Tensor


def iou_matrix(boxes: Tensor) -> Tensor:
    """IoU of every pair, float32, the operations in the order of the published kernel."""
    b = boxes.float()
    area = (b[:, 2] - b[:, 0]) * (b[:, 3] - b[:, 1])
    xx1 = torch.maximum(b[:, None, 0], b[None, :, 0])
    yy1 = torch.maximum(b[:, None, 1], b[None, :, 1])
    xx2 = torch.minimum(b[:, None, 2], b[None, :, 2])
    yy2 = torch.minimum(b[:, None, 3], b[None, :, 3])
    w = (xx2 - xx1).clamp(min=0)
    h = (yy2 - yy1).clamp(min=0)
    inter = w * h
    return inter / ((area[:, None] + area[None, :]) - inter)


def nms(boxes: Tensor, scores: Tensor, iou_threshold: float) -> Tensor:
    """Indices of the kept boxes, in order of descending score."""
    n = boxes.size(0)
    if n == 0:
        return torch.zeros(0, dtype=torch.long)
    order = torch.sort(scores.float(), descending=True, stable=True).indices
    b = boxes[order].float()
    x1, y1, x2, y2 = b[:, 0], b[:, 1], b[:, 2], b[:, 3]
    area = (x2 - x1) * (y2 - y1)
    suppressed = torch.zeros(n, dtype=torch.bool)
    keep = []
    for i in range(n):
        if suppressed[i]:
            continue
        keep.append(i)
        # box i against every later one: the row of iou_matrix, computed when it is needed
        w = (torch.minimum(x2[i], x2[i + 1:]) - torch.maximum(x1[i], x1[i + 1:])).clamp(min=0)
        h = (torch.minimum(y2[i], y2[i + 1:]) - torch.maximum(y1[i], y1[i + 1:])).clamp(min=0)
        inter = w * h
        iou = inter / ((area[i] + area[i + 1:]) - inter)
        suppressed[i + 1:] |= iou > iou_threshold   # NaN (0 / 0) compares false: degenerate boxes suppress nothing
    return order[torch.tensor(keep, dtype=torch.long)]


def batched_nms(boxes: Tensor, scores: Tensor, idxs: Tensor, iou_threshold: float = 0.45) -> Tuple[Tensor, Tensor]:
    """(dets [K, 5], keep [K]): boxes of different classes never suppress each other, because
    every class is moved by its own multiple of (largest coordinate + 1)."""
    if boxes.size(0) == 0:   # boxes.max() of the reference has no value here; nothing is kept
        return torch.zeros(0, 5), torch.zeros(0, dtype=torch.long)
    max_coordinate = boxes.max()
    offsets = idxs.to(boxes) * (max_coordinate + 1)
    boxes_for_nms = boxes + offsets[:, None]
    keep = nms(boxes_for_nms, scores, iou_threshold)
    dets = torch.cat([boxes[keep], scores[keep][:, None]], -1)
    return dets, keep


def multiclass_nms(multi_bboxes: Tensor, multi_scores: Tensor, score_factors: Tensor, score_thr: float = 0.05,
                   iou_threshold: float = 0.45, max_num: int = 100) -> Tuple[Tensor, Tensor, Tensor]:
    """multi_bboxes [K, 4], multi_scores [K, C] (the reference carries one more, all-zero column
    that it drops first), score_factors [K].  Returns (dets [<= max_num, 5], labels, index of the
    candidate as row * C + class)."""
    k, c = multi_scores.shape
    bboxes = multi_bboxes[:, None].expand(k, c, 4).reshape(-1, 4)
    scores = multi_scores.reshape(-1)
    labels = torch.arange(c, dtype=torch.long).reshape(1, -1).expand(k, c).reshape(-1)
    valid = scores > score_thr
    scores = scores * score_factors.reshape(-1, 1).expand(k, c).reshape(-1)
    inds = valid.nonzero()[:, 0]
    bboxes, scores, labels = bboxes[inds], scores[inds], labels[inds]
    dets, keep = batched_nms(bboxes, scores, labels, iou_threshold)
    return dets[:max_num], labels[keep][:max_num], inds[keep][:max_num]


def filter_scores_and_topk(scores: Tensor, score_thr: float, topk: int) -> Tuple[Tensor, Tensor, Tensor]:
    """scores [N, C] -> (scores, labels, row index) of the topk entries above the threshold."""
    valid_mask = scores > score_thr
    kept = scores[valid_mask]
    valid_idxs = torch.nonzero(valid_mask)
    num_topk = min(topk, valid_idxs.size(0))
    order = torch.sort(kept, descending=True, stable=True)
    topk_idxs = valid_idxs[order.indices[:num_topk]]
    return order.values[:num_topk], topk_idxs[:, 1], topk_idxs[:, 0]
