"""The step behind row compaction in the reference's detection programs - score threshold, sort by
descending score, class-aware greedy NMS, top-k - as ONE launch for all images (fx_sort_nms).

Same names and argument meaning as the reference's Python
(functs/benchmark/ai_model/yolov3/yolov3_bbox.py:104-179, functs/benchmark/ai_model/ssd/ssd_bbox.py:175-214),
which runs it as a chain of ATen and torchvision kernels with host synchronisations in between
(nonzero, index, max, sort, torchvision::nms, slicing).  Differences, all stated where they occur:
the batched forms take every image at once, the class scores carry no padding column, and the
per-class branch the reference takes from 10000 candidates on is the same function here up to
16384 candidates per image (more are refused).

GPU tensors only: there is no host fallback.
"""
import ctypes
from typing import List, Optional, Sequence, Tuple

import torch
from torch import Tensor

from . import _lib
from ._lib import C, FxNmsDesc, check, lib

MAX_CANDIDATES = C["FX_NMS_MAX_CANDIDATES"]
MAX_OUT = C["FX_NMS_MAX_OUT"]


def _f32(t: Tensor, what: str) -> Tensor:
    if not t.is_cuda:
        raise _lib.FxError(C["FX_E_INVALID"], "%s: the detection tail runs on the GPU only (got a %s tensor)" % (what, t.device))
    if t.dtype != torch.float32:
        raise _lib.FxError(C["FX_E_INVALID"], "%s must be float32" % what)
    # images may lie at any distance from each other (dimension 0), each one contiguous
    if t.dim() >= 2 and t.size(0) > 0 and t[0].is_contiguous() and t.stride(0) >= t[0].numel():
        return t
    return t.contiguous()


class NmsResult:
    """Fixed-shape outputs of one launch, all on the device: dets [T, max_num, 5], labels / index
    [T, max_num] and the number of kept boxes per image `n` (int32; rows from n[t] on are zero).
    Nothing here waits for the device; `lists()` does, to cut the outputs to size."""

    def __init__(self, dets, labels, index, n, stream):
        self.dets, self.labels, self.index, self.n, self.stream = dets, labels, index, n, stream

    def lists(self) -> List[Tuple[Tensor, Tensor, Tensor]]:
        """Per image (dets [K, 5], labels [K], index [K]), the way the reference returns them."""
        n = self.n.cpu()   # waits for the launch
        if bool((n < 0).any()):   # FX_NMS_OVERFLOW
            lib.fx_async_error_take(C["FX_ASYNC_NMS_CAPACITY"])   # this report is handled here; others stay
            raise _lib.FxError(C["FX_E_LIMIT"], "fx_sort_nms: an image has more candidates than the launch was sized for "
                               "(key_capacity; at most %d)" % MAX_CANDIDATES)
        out = []
        for t in range(self.dets.size(0)):
            k = int(n[t])
            out.append((self.dets[t, :k], self.labels[t, :k], self.index[t, :k]))
        return out


_workspaces = {}


def _workspace(dev, stream, n_tasks, key_capacity):
    """Counters and key buffers of the kernel, one per (device, stream) and layout (number of
    images, key capacity): cleared when allocated, every launch leaves the counters clear."""
    nbytes = lib.fx_sort_nms_workspace_bytes(n_tasks, key_capacity)
    key = (dev.index, stream.cuda_stream, n_tasks, nbytes)
    ws = _workspaces.get(key)
    if ws is None:
        with torch.cuda.stream(stream):
            ws = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=dev)
        _workspaces[key] = ws
    return ws


def _launch(mode, boxes, scores, factors, labels, counts, n_classes, score_thr, iou_thr, max_num, key_capacity):
    dev = boxes.device
    T, rows = boxes.size(0), boxes.size(1)
    dets = torch.empty(T, max_num, 5, device=dev)
    out_labels = torch.empty(T, max_num, dtype=torch.long, device=dev)
    out_index = torch.empty(T, max_num, dtype=torch.long, device=dev)
    n_out = torch.empty(T, dtype=torch.int32, device=dev)
    d = FxNmsDesc()
    d.mode, d.n_tasks, d.rows, d.n_classes = mode, T, rows, n_classes
    d.boxes, d.boxes_task_stride = boxes.data_ptr(), boxes.stride(0)
    d.scores, d.scores_task_stride = scores.data_ptr(), scores.stride(0)
    if factors is not None:
        d.factors, d.factors_task_stride = factors.data_ptr(), factors.stride(0)
    if labels is not None:
        d.labels, d.labels_task_stride = labels.data_ptr(), labels.stride(0)
    if counts is not None:
        d.counts = counts.data_ptr()
    d.score_thr, d.iou_thr, d.max_num = score_thr, iou_thr, max_num
    d.key_capacity = key_capacity
    d.dets, d.out_labels, d.out_index, d.n_out = dets.data_ptr(), out_labels.data_ptr(), out_index.data_ptr(), n_out.data_ptr()
    stream = torch.cuda.current_stream(dev)
    if T > 0:
        ws = _workspace(dev, stream, T, key_capacity)
        d.workspace, d.workspace_bytes = ws.data_ptr(), ws.numel()
    with torch.cuda.device(dev):
        check(lib.fx_sort_nms(ctypes.byref(d), ctypes.c_void_p(stream.cuda_stream)))
    return NmsResult(dets, out_labels, out_index, n_out, stream)


def _counts(counts: Optional[Tensor], T: int) -> Optional[Tensor]:
    """Valid rows per image: int32, on the device or in pinned host memory (what a compaction
    wrote for its caller is read by the kernel, not by the host)."""
    if counts is None:
        return None
    if counts.dtype != torch.int32 or counts.numel() != T or not (counts.is_cuda or counts.is_pinned()):
        raise _lib.FxError(C["FX_E_INVALID"], "counts must be %d int32 values on the device or in pinned host memory" % T)
    return counts.contiguous()


def multiclass_nms_batched(multi_bboxes: Tensor, multi_scores: Tensor, score_factors: Optional[Tensor],
                           counts: Optional[Tensor] = None, score_thr: float = 0.05, iou_threshold: float = 0.45,
                           max_num: int = 100, key_capacity: int = MAX_CANDIDATES) -> NmsResult:
    """multiclass_nms (yolov3_bbox.py:104-138) for every image at once: multi_bboxes [T, K, 4],
    multi_scores [T, K, C] (no padding column), score_factors [T, K]; rows from counts[t] on are
    ignored."""
    b = _f32(multi_bboxes, "multi_bboxes")
    s = _f32(multi_scores, "multi_scores")
    f = None if score_factors is None else _f32(score_factors, "score_factors")
    if b.dim() != 3 or b.size(2) != 4 or s.dim() != 3 or s.shape[:2] != b.shape[:2] or (f is not None and f.shape != b.shape[:2]):
        raise _lib.FxError(C["FX_E_INVALID"], "multiclass_nms: expected boxes [T, K, 4], scores [T, K, C], factors [T, K]")
    return _launch(1, b, s, f, None, _counts(counts, b.size(0)), s.size(2), score_thr, iou_threshold, max_num, key_capacity)


def multiclass_nms(multi_bboxes: Tensor, multi_scores: Tensor, score_factors: Tensor, score_thr: float = 0.05,
                   iou_threshold: float = 0.45, max_num: int = 100) -> Tuple[Tensor, Tensor]:
    """One image, the reference's signature and return value: (dets [<= max_num, 5], labels)."""
    r = multiclass_nms_batched(multi_bboxes[None], multi_scores[None], score_factors[None], None, score_thr, iou_threshold, max_num)
    dets, labels, _ = r.lists()[0]
    return dets, labels


def batched_nms_batched(boxes: Tensor, scores: Tensor, idxs: Optional[Tensor], counts: Optional[Tensor] = None,
                        iou_threshold: float = 0.45, max_num: int = MAX_OUT, score_thr: float = float("-inf"),
                        key_capacity: int = MAX_CANDIDATES) -> NmsResult:
    """batched_nms (ssd_bbox.py:175-206) followed by [:max_num], for every image at once:
    boxes [T, N, 4], scores [T, N], idxs [T, N] int64 class of each box (None: one class)."""
    b = _f32(boxes, "boxes")
    s = _f32(scores, "scores")
    if b.dim() != 3 or b.size(2) != 4 or s.shape != b.shape[:2]:
        raise _lib.FxError(C["FX_E_INVALID"], "batched_nms: expected boxes [T, N, 4], scores [T, N]")
    lab = None
    if idxs is not None:
        if idxs.dtype != torch.long or idxs.shape != s.shape or not idxs.is_cuda:
            raise _lib.FxError(C["FX_E_INVALID"], "batched_nms: idxs must be int64 [T, N] on the GPU")
        lab = idxs.contiguous()
    return _launch(0, b, s, None, lab, _counts(counts, b.size(0)), 1, score_thr, iou_threshold, max_num, key_capacity)


def batched_nms(boxes: Tensor, scores: Tensor, idxs: Tensor, iou_threshold: float = 0.45, max_num: int = MAX_OUT) -> Tuple[Tensor, Tensor]:
    """One image, the reference's signature and return value: (dets [K, 5], keep [K])."""
    r = batched_nms_batched(boxes[None], scores[None], idxs[None], None, iou_threshold, max_num)
    dets, _, keep = r.lists()[0]
    return dets, keep


def nms(boxes: Tensor, scores: Tensor, iou_threshold: float, max_num: int = MAX_OUT) -> Tensor:
    """torchvision.ops.nms's contract (indices of the kept boxes by descending score), up to
    max_num of them."""
    r = batched_nms_batched(boxes[None], scores[None], None, None, iou_threshold, max_num)
    return r.lists()[0][2]
