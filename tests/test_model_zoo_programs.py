"""Programs in the style of the reference's recurrent benchmark models (its NASRNN cell loop,
functs/benchmark/ai_model/nasrnn/nasrnn.py:39-101, and its seq2seq greedy decoder, a `while` loop
that ends on a value computed on the device and writes one row of an int64 result per step,
functs/benchmark/ai_model/seq2seq/seq2seq.py:95-142), written here as functions with the weights
as arguments.  Their loops carry state, so they stay host loops around one fused region per step
(the matrix products are ATen's); the tests check the graphs and, on the GPU, the results against
eager mode (1e-4 relative after the recurrence, the decoder's tokens exactly).  Two detection
post-processing programs follow: an anchor-free head over pyramid levels of different sizes (one
compacting map over ragged tasks) and mask assembly behind a library GEMM (one dense region)."""
from typing import List

import pytest
import torch
from torch import Tensor

import functs_amd.aot as aot
import functs_amd.jit as fj


def nas_cell_loop(inputs: Tensor, w_ih: Tensor, w_hh: Tensor):
    """inputs [T, B, I]; w_ih [8, I, H]; w_hh [8, H, H]."""
    state_c = torch.zeros(inputs.size(1), w_hh.size(2), device=inputs.device)
    state_m = torch.zeros(inputs.size(1), w_hh.size(2), device=inputs.device)
    for i in range(inputs.size(0)):
        ih = torch.matmul(inputs[i], w_ih)
        hh = torch.matmul(state_m, w_hh)
        l1_0 = torch.sigmoid(ih[0] + hh[0])
        l1_1 = torch.relu(ih[1] + hh[1])
        l1_2 = torch.sigmoid(ih[2] + hh[2])
        l1_3 = torch.relu(ih[3] + hh[3])
        l1_4 = torch.tanh(ih[4] + hh[4])
        l1_5 = torch.sigmoid(ih[5] + hh[5])
        l1_6 = torch.tanh(ih[6] + hh[6])
        l1_7 = torch.sigmoid(ih[7] + hh[7])
        l2_0 = torch.tanh(torch.tanh(l1_0 * l1_1) + state_c)
        l2_1 = torch.tanh(l1_2 + l1_3)
        l2_2 = torch.tanh(l1_4 * l1_5)
        l2_3 = torch.sigmoid(l1_6 + l1_7)
        state_c = l2_0 * l2_1
        state_m = torch.tanh(state_c * torch.tanh(l2_2 + l2_3))
    return state_c + state_m


def greedy_decoder(emb: Tensor, w_ih: Tensor, w_hh: Tensor, b_ih: Tensor, b_hh: Tensor, w_out: Tensor, b_out: Tensor,
                   std: Tensor, h: Tensor, c: Tensor, max_length: int):
    """emb [V, H]; w_ih / w_hh [4, H, H]; b_ih / b_hh [4, H]; w_out [H, V]; b_out [V]; std [L, B, V]
    (a bias per step that steers the tokens); h, c [B, H].  Ends when every row emits token 0."""
    batch = h.size(0)
    tokens = torch.zeros(max_length, batch, dtype=torch.int64, device=h.device)
    output = torch.full([batch], 1, dtype=torch.int64, device=h.device)
    cond = True
    step = 0
    while cond:
        x = emb[output]
        ih = torch.matmul(x, w_ih)
        hh = torch.matmul(h, w_hh)
        ingate = torch.sigmoid(ih[0] + b_ih[0] + hh[0] + b_hh[0])
        forgetgate = torch.sigmoid(ih[1] + b_ih[1] + hh[1] + b_hh[1])
        cellgate = torch.tanh(ih[2] + b_ih[2] + hh[2] + b_hh[2])
        outgate = torch.sigmoid(ih[3] + b_ih[3] + hh[3] + b_hh[3])
        c = forgetgate * c + ingate * cellgate
        h = outgate * torch.tanh(c)
        output = (torch.matmul(h, w_out) + b_out + std[step]).argmax(1)
        tokens[step] = output
        step = step + 1
        cond = bool((torch.max(output) > 0).item()) and step < max_length
    return tokens, h


def fcos_levels(cls_scores: List[Tensor], bbox_preds: List[Tensor], centerness: List[Tensor], points: List[Tensor],
                strides: List[float]):
    """An anchor-free head in the style of the reference's FCOS post-processing
    (functs/benchmark/ai_model/fcos/fcos_bbox.py): per level, NCHW maps are flattened, scores are
    weighted by the centre-ness, boxes are decoded from distances to the four sides, and the rows
    whose best class passes a threshold are kept.  Levels differ in size: a map with ragged tasks."""
    out_boxes: List[Tensor] = []
    out_scores: List[Tensor] = []
    for i in range(len(cls_scores)):
        cls = cls_scores[i]
        scores = cls[0].permute(1, 2, 0).reshape(-1, cls.size(1)).sigmoid()
        ctr = centerness[i][0].permute(1, 2, 0).reshape(-1).sigmoid()
        dist = bbox_preds[i][0].permute(1, 2, 0).reshape(-1, 4) * strides[i]
        scores = scores * ctr.unsqueeze(-1)
        pts = points[i]
        boxes = torch.stack([pts[:, 0] - dist[:, 0], pts[:, 1] - dist[:, 1], pts[:, 0] + dist[:, 2], pts[:, 1] + dist[:, 3]], -1)
        best, _ = scores.max(1)
        keep = best > 0.3
        out_boxes.append(boxes[keep])
        out_scores.append(scores[keep])
    return out_boxes, out_scores


def crop_masks(proto: Tensor, coeffs: Tensor, boxes: Tensor):
    """Mask assembly in the style of the reference's YOLACT post-processing
    (functs/benchmark/ai_model/yolact/yolact_mask.py): prototype masks are combined linearly per
    detection (a library GEMM, outside any region), squashed, and cut to the detection's box with
    comparisons against pixel coordinates; the elementwise part is one region."""
    h, w, n = proto.size(0), proto.size(1), coeffs.size(0)
    masks = (proto @ coeffs.t()).sigmoid()                        # [h, w, n]
    rows = torch.arange(h, device=proto.device, dtype=proto.dtype).view(-1, 1, 1).expand(h, w, n)
    cols = torch.arange(w, device=proto.device, dtype=proto.dtype).view(1, -1, 1).expand(h, w, n)
    x1, y1, x2, y2 = boxes[:, 0], boxes[:, 1], boxes[:, 2], boxes[:, 3]
    inside = (cols >= x1.view(1, 1, -1)) & (cols < x2.view(1, 1, -1)) & (rows >= y1.view(1, 1, -1)) & (rows < y2.view(1, 1, -1))
    return masks * inside.to(masks.dtype)


def _crop_inputs(seed=0, h=34, w=38, k=8, n=5):
    g = torch.Generator().manual_seed(seed)
    proto = torch.randn(h, w, k, generator=g)
    coeffs = torch.randn(n, k, generator=g)
    xy = torch.rand(n, 2, generator=g) * 20
    boxes = torch.cat([xy, xy + torch.rand(n, 2, generator=g) * 15 + 2], 1)
    return [proto, coeffs, boxes]


def _fcos_inputs(seed=0, classes=20, sizes=((20, 24), (10, 12), (5, 6))):
    g = torch.Generator().manual_seed(seed)
    cls, box, ctr, pts, strides = [], [], [], [], []
    for k, (h, w) in enumerate(sizes):
        cls.append(torch.randn(1, classes, h, w, generator=g))
        box.append(torch.rand(1, 4, h, w, generator=g) * 4)
        ctr.append(torch.randn(1, 1, h, w, generator=g) + 1.0)
        stride = 8.0 * 2 ** k
        ys, xs = torch.meshgrid(torch.arange(h), torch.arange(w), indexing="ij")
        pts.append(torch.stack([xs.reshape(-1), ys.reshape(-1)], -1).float() * stride + stride / 2)
        strides.append(stride)
    return [cls, box, ctr, pts, strides]


def _nas_inputs(seed=0, T=12, B=2, I=64, H=64):
    g = torch.Generator().manual_seed(seed)
    return [torch.rand(T, B, I, generator=g), (torch.rand(8, I, H, generator=g) - 0.5) * 0.3,
            (torch.rand(8, H, H, generator=g) - 0.5) * 0.3]


def _decoder_inputs(seed=0, V=50, H=32, B=3, L=9, stop_at=6):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: (torch.rand(*s, generator=g) - 0.5) * 0.4
    std = torch.zeros(L, B, V)
    for t in range(L):                      # steer: token 1 + t % 7 until stop_at, then token 0 for every row
        std[t, :, 0 if t >= stop_at else 1 + t % 7] = 1000.0
    return [r(V, H), r(4, H, H), r(4, H, H), r(4, H), r(4, H), r(H, V), r(V), std, r(B, H), r(B, H), L]


def _kinds(block, out=None):
    out = [] if out is None else out
    for n in block.nodes():
        out.append(n.kind())
        for b in n.blocks():
            _kinds(b, out)
    return out


def _cuda(args):
    def go(a):
        if isinstance(a, torch.Tensor):
            return a.cuda()
        if isinstance(a, list):
            return [go(e) for e in a]
        return a
    return [go(a) for a in args]


def test_the_cell_of_a_step_is_one_region():
    built = fj.build(fj.script(nas_cell_loop), _nas_inputs())
    kinds = _kinds(built.graph)
    assert kinds.count("prim::Loop") == 1 and kinds.count("aten::matmul") == 2
    assert kinds.count("tssa::ParallelFunctor") == 1          # inside the loop: the whole cell
    for k in ("aten::sigmoid", "aten::tanh", "aten::relu"):
        assert k not in kinds                                  # nothing of the cell is left outside


def test_the_decoder_is_functionalized_and_keeps_its_while_loop():
    f = fj.script(greedy_decoder)
    kinds = _kinds(f.graph)
    assert "aten::copy_" not in kinds and "aten::index_put_" not in kinds
    assert "immut::select_rev" in kinds                        # tokens[step] = output
    built = fj.build(f, _decoder_inputs())
    kinds = _kinds(built.graph)
    assert kinds.count("prim::Loop") == 1 and "aten::item" in kinds


@pytest.mark.gpu
def test_nas_cell_loop_equals_eager():
    args = _nas_inputs()
    built = fj.build(fj.script(nas_cell_loop), args)
    total0, _ = aot.launch_stats()
    got = built(*_cuda(args))
    torch.cuda.synchronize()
    total1, _ = aot.launch_stats()
    assert total1 - total0 == args[0].size(0)                  # one launch per step
    torch.testing.assert_close(got.cpu(), nas_cell_loop(*args), rtol=1e-4, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("stop_at", [1, 6, 100])
def test_greedy_decoder_equals_eager(stop_at):
    args = _decoder_inputs(stop_at=stop_at)
    built = fj.build(fj.script(greedy_decoder), args)
    tokens, h = built(*_cuda(args))
    ref_tokens, ref_h = greedy_decoder(*args)
    assert torch.equal(tokens.cpu(), ref_tokens)
    steps = min(stop_at + 1, args[-1])
    assert int((ref_tokens.sum(1) > 0).sum()) == min(stop_at, args[-1]) and steps >= 1
    torch.testing.assert_close(h.cpu(), ref_h, rtol=1e-4, atol=1e-6)


def test_the_anchor_free_head_is_one_map_over_ragged_levels():
    built = fj.build(fj.script(fcos_levels), _fcos_inputs())
    kinds = _kinds(built.graph)
    fs = [n for n in built.graph.nodes() if n.kind() == "tssa::ParallelFunctor"]
    assert "prim::Loop" not in kinds and len(fs) == 1
    f = fs[0]
    assert f.i("is_parallel_map") == 1 and f.i("compact_rows") == 1 and f.i("parallel_degree") == 3


@pytest.mark.gpu
def test_anchor_free_head_equals_eager():
    args = _fcos_inputs()
    built = fj.build(fj.script(fcos_levels), args)
    total0, _ = aot.launch_stats()
    boxes, scores = built(*_cuda(args))
    torch.cuda.synchronize()
    total1, _ = aot.launch_stats()
    assert total1 - total0 == 2                                # count + scatter over the three levels together
    ref_boxes, ref_scores = fcos_levels(*args)
    assert [t.shape for t in boxes] == [t.shape for t in ref_boxes] and sum(t.shape[0] for t in ref_boxes) > 50
    for a, b in zip(boxes, ref_boxes):
        torch.testing.assert_close(a.cpu(), b, rtol=1e-5, atol=1e-5)
    for a, b in zip(scores, ref_scores):
        torch.testing.assert_close(a.cpu(), b, rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_mask_assembly_equals_eager():
    args = _crop_inputs()
    built = fj.build(fj.script(crop_masks), args)
    got = built(*_cuda(args))
    ref = crop_masks(*args)
    assert got.shape == ref.shape and (ref != 0).sum().item() > 100 and (ref == 0).sum().item() > 100
    torch.testing.assert_close(got.cpu(), ref, rtol=1e-5, atol=1e-6)
    assert "tssa::ParallelFunctor" in _kinds(built.graph)          # the elementwise part runs as a region
