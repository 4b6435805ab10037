"""Graphs the reference's README prints, step by step, as golden operator
sequences (tests/golden/readme_graphs.json), plus the two README programs
that exercise vertical fusion (Normalize) and horizontal parallelization
(MultiScaleBboxProcess)."""
import json
import os
from typing import List

import pytest
import torch

import functs_amd.jit as fj
from functs_amd import _C
from functs_amd.benchmark import get_started

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "readme_graphs.json")))


def ops(block, out=None):
    out = [] if out is None else out
    for n in block.nodes():
        if n.kind() != "prim::Constant":
            out.append(n.kind())
        for b in n.blocks():
            ops(b, out)
    return out


def test_get_started_step_by_step():
    gold = GOLD["get_started"]
    g = torch.jit.script(get_started).graph.copy()
    info = _C.TensorSSAMutateInfo()
    _C._jit_pass_rewrite_mutation(g, info)
    assert ops(g) == gold["after_rewrite_mutation"]["ops"]
    assert [v.node().kind() for v in info.mutValues] == gold["mut_values"]["defining_ops"]
    # b.5, the view that is written (it feeds immut::assign), the view that is read, the assign
    written = info.mutValues[1]
    assert any(u.user.kind() == "immut::assign" for u in written.uses())
    assert set(info.mutNodes.keys()) == set(info.mutValues)
    assert all(len(v) == 1 and v[0].kind() == "tssa::update" for v in info.mutNodes.values())

    _C._jit_pass_block_propagation(g, info)
    assert ops(g) == gold["after_block_propagation"]["ops"]
    loop = [n for n in g.nodes() if n.kind() == "prim::Loop"][0]
    assert len(list(loop.outputs())) == gold["after_block_propagation"]["loop_carried"]

    _C._jit_pass_rename(g)
    assert ops(g) == gold["after_block_propagation"]["ops"]  # renaming moves no node
    assert list(g.outputs())[0].node().kind() == "prim::Loop"  # return (%48)

    _C._jit_pass_tensorssa_remove_update(g)
    assert ops(g) == gold["after_remove_update"]["ops"]

    torch._C._jit_pass_cse(g)
    torch._C._jit_pass_dce(g)
    torch._C._jit_pass_constant_propagation(g)
    assert ops(g) == gold["final"]["ops"]
    _C._jit_pass_validate(g)


def if_else(a: torch.Tensor, b: torch.Tensor, idx: int):
    a = a.clone()
    b = b.clone()
    if idx >= 0:
        a = a + 1
        b[idx] = a[idx]
    else:
        a = a - 1
        b[-idx] = a[-idx]
    return a + b


def test_if_else_program():
    gold = GOLD["if_else"]
    f = fj.script(if_else, add_clone=True)
    # The reference drops the view tree of a value that leaves an If body
    # (convert_to_tensorssa.cpp:52-53), so its reads of a.9 / a.17 stay aten::select;
    # this build keeps such trees and prints the same reads as immut::select.
    assert [k.replace("immut::select_rev", "REV").replace("immut::select", "aten::select").replace(
        "REV", "immut::select_rev") for k in ops(f.graph)] == gold["ops"]
    node = [n for n in f.graph.nodes() if n.kind() == "prim::If"][0]
    assert len(list(node.outputs())) == gold["if_outputs"]
    for idx in (1, -2):
        a, b = torch.rand(4, 3), torch.rand(4, 3)
        assert torch.equal(f(a, b, idx), if_else(a, b, idx))


class Normalize(torch.nn.Module):
    def forward(self, src: torch.Tensor, mean: float, scale: float):
        src = src.clone()
        dup = src.clone()
        dup[..., 0] = src[..., 2]
        dup[..., 2] = src[..., 0]
        return (dup - mean) * scale


class MultiScaleBboxProcess(torch.nn.Module):
    def decode_bboxes(self, bboxes, pred_bboxes, stride: float):
        xy_centers = (bboxes[..., :2] + bboxes[..., 2:]) * 0.5 + (pred_bboxes[..., :2] - 0.5) * stride
        whs = (bboxes[..., 2:] - bboxes[..., :2]) * 0.5 * pred_bboxes[..., 2:].exp()
        decoded_bboxes = torch.stack(
            (
                xy_centers[..., 0] - whs[..., 0],
                xy_centers[..., 1] - whs[..., 1],
                xy_centers[..., 0] + whs[..., 0],
                xy_centers[..., 1] + whs[..., 1],
            ),
            dim=-1,
        )
        return decoded_bboxes.clone()

    def forward(self, bboxes_list: List[torch.Tensor], pred_bboxes_list: List[torch.Tensor], stride_list: List[float]):
        outs = []
        for bboxes, pred_bboxes, stride in zip(bboxes_list, pred_bboxes_list, stride_list):
            out = self.decode_bboxes(bboxes, pred_bboxes, stride)
            outs.append(out)
        return outs


def _functors(graph):
    return [n for n in graph.nodes() if n.kind() == "tssa::ParallelFunctor"]


def test_normalize_is_one_fused_region():
    src = torch.rand(8, 13, 3)
    f = fj.script(Normalize())
    assert torch.equal(f(src, 0.25, 2.0), Normalize()(src, 0.25, 2.0))  # functionalized, stock interpreter
    built = fj.build(f, [src, 0.25, 2.0])
    fs = _functors(built.graph)
    assert len(fs) == 1 and ops(built.graph) == ["tssa::ParallelFunctor"]
    assert ops(fs[0].g("Subgraph")) == GOLD["normalize_fused_subgraph"]["ops"]


def _bbox_inputs(seed=0):
    g = torch.Generator().manual_seed(seed)
    sizes = (48, 12, 3)
    boxes = [torch.rand(n, 4, generator=g) * 100 for n in sizes]
    preds = [torch.randn(n, 4, generator=g) for n in sizes]
    return boxes, preds, [8.0, 16.0, 32.0]


def test_multi_scale_bbox_is_one_parallel_map():
    gold = GOLD["multi_scale_bbox"]
    boxes, preds, strides = _bbox_inputs()
    f = fj.script(MultiScaleBboxProcess())
    want = MultiScaleBboxProcess()(boxes, preds, strides)
    got = f(boxes, preds, strides)
    assert all(torch.equal(a, b) for a, b in zip(got, want))
    built = fj.build(f, [boxes, preds, strides])
    fs = _functors(built.graph)
    assert len(fs) == 1 and "prim::Loop" not in ops(built.graph)
    n = fs[0]
    assert n.i("is_parallel_map") == gold["is_parallel_map"]
    assert list(getattr(n, "is")("is_parallel_args")) == gold["is_parallel_args"]
    assert n.i("parallel_degree") in (gold["parallel_degree"], -1)  # -1: trip count passed at run time
    assert sorted(ops(n.g("Subgraph"))) == sorted(gold["subgraph_ops"])


@pytest.mark.gpu
def test_normalize_gpu():
    src = torch.rand(800, 1333, 3)
    built = fj.build(fj.script(Normalize()), [src, 0.5, 3.0])
    got = built(src.cuda(), 0.5, 3.0).cpu()
    assert torch.equal(got, Normalize()(src, 0.5, 3.0))  # sub and mul round once each on both sides


@pytest.mark.gpu
def test_multi_scale_bbox_gpu():
    boxes, preds, strides = _bbox_inputs(3)
    built = fj.build(fj.script(MultiScaleBboxProcess()), [boxes, preds, strides])
    got = built([b.cuda() for b in boxes], [p.cuda() for p in preds], strides)
    want = MultiScaleBboxProcess()(boxes, preds, strides)
    assert len(got) == 3
    for g_, w in zip(got, want):
        torch.testing.assert_close(g_.cpu(), w, rtol=1e-5, atol=1e-4)
