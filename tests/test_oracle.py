"""Pins the oracle (oracle/) before anything is compared against it.

* oracle/immut_ref.py (index arithmetic restated from the reference's
  lowerings) against the ATen operators over exhaustive small cases and the
  reference-held cases of tests/golden/lowering_tests.json.  A dropped term, a
  wrong sign or an off-by-one in any restated formula fails here.
* oracle/configs.py against closed forms and independent library routines
  (torch.nn.LSTM for c4, anchors / priors for zero logits, softmax row sums,
  count == mask.sum()).
"""
import itertools
import json
import os

import numpy as np
import pytest
import torch

from oracle import configs as oc
from oracle import immut_ref as ir

HERE = os.path.dirname(os.path.abspath(__file__))
SHAPE = (3, 4, 5)


def _t():
    return torch.rand(SHAPE, generator=torch.Generator().manual_seed(0))


def test_select_matches_aten():
    t = _t()
    for dim in range(-3, 3):
        for idx in range(-SHAPE[dim], SHAPE[dim]):
            assert np.array_equal(ir.select(t.numpy(), dim, idx), t.select(dim, idx).numpy())


def test_select_rev_matches_aten():
    t = _t()
    g = torch.Generator().manual_seed(1)
    for dim in range(-3, 3):
        for idx in range(-SHAPE[dim], SHAPE[dim]):
            src = torch.rand(t.select(dim, idx).shape, generator=g)
            ref = t.clone()
            ref.select(dim, idx).copy_(src)
            assert np.array_equal(ir.select_rev(t.numpy(), src.numpy(), dim, idx), ref.numpy())


BOUNDS = [None, 0, 1, 2, 3, 7, -1, -2, -9]


def test_slice_and_slice_rev_match_aten():
    t = _t()
    g = torch.Generator().manual_seed(2)
    for dim in (0, 1, 2, -1):
        for start, end in itertools.product(BOUNDS, BOUNDS):
            for step in (1, 2, 3):
                view = torch.ops.aten.slice(t, dim, start, end, step)
                assert np.array_equal(ir.slice_(t.numpy(), dim, start, end, step), view.numpy())
                src = torch.rand(view.shape, generator=g)
                ref = t.clone()
                torch.ops.aten.slice(ref, dim, start, end, step).copy_(src)
                assert np.array_equal(ir.slice_rev(t.numpy(), src.numpy(), dim, start, end, step), ref.numpy())


def test_view_permute_expand_repeat_index_cat_stack_triu_match_aten():
    t = _t()
    n = t.numpy()
    for shape in ([60], [4, 15], [2, -1, 5], [3, 4, 5, 1], [5, 4, 3]):
        assert np.array_equal(ir.view(n, shape), t.reshape(shape).numpy())
    for perm in itertools.permutations(range(3)):
        assert np.array_equal(ir.permute(n, list(perm)), t.permute(perm).numpy())
    for d in range(-4, 4):
        assert np.array_equal(ir.unsqueeze(n, d), t.unsqueeze(d).numpy())
    s = torch.rand(3, 1, 5)
    assert np.array_equal(ir.expand(s.numpy(), [2, 3, 4, 5]), s.expand(2, 3, 4, 5).numpy())
    assert np.array_equal(ir.expand(s.numpy(), [-1, 4, -1]), s.expand(-1, 4, -1).numpy())
    for reps in ([1, 1, 1], [2, 1, 3], [2, 2, 1, 2]):
        assert np.array_equal(ir.repeat(n, reps), t.repeat(reps).numpy())
    idx = torch.randint(0, 3, (2, 3))
    assert np.array_equal(ir.index(n, idx.numpy()), t[idx].numpy())
    parts = [torch.rand(3, k, 5) for k in (1, 2, 3)]
    assert np.array_equal(ir.cat([p.numpy() for p in parts], 1), torch.cat(parts, 1).numpy())
    same = [torch.rand(3, 4) for _ in range(3)]
    for d in (-3, -1, 0, 1, 2):
        assert np.array_equal(ir.stack([p.numpy() for p in same], d), torch.stack(same, d).numpy())
    for diag in (-2, 0, 1):
        assert np.array_equal(ir.triu(n, diag), torch.triu(t, diag).numpy())


def test_reference_held_cases():
    """The argument sets the reference's own suite uses (lowering_tests.json)."""
    suite = json.load(open(os.path.join(HERE, "golden", "lowering_tests.json")))
    g = torch.Generator().manual_seed(3)
    a = suite["select"]["cases"][0][0]
    t = torch.rand(a[0]["shape"], generator=g)
    assert np.array_equal(ir.select(t.numpy(), a[1], a[2]), t.select(a[1], a[2]).numpy())
    for case, _ in suite["slice"]["cases"]:
        t = torch.rand(case[0]["shape"], generator=g)
        dim, start, end = case[1], case[2], case[3]
        step = case[4] if len(case) > 4 else 1
        assert np.array_equal(ir.slice_(t.numpy(), dim, start, end, step),
                              torch.ops.aten.slice(t, dim, start, end, step).numpy())
    a = suite["reshape"]["cases"][0][0]
    t = torch.rand(a[0]["shape"], generator=g)
    assert np.array_equal(ir.view(t.numpy(), a[1]), t.reshape(a[1]).numpy())
    a = suite["index"]["cases"][0][0]
    t = torch.rand(a[0]["shape"], generator=g)
    idx = torch.randint(0, 5, a[1][0]["shape"], generator=g)
    assert np.array_equal(ir.index(t.numpy(), idx.numpy()), t[idx].numpy())


def test_compact_matches_aten():
    g = torch.Generator().manual_seed(4)
    for n in (0, 1, 17, 64):
        m = torch.rand(n, generator=g) < 0.5
        x = torch.rand(n, 3, generator=g)
        (got,) = ir.compact(m.numpy(), [x.numpy()])
        assert np.array_equal(got, x[m].numpy())


# ---------------------------------------------------------------------------
# configs
# ---------------------------------------------------------------------------


def test_c1_closed_form():
    a, b, n = oc.c1_inputs(0, 64, 40)
    out = oc.run("c1", a, b, n)
    ref = b.clone()
    ref[:n] += 1
    assert torch.equal(out, ref)
    assert torch.equal(oc.c1_inputs(0, 64, 40)[1], b)  # inputs untouched


def test_yolo_anchor_layout():
    anchors, strides = oc.yolo_anchors()
    assert anchors.shape == (10647, 4) and strides.shape == (10647,)
    # first cell of level 0, first base size (116, 90), stride 32
    assert torch.allclose(anchors[0], torch.tensor([16 - 58.0, 16 - 45.0, 16 + 58.0, 16 + 45.0]))
    # anchor-minor ordering: next entry is the second base size of the same cell
    assert torch.allclose(anchors[1], torch.tensor([16 - 78.0, 16 - 99.0, 16 + 78.0, 16 + 99.0]))
    # x advances first (xx = x.repeat(h)): 4th entry is cell x=1, y=0
    assert torch.allclose(anchors[3], torch.tensor([48 - 58.0, 16 - 45.0, 48 + 58.0, 16 + 45.0]))
    assert strides[0] == 32 and strides[3 * 169] == 16 and strides[-1] == 8


def test_c2_closed_forms():
    pred, anchors, strides = oc.c2_inputs(0, [2, 3])
    boxes, cls, obj = oc.run("c2", torch.zeros_like(pred), anchors, strides)
    assert torch.allclose(boxes, anchors, atol=1e-4)  # zero logits -> the anchors
    assert torch.equal(obj, torch.full_like(obj, 0.5))
    boxes, cls, obj = oc.run("c2", pred, anchors, strides)
    keep = torch.sigmoid(pred[0, :, 4]) >= 0.3
    assert boxes.shape[0] == cls.shape[0] == obj.shape[0] == int(keep.sum())
    assert torch.equal(obj, torch.sigmoid(pred[0, :, 4])[keep])
    assert torch.equal(cls, torch.sigmoid(pred[0, :, 5:])[keep])
    # independent decode of one kept row
    i = int(torch.nonzero(keep)[0])
    a, p, s = anchors[i], pred[0, i], strides[i]
    cx = (a[0] + a[2]) * 0.5 + (torch.sigmoid(p[0]) - 0.5) * s
    w = (a[2] - a[0]) * 0.5 * torch.exp(p[2])
    assert torch.allclose(boxes[0, 0], cx - w) and torch.allclose(boxes[0, 2], cx + w)


def test_c3_closed_forms():
    loc, conf, priors = oc.c3_inputs(0, 40, 6)
    bs, ss = oc.run("c3", torch.zeros_like(loc), conf, priors)
    scores = conf[0].softmax(-1)
    assert torch.allclose(scores.sum(-1), torch.ones(40), atol=1e-6)
    ref_boxes = torch.cat([priors[:, :2] - priors[:, 2:] / 2, priors[:, :2] + priors[:, 2:] / 2], 1)
    assert len(bs) == 5
    for c in range(1, 6):
        m = scores[:, c] > 0.05
        assert torch.equal(bs[c - 1], ref_boxes[m])
        assert torch.equal(ss[c - 1], scores[m, c])


def test_c3_decode_of_one_row_with_its_variances():
    """Independent decode of single rows with loc != 0, written from the textbook SSD formulas
    (centre variance 0.1, size variance 0.2): a swapped pair of variances, a dropped prior size or a
    wrong sign fails here (with loc == 0 all of these vanish)."""
    import math
    loc, conf, priors = oc.c3_inputs(1, 40, 6)
    bs, ss = oc.run("c3", loc, conf, priors)
    scores = conf[0].softmax(-1)
    checked = 0
    for c in range(1, 6):
        rows = torch.nonzero(scores[:, c] > 0.05).flatten().tolist()
        for k, i in enumerate(rows[:3]):
            pcx, pcy, pw, ph = [float(v) for v in priors[i]]
            lx, ly, lw, lh = [float(v) for v in loc[0, i]]
            cx, cy = pcx + lx * 0.1 * pw, pcy + ly * 0.1 * ph
            w, h = pw * math.exp(lw * 0.2), ph * math.exp(lh * 0.2)
            want = torch.tensor([cx - w / 2, cy - h / 2, cx + w / 2, cy + h / 2])
            assert torch.allclose(bs[c - 1][k], want, rtol=1e-5, atol=1e-6), (c, i)
            # the same row with the variances swapped is far outside that tolerance
            cx2, w2 = pcx + lx * 0.2 * pw, pw * math.exp(lw * 0.1)
            assert abs((cx2 - w2 / 2) - float(want[0])) > 1e-4 or abs(lx) + abs(lw) < 1e-2
            checked += 1
    assert checked >= 5


def test_c4_matches_nn_lstm():
    """Cross-check of the cell formulas against torch.nn.LSTM with re-packed
    weights (the packing functs/benchmark/ai_model/lstm/lstm.py:168-175 uses)."""
    x, wih, whh, bih, bhh = oc.c4_inputs(0, seq_len=7, hidden=16, layers=2, batch=1)
    out, sh, sc = oc.run("c4", x, wih, whh, bih, bhh)
    lstm = torch.nn.LSTM(16, 16, 2)
    with torch.no_grad():
        for l in range(2):
            getattr(lstm, "weight_ih_l%d" % l).copy_(wih[l].transpose(1, 2).reshape(64, 16))
            getattr(lstm, "weight_hh_l%d" % l).copy_(whh[l].transpose(1, 2).reshape(64, 16))
            getattr(lstm, "bias_ih_l%d" % l).copy_(bih[l].reshape(64))
            getattr(lstm, "bias_hh_l%d" % l).copy_(bhh[l].reshape(64))
        ref, (hn, cn) = lstm(x)
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-6)
    assert torch.allclose(sh, hn, rtol=1e-4, atol=1e-6) and torch.allclose(sc, cn, rtol=1e-4, atol=1e-6)


def test_c5_is_a_loop_over_c2():
    preds, anchors, strides = oc.c5_inputs(0, [2, 3], 3)
    rb, rc, ro = oc.run("c5", preds, anchors, strides)
    for i in range(3):
        b, c, o = oc.run("c2", preds[i:i + 1], anchors, strides)
        assert torch.equal(rb[i], b) and torch.equal(rc[i], c) and torch.equal(ro[i], o)
