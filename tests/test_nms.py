"""Detection tail (score threshold + sort + class-aware greedy NMS + top-k).

CPU: the oracle (oracle/nms.py) is pinned without torchvision, which is not importable here
("parity unpinned" against torchvision itself): by the property that defines the greedy result
uniquely, by brute force over all subsets of tiny inputs, and by hand-computed cases.
GPU: fx_sort_nms through the C ABI against the oracle - indices and labels bit-exact, boxes and
scores bit-exact as well (they are copies and one float32 product)."""
import itertools

import pytest
import torch

from oracle import nms as onms


def _boxes(g, n, span=100.0, size=40.0):
    xy = torch.rand(n, 2, generator=g) * span
    wh = torch.rand(n, 2, generator=g) * size + 1.0
    return torch.cat([xy, xy + wh], 1)


# --- the oracle ---------------------------------------------------------------------------------
def test_hand_computed_cases():
    # two boxes with IoU exactly 1/3 and a third far away
    b = torch.tensor([[0., 0., 2., 2.], [1., 0., 3., 2.], [10., 10., 12., 12.]])
    s = torch.tensor([0.9, 0.8, 0.7])
    iou = onms.iou_matrix(b)
    assert iou[0, 1].item() == pytest.approx(1.0 / 3.0) and iou[0, 2].item() == 0.0 and iou[0, 0].item() == 1.0
    assert onms.nms(b, s, 0.3).tolist() == [0, 2]        # 1/3 > 0.3: suppressed
    assert onms.nms(b, s, 0.34).tolist() == [0, 1, 2]    # 1/3 <= 0.34: kept
    # IoU exactly at the threshold is kept (the comparison is strict): 2x2 boxes shifted by 1 -> 0.5 / 1.5... use halves
    b2 = torch.tensor([[0., 0., 4., 1.], [2., 0., 6., 1.]])   # inter 2, union 6
    thr = (torch.tensor(2.0) / torch.tensor(6.0)).item()
    assert onms.nms(b2, torch.tensor([1.0, 0.5]), thr).tolist() == [0, 1]
    assert onms.nms(b2, torch.tensor([1.0, 0.5]), thr - 1e-6).tolist() == [0]
    # nested boxes: IoU = small / large
    b3 = torch.tensor([[0., 0., 10., 10.], [2., 2., 4., 4.]])
    assert onms.nms(b3, torch.tensor([0.5, 0.9]), 0.03).tolist() == [1]       # 4 / 100 > 0.03, the small one leads
    assert onms.nms(b3, torch.tensor([0.5, 0.9]), 0.05).tolist() == [1, 0]
    # equal scores: input order decides
    b4 = torch.tensor([[0., 0., 2., 2.], [0., 0., 2., 2.], [5., 5., 6., 6.]])
    assert onms.nms(b4, torch.tensor([0.5, 0.5, 0.5]), 0.5).tolist() == [0, 2]
    # a suppressed box suppresses nothing: 0 kills 1, 1 would have killed 2
    b5 = torch.tensor([[0., 0., 4., 4.], [2., 0., 6., 4.], [4., 0., 8., 4.]])   # IoU(0,1) = IoU(1,2) = 1/3, IoU(0,2) = 0
    assert onms.nms(b5, torch.tensor([0.9, 0.8, 0.7]), 0.3).tolist() == [0, 2]
    # degenerate boxes (zero area twice: 0 / 0) suppress nothing
    b6 = torch.tensor([[1., 1., 1., 1.], [1., 1., 1., 1.]])
    assert onms.nms(b6, torch.tensor([0.9, 0.8]), 0.5).tolist() == [0, 1]
    assert onms.nms(torch.zeros(0, 4), torch.zeros(0), 0.5).numel() == 0


@pytest.mark.parametrize("seed", range(6))
def test_greedy_result_is_the_unique_fixed_point(seed):
    """i is kept  <=>  no kept j ranked before i overlaps it: this has exactly one solution
    (decide candidates in rank order), found here by brute force over all subsets."""
    g = torch.Generator().manual_seed(seed)
    n = 9
    b = _boxes(g, n, span=30.0, size=25.0)
    s = torch.rand(n, generator=g)
    if seed % 2:
        s[3] = s[5]   # a tie
    thr = 0.2
    keep = onms.nms(b, s, thr)
    order = torch.sort(s, descending=True, stable=True).indices.tolist()
    rank = {i: r for r, i in enumerate(order)}
    over = onms.iou_matrix(b) > thr
    solutions = []
    for bits in itertools.product([False, True], repeat=n):
        ok = all(bits[i] == (not any(bits[j] and rank[j] < rank[i] and bool(over[i, j]) for j in range(n))) for i in range(n))
        if ok:
            solutions.append([i for i in order if bits[i]])
    assert len(solutions) == 1 and solutions[0] == keep.tolist()


@pytest.mark.parametrize("seed", range(3))
def test_invariants_on_larger_inputs(seed):
    g = torch.Generator().manual_seed(100 + seed)
    n = 300
    b, s = _boxes(g, n), torch.rand(n, generator=g)
    keep = onms.nms(b, s, 0.45)
    ks = s[keep]
    assert bool((ks[:-1] >= ks[1:]).all())                    # by descending score
    iou = onms.iou_matrix(b)
    sub = iou[keep][:, keep]
    sub.fill_diagonal_(0)
    assert not bool((sub > 0.45).any())                        # kept boxes do not overlap each other
    kept = set(keep.tolist())
    for i in range(n):                                         # every dropped box has a kept, better one on top of it
        if i not in kept:
            assert any(iou[i, j] > 0.45 and (s[j] > s[i] or (s[j] == s[i] and j < i)) for j in kept)
    # prefix stability: the result on the top-m candidates is a prefix of the full result
    order = torch.sort(s, descending=True, stable=True).indices
    top = order[:120]
    sub_keep = top[onms.nms(b[top], s[top], 0.45)]
    assert sub_keep.tolist() == keep[:sub_keep.numel()].tolist()


def test_batched_nms_separates_classes():
    b = torch.tensor([[0., 0., 2., 2.], [0., 0., 2., 2.], [0.5, 0., 2.5, 2.]])
    s = torch.tensor([0.9, 0.8, 0.7])
    dets, keep = onms.batched_nms(b, s, torch.tensor([0, 1, 0]))
    assert keep.tolist() == [0, 1] and torch.equal(dets[:, :4], b[keep]) and torch.equal(dets[:, 4], s[keep])
    dets, keep = onms.batched_nms(b, s, torch.tensor([0, 0, 0]))
    assert keep.tolist() == [0]
    # per-class NMS (the reference's other branch) gives the same set
    g = torch.Generator().manual_seed(5)
    b, s = _boxes(g, 200), torch.rand(200, generator=g)
    lab = torch.randint(0, 4, (200,), generator=g)
    _, keep = onms.batched_nms(b, s, lab)
    per_class = []
    for c in range(4):
        m = (lab == c).nonzero()[:, 0]
        per_class += m[onms.nms(b[m], s[m], 0.45)].tolist()
    assert sorted(per_class) == sorted(keep.tolist())


def test_multiclass_nms_follows_the_reference_steps():
    g = torch.Generator().manual_seed(7)
    k, c = 40, 5
    b = _boxes(g, k)
    cls = torch.rand(k, c, generator=g) * 0.2
    obj = torch.rand(k, generator=g)
    dets, labels, index = onms.multiclass_nms(b, cls, obj, score_thr=0.05, max_num=10)
    assert dets.size(0) <= 10 and dets.size(0) == labels.numel() == index.numel()
    rows, classes = index // c, index % c
    assert torch.equal(labels, classes) and torch.equal(dets[:, :4], b[rows])
    assert torch.equal(dets[:, 4], cls[rows, classes] * obj[rows]) and bool((cls[rows, classes] > 0.05).all())
    assert onms.multiclass_nms(b, cls * 0, obj)[0].size(0) == 0   # nothing passes the threshold


def test_filter_scores_and_topk():
    s = torch.tensor([[0.1, 0.9], [0.5, 0.01], [0.7, 0.5]])
    scores, labels, rows = onms.filter_scores_and_topk(s, 0.05, 3)
    assert scores.tolist() == pytest.approx([0.9, 0.7, 0.5]) and labels.tolist() == [1, 0, 0] and rows.tolist() == [0, 2, 1]


# --- the kernel -----------------------------------------------------------------------------------
def _check_multiclass(boxes, cls, obj, counts, score_thr, iou_thr, max_num, key_capacity=16384):
    from functs_amd import detection
    dev = torch.device("cuda:0")
    cnt = None if counts is None else torch.tensor(counts, dtype=torch.int32, device=dev)
    print("fx_sort_nms mode 1 T=%d K=%d C=%d max_num=%d" % (boxes.size(0), boxes.size(1), cls.size(2), max_num), flush=True)
    res = detection.multiclass_nms_batched(boxes.to(dev), cls.to(dev), None if obj is None else obj.to(dev), cnt, score_thr,
                                           iou_thr, max_num, key_capacity)
    got = res.lists()
    for t in range(boxes.size(0)):
        k = boxes.size(1) if counts is None else counts[t]
        o = torch.ones(k) if obj is None else obj[t, :k]
        dets, labels, index = onms.multiclass_nms(boxes[t, :k], cls[t, :k], o, score_thr, iou_thr, max_num)
        gd, gl, gi = [x.cpu() for x in got[t]]
        assert gi.tolist() == index.tolist(), "image %d: kept candidates differ" % t
        assert torch.equal(gl, labels) and torch.equal(gd, dets)
    # rows past the kept ones are zero
    n = res.n.cpu()
    for t in range(boxes.size(0)):
        k = int(n[t])
        assert not bool(res.dets[t, k:].any()) and not bool(res.labels[t, k:].any())
    return got


def _multiclass_inputs(seed, T, K, C, rate):
    """Class scores of which a fraction `rate` passes 0.05, boxes that overlap a lot."""
    g = torch.Generator().manual_seed(seed)
    boxes = torch.stack([_boxes(g, K, span=60.0, size=50.0) for _ in range(T)])
    u = torch.rand(T, K, C, generator=g)
    cls = torch.where(u < rate, 0.05 + 0.9 * torch.rand(T, K, C, generator=g), 0.04 * torch.rand(T, K, C, generator=g))
    obj = torch.rand(T, K, generator=g)
    return boxes, cls, obj


@pytest.mark.gpu
@pytest.mark.parametrize("T,K,C,rate,max_num", [(1, 50, 3, 0.5, 100), (3, 700, 80, 0.02, 100), (2, 2000, 4, 0.6, 100),
                                                (16, 1000, 80, 0.05, 100), (1, 333, 7, 1.0, 1024), (2, 64, 1, 1.0, 5)])
def test_multiclass_nms_equals_the_oracle(T, K, C, rate, max_num):
    boxes, cls, obj = _multiclass_inputs(T * 1000 + K, T, K, C, rate)
    _check_multiclass(boxes, cls, obj, None, 0.05, 0.45, max_num)


@pytest.mark.gpu
def test_counts_come_from_memory_and_edge_cases():
    boxes, cls, obj = _multiclass_inputs(3, 4, 300, 6, 0.3)
    cls[2] = 0.0                                  # an image without candidates
    cls[3, :, :] = 0.5                            # all scores equal: index order decides
    obj[3] = 1.0
    _check_multiclass(boxes, cls, obj, [300, 17, 300, 64], 0.05, 0.45, 50)
    _check_multiclass(boxes, cls, obj, [0, 1, 2, 3], 0.05, 0.45, 50)
    _check_multiclass(boxes, cls, None, None, 0.05, 0.45, 50)   # no score factors


@pytest.mark.gpu
def test_counts_in_pinned_host_memory():
    from functs_amd import detection
    boxes, cls, obj = _multiclass_inputs(9, 2, 128, 4, 0.5)
    dev = torch.device("cuda:0")
    cnt = torch.tensor([100, 7], dtype=torch.int32).pin_memory()
    got = detection.multiclass_nms_batched(boxes.to(dev), cls.to(dev), obj.to(dev), cnt).lists()
    for t, k in enumerate((100, 7)):
        _, _, index = onms.multiclass_nms(boxes[t, :k], cls[t, :k], obj[t, :k])
        assert got[t][2].cpu().tolist() == index.tolist()


@pytest.mark.gpu
@pytest.mark.parametrize("n,classes", [(1, 1), (65, 2), (1000, 80), (5000, 3), (16384, 80)])
def test_batched_nms_equals_the_oracle(n, classes):
    from functs_amd import detection
    g = torch.Generator().manual_seed(n)
    span = 100.0 if n < 5000 else 600.0
    b, s = _boxes(g, n, span=span), torch.rand(n, generator=g)
    s[n // 2:] = s[:n - n // 2].clone()            # ties
    lab = torch.randint(0, classes, (n,), generator=g)
    dets, keep = onms.batched_nms(b, s, lab)
    dev = torch.device("cuda:0")
    print("fx_sort_nms mode 0 n=%d classes=%d" % (n, classes), flush=True)
    gd, gk = detection.batched_nms(b.to(dev), s.to(dev), lab.to(dev))
    m = min(keep.numel(), detection.MAX_OUT)
    assert gk.cpu().tolist() == keep[:m].tolist() and torch.equal(gd.cpu(), dets[:m])
    if classes == 1:
        assert detection.nms(b.to(dev), s.to(dev), 0.45).cpu().tolist() == keep[:m].tolist()


@pytest.mark.gpu
def test_a_chain_of_overlaps_is_resolved_in_order():
    """Every box overlaps only its neighbours in score order (IoU 7/13 with the next, 1/4 with the one
    after): whether a box is kept depends on all boxes before it, the longest chain a chunk can hold."""
    from functs_amd import detection
    n = 300
    x = torch.arange(n, dtype=torch.float32) * 3.0
    b = torch.stack([x, torch.zeros(n), x + 10.0, torch.full((n,), 5.0)], 1)
    s = torch.linspace(0.99, 0.01, n)
    lab = torch.zeros(n, dtype=torch.int64)
    dets, keep = onms.batched_nms(b, s, lab)
    assert keep.tolist() == list(range(0, n, 2))                  # every other box
    dev = torch.device("cuda:0")
    gd, gk = detection.batched_nms(b.to(dev), s.to(dev), lab.to(dev))
    assert gk.cpu().tolist() == keep.tolist() and torch.equal(gd.cpu(), dets)
    # the same chain broken in places: a gap starts a new chain
    b2 = b.clone()
    b2[97:, 0] += 100.0
    b2[97:, 2] += 100.0
    dets, keep = onms.batched_nms(b2, s, lab)
    gd, gk = detection.batched_nms(b2.to(dev), s.to(dev), lab.to(dev))
    assert gk.cpu().tolist() == keep.tolist() and torch.equal(gd.cpu(), dets)


@pytest.mark.gpu
def test_more_candidates_than_the_launch_is_sized_for_is_reported():
    from functs_amd import detection
    from functs_amd._lib import FxError
    boxes, cls, obj = _multiclass_inputs(1, 1, 200, 4, 1.0)    # 800 candidates
    dev = torch.device("cuda:0")
    res = detection.multiclass_nms_batched(boxes.to(dev), cls.to(dev), obj.to(dev), key_capacity=256)
    with pytest.raises(FxError, match="more candidates"):
        res.lists()
    assert int(res.n.cpu()[0]) == -1 and not bool(res.dets.any())   # FX_NMS_OVERFLOW, zeros
    # and the next launch is not affected
    _check_multiclass(boxes, cls, obj, None, 0.05, 0.45, 100)


def test_host_tensors_and_bad_limits_are_refused():
    from functs_amd import detection
    from functs_amd._lib import FxError
    with pytest.raises(FxError, match="GPU only"):
        detection.nms(torch.zeros(3, 4), torch.zeros(3), 0.5)


@pytest.mark.gpu
def test_compaction_feeds_the_tail_without_the_host():
    """The map's outputs and kept-row counts go from the compaction kernels to fx_sort_nms on the
    same stream: nothing waits for the host in between.  Expected values: the oracle's
    multiclass_nms on what the region itself returned (the region's own parity with the oracle is
    tests/test_configs.py's business; a box that differs in its last bit may flip an overlap test)."""
    from functs_amd import configs, detection
    from oracle import configs as oc
    T = 5
    preds, anchors, strides = oc.c5_inputs(2, [4, 6, 8], T)
    preds[..., 5:] -= 3.5          # few class scores pass 0.05, as behind a trained head
    dev = torch.device("cuda:0")
    r = configs.build_c5(T)
    bc = r.bind(preds.to(dev), anchors.to(dev), strides.to(dev))
    bc.launch()
    res = detection.multiclass_nms_batched(bc.batched(0), bc.batched(1), bc.batched(2), counts=bc.totals, max_num=100)
    got = res.lists()
    boxes, cls, obj = bc.results()
    assert any(b.size(0) not in (0, preds.size(1)) for b in boxes)
    for t in range(T):
        dets, labels, index = onms.multiclass_nms(boxes[t].cpu(), cls[t].cpu(), obj[t].cpu())
        assert got[t][2].cpu().tolist() == index.tolist() and torch.equal(got[t][0].cpu(), dets) and torch.equal(got[t][1].cpu(), labels)
    assert int(res.n.sum()) > 0
