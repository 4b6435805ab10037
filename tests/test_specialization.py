"""Ahead-of-time compiled regions (functs_amd.aot): the compiled kernels must compute what
the bytecode interpreter computes, bit for bit, and the generated sources that are
committed must be the ones the current lowering produces for the benchmark programs."""
import glob
import os

import pytest
import torch

import functs_amd.aot as aot
from functs_amd import Region, _lib, configs
from functs_amd.benchmark.inputs import INPUTS
from oracle import configs as oc

SPEC_DIR = aot.SPEC_DIR


def _region_calls(name):
    """(region, cpu arguments) of a benchmark configuration described through the Region API."""
    args = INPUTS[name](0)
    if name == "c1":
        a, b, n = args
        return [(configs.build_c1(), (b, n))]
    if name == "c2":
        return [(configs.build_c2(), args)]
    if name == "c5":
        return [(configs.build_c5(16), args)]
    if name == "c3":
        return [(configs.build_c3_decode(), args)]
    raise KeyError(name)


def test_product_inputs_equal_oracle_inputs():
    for name in ("c1", "c2", "c3", "c4", "c5"):
        mine, theirs = INPUTS[name](0), getattr(oc, name + "_inputs")(0)
        assert len(mine) == len(theirs)
        for x, y in zip(mine, theirs):
            assert torch.equal(x, y) if isinstance(x, torch.Tensor) else x == y


def test_library_links_the_committed_specialisations(tmp_path):
    files = glob.glob(os.path.join(SPEC_DIR, "fx_spec_*.hip"))
    assert files, "no generated sources under csrc/fxhip/spec"
    # counted in a process of its own with an empty kernel cache: kernels that other tests have
    # compiled and registered in this process are not the library's
    import subprocess
    import sys
    env = dict(os.environ, FUNCTS_AMD_KERNEL_CACHE=str(tmp_path))
    out = subprocess.run([sys.executable, "-c", "import functs_amd.aot as aot; print(aot.linked())"],
                         cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))), env=env,
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert out.returncode == 0, out.stderr
    assert int(out.stdout.strip().splitlines()[-1]) == len(files)
    assert aot.linked() >= len(files)


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c5"])
def test_benchmark_regions_have_compiled_kernels(name):
    # planning needs no GPU: the key of the lowered programs must be one that is linked in
    for region, args in _region_calls(name):
        key = region.spec_key(*args)
        assert key != 0
        assert region.specialized(*args), "no compiled kernels for key %016x: regenerate with python -m functs_amd.aot" % key
        # and the committed source is what the lowering produces today
        path = os.path.join(SPEC_DIR, "fx_spec_%016x.hip" % key)
        committed = open(path).read().split("\n", 1)[1]
        assert region.spec_source(*args).split("\n", 1)[1] == committed


def test_switch_and_key_of_a_new_region():
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output((x * 3.0 - 0.25).relu())
    r.finalize()
    t = torch.zeros(5, 7)
    assert r.spec_key(t) != 0 and not r.specialized(t)      # nobody compiled this one
    src = r.spec_source(t, label="test")
    assert "FX_SPEC_DENSE(P_%016x, 2)" % r.spec_key(t) in src and "FX_RELU" in src
    # same programs, other sizes: dense programs do not depend on the extents here
    assert r.spec_key(torch.zeros(9, 7)) == r.spec_key(t)
    aot.enable(False)
    try:
        for region, args in _region_calls("c1"):
            assert not region.specialized(*args)
    finally:
        aot.enable(True)


def test_capture_writes_one_file_per_unknown_region(tmp_path):
    r = Region()
    x = r.tensor_input(torch.float32, 1)
    r.output(x.sigmoid() + 1.0)
    r.finalize()
    with aot.capture(str(tmp_path)):
        r.disasm(torch.zeros(100))        # planning is enough
        for region, args in _region_calls("c1"):
            region.disasm(*args)          # already linked: leaves nothing
    files = os.listdir(tmp_path)
    assert files == ["fx_spec_%016x.hip" % r.spec_key(torch.zeros(100))]
    r.disasm(torch.zeros(50))             # capture is over
    assert os.listdir(tmp_path) == files


def _flat(o):
    if isinstance(o, (list, tuple)):
        for x in o:
            yield from _flat(x)
    else:
        yield o


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c5"])
def test_compiled_equals_interpreter_region_api(name):
    dev = torch.device("cuda:0")
    prev = None
    for region, args in _region_calls(name) + ([(configs.build_c3_classes(80), None)] if name == "c3" else []):
        gargs = prev if args is None else [a.to(dev) if isinstance(a, torch.Tensor) else a for a in args]
        assert region.specialized(*gargs)
        total0, spec0 = aot.launch_stats()
        fast = list(_flat(region(*gargs)))
        total1, spec1 = aot.launch_stats()
        assert spec1 - spec0 == total1 - total0 > 0
        aot.enable(False)
        try:
            slow = list(_flat(region(*gargs)))
            assert aot.launch_stats()[1] == spec1
        finally:
            aot.enable(True)
        assert len(fast) == len(slow)
        for x, y in zip(fast, slow):
            assert x.shape == y.shape and torch.equal(x, y)
        prev = region(*gargs)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_compiled_equals_interpreter_torchscript_route(name):
    import functs_amd.jit as fj
    from functs_amd.benchmark import PROGRAMS
    dev = torch.device("cuda:0")
    cpu_args = INPUTS[name](0)
    fn = fj.build(fj.script(PROGRAMS[name]), list(cpu_args))
    gargs = [a.to(dev) if isinstance(a, torch.Tensor) else a for a in cpu_args]
    total0, spec0 = aot.launch_stats()
    fast = list(_flat(fn(*gargs)))
    total1, spec1 = aot.launch_stats()
    assert total1 > total0 and spec1 - spec0 == total1 - total0, "a region of %s ran interpreted" % name
    aot.enable(False)
    try:
        slow = list(_flat(fn(*gargs)))
    finally:
        aot.enable(True)
    assert len(fast) == len(slow)
    for x, y in zip(fast, slow):
        assert x.shape == y.shape
        if name == "c3":
            # one region (decode + softmax inside the class map): the hand-written kernel sums a
            # row of scores across the lanes of a half-wave, the interpreter one by one per class
            torch.testing.assert_close(x, y, rtol=1e-6, atol=1e-9)
        else:
            assert torch.equal(x, y)



def test_generated_source_compiles(tmp_path):
    """The generator's output for a region nobody compiled yet (predicated branches, a reduction
    loop, a wave reduction) goes through hipcc for gfx950: the templates accept every construct
    the lowering emits."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not installed")
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    y = x.slice_rev(x.slice(1, 0, 2).sigmoid(), 1, 0, 2)       # predicated branch
    r.output(y.softmax(1))                                     # wave reductions
    r.output(r.op("SUM_DIM", y * 2.0, 0, False))               # reduction loop
    r.finalize()
    t = torch.zeros(33, 7)
    src = r.spec_source(t, label="test")
    path = tmp_path / ("fx_spec_%016x.hip" % r.spec_key(t))
    path.write_text(src.replace('#include "../fx_spec.h"', '#include "fx_spec.h"'))
    inc = os.path.join(os.path.dirname(aot.SPEC_DIR))
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-O1", "-std=c++17", "-ffp-contract=off", "-Xclang",
                           "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-c", str(path),
                           "-I", inc, "-o", str(tmp_path / "spec.o")], stderr=subprocess.DEVNULL)
    assert (tmp_path / "spec.o").stat().st_size > 0


@pytest.mark.gpu
def test_compiled_reduction_loops_where_cat_softmax():
    """A compiled region with serial reduction loops, max over a dimension, `where`, `cat`
    branches and a row softmax (none of which the five configurations' compiled regions
    contain): equal to the interpreter bit for bit, and to torch within 1e-5."""
    dev = torch.device("cuda:0")
    r = configs.build_column_standardize()
    x = (torch.rand(*configs.COLUMN_STANDARDIZE_SHAPE, generator=torch.Generator().manual_seed(4)) - 0.5)
    gx = x.to(dev)
    assert r.specialized(gx)
    fast = r(gx)
    aot.enable(False)
    try:
        slow = r(gx)
    finally:
        aot.enable(True)
    for a, b in zip(fast, slow):
        assert torch.equal(a, b)
    mean = x.sum(0) / x.size(0)
    z = x - mean
    spread = z.abs().max(0).values
    want0 = torch.where(z > 0, z, 0.1 * z) / (spread + 1)
    want1 = torch.cat([x[:, :2].exp(), x[:, 2:]], 1).softmax(1)
    torch.testing.assert_close(fast[0].cpu(), want0, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(fast[1].cpu(), want1, rtol=1e-5, atol=1e-6)


def _row_filter_inputs(n, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.rand(n, sh[1], generator=g) - 0.5 for sh in configs.ROW_FILTER_SHAPES]


def test_row_filter_region_is_linked_and_current():
    r = configs.build_row_filter()
    args = _row_filter_inputs(configs.ROW_FILTER_SHAPES[0][0], 0)
    key = r.spec_key(*args)
    assert r.specialized(*args), "no compiled kernels for key %016x: regenerate with python -m functs_amd.aot" % key
    committed = open(os.path.join(SPEC_DIR, "fx_spec_%016x.hip" % key)).read().split("\n", 1)[1]
    assert r.spec_source(*args).split("\n", 1)[1] == committed


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 63, 256, 257, 1000, 4099])
def test_compiled_row_compaction_routes(n):
    """One launch with an output made of whole groups of four (the lean batch path, with and
    without a last incomplete batch), one with a ragged last group (the general batch path), a
    column-wise narrow one whose programs read their inputs twice (repeated loads are reused
    in compiled programs) and a rank-1 one: compiled == interpreter bit for bit, and equal to
    torch on the kept rows (bit-exact for the copies, 1e-5 for the arithmetic)."""
    dev = torch.device("cuda:0")
    r = configs.build_row_filter()
    x, s = _row_filter_inputs(n, n)
    gx, gs = x.to(dev), s.to(dev)
    assert r.specialized(gx, gs)   # the row count is not part of the programs
    fast = r(gx, gs)
    aot.enable(False)
    try:
        slow = r(gx, gs)
    finally:
        aot.enable(True)
    for a, b in zip(_flat(fast), _flat(slow)):
        assert torch.equal(a, b)
    keep = x[:, 0] > 0
    xk, sk = x[keep], s[keep]
    a = xk[:, 1:2] * sk[:, 0:1]
    b = xk[:, 2:3] + sk[:, 1:2]
    outs = [o.cpu() for o in _flat(fast) if isinstance(o, torch.Tensor)]
    wide, ragged, narrow, first = outs[:4]
    assert wide.shape == (int(keep.sum()), 16)
    torch.testing.assert_close(wide, xk[:, 3:].sigmoid(), rtol=1e-5, atol=1e-6)
    assert torch.equal(ragged, xk[:, :7] * 2.0)
    torch.testing.assert_close(narrow, torch.cat([a * b + a, a * b - b], 1), rtol=1e-5, atol=1e-6)
    assert torch.equal(first, xk[:, 0])


@pytest.mark.gpu
def test_batched_kernel_timing_leaves_results_alone():
    """Timing a kernel over a batch of launches (the kernels of a region are idempotent) gives
    the outputs of a plain launch and a mean below the single-launch reading plus noise."""
    dev = torch.device("cuda:0")
    r = configs.build_row_filter()
    x, s = _row_filter_inputs(1000, 5)
    bc = r.bind(x.to(dev), s.to(dev))
    bc.launch()
    want = [o.clone() for o in _flat(bc.results()) if isinstance(o, torch.Tensor)]
    single = bc.launch_timed()
    batched = bc.launch_timed(repeat=10)
    got = [o for o in _flat(bc.results()) if isinstance(o, torch.Tensor)]
    assert len(single) == len(batched) == bc.plan.launches and all(t > 0 for t in batched)
    assert sum(batched) < sum(single) * 1.5
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    from functs_amd._lib import FxError
    with pytest.raises(FxError, match="repeat"):
        bc.launch_timed(repeat=0)
