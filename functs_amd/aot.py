"""Ahead-of-time specialisation of fused regions.

The library runs the programs of a lowered region with a bytecode interpreter.  For a
region whose shapes are known it can also hold compiled kernels: the programs become a
compile-time table (one generated ``fx_spec_<key>.hip`` per region), the region kernels
are instantiated for that table when the library is built, and at run time a plan whose
programs hash to a linked key runs the compiled kernels, any other plan the interpreter.
Results are identical instruction for instruction.

This is where the reference compiles each ``tssa::ParallelFunctor`` subgraph with NVRTC
when the operator is created (fait/fuser/graph_builder.cpp:259-712,
fait/tensorexpr/cuda_codegen_tssa.cpp:1319-1414); here the compiler runs at build time.

A compacting region whose widest input is read row by row gets a second generated unit,
``fx_rs_<key>.hip``: its programs as straight-line code per row for the one-launch row-stream
kernel (``fx_plan_rowstream_source``).

Use, for your own model::

    import functs_amd.aot as aot
    fn = functs_amd.jit.build(functs_amd.jit.script(model), example_inputs)
    with aot.capture():                 # default: functs_amd/csrc/fxhip/spec
        aot.plan(fn)                    # plans every region for the example's static types (no GPU needed)
        # or, on a GPU:  fn(*example_inputs)   - every region planned while it runs leaves its source
    # then rebuild the library:  python -c "import __graft_entry__ as g; g.build()"

``python -m functs_amd.aot`` does this for the benchmark programs of ``functs_amd.benchmark``
(both routes: the Region API and the TorchScript operator) and for the other spellings of the
detection head in ``functs_amd.configs.HEAD_VARIANTS``; with ``--plan-only`` it needs no GPU.
"""
import argparse
import contextlib
import os

from . import _lib

SPEC_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "fxhip", "spec")


@contextlib.contextmanager
def capture(directory: str = SPEC_DIR, program_tables: bool = True, rowstream: bool = True):
    """Every region planned inside the block that has no compiled kernels linked in writes
    ``fx_spec_<key>.hip`` (its programs as a table for the generic kernels) and, when it has a
    row-stream form, ``fx_rs_<key>.hip`` into ``directory``."""
    os.makedirs(directory, exist_ok=True)
    _lib.lib.fx_spec_dump_what((1 if program_tables else 0) | (2 if rowstream else 0))
    _lib.check(_lib.lib.fx_spec_dump_dir(directory.encode()))
    try:
        yield directory
    finally:
        _lib.check(_lib.lib.fx_spec_dump_dir(None))
        _lib.lib.fx_spec_dump_what(3)


def linked() -> int:
    """Number of specialised regions linked into the loaded library."""
    return int(_lib.lib.fx_specialization_count())


def enable(on: bool = True) -> None:
    """Process-wide switch between compiled kernels (default) and the interpreter."""
    _lib.lib.fx_set_specialization(1 if on else 0)


def launch_stats():
    """(kernel launches so far, launches that ran compiled kernels)."""
    import ctypes
    total, spec = ctypes.c_uint64(), ctypes.c_uint64()
    _lib.lib.fx_launch_stats(ctypes.byref(total), ctypes.byref(spec))
    return int(total.value), int(spec.value)


def plan(fn):
    """Plan every ``tssa::ParallelFunctor`` of a built function for the static types of the example
    it was built with (nothing runs; no GPU needed).  Returns one line per functor."""
    from . import _C
    graphs = [fn.graph] if hasattr(fn, "graph") else []
    for v in (getattr(fn, "_variants", None) or {}).values():
        g = getattr(v, "graph", None)
        if g is not None and all(g is not h for h in graphs):
            graphs.append(g)
    report = []
    for g in graphs:
        report += list(_C._plan_functors(g))
    return report


def _plan_region(region, *args):
    arr, n, _ = region._flatten(args)
    region.plan(arr, n)


def _plan_benchmark_programs(names):
    """The device-free form of _run_benchmark_programs: every region is planned, none is run."""
    import torch
    import functs_amd.jit as fj
    from . import Region, configs
    from .benchmark import PROGRAMS
    from .benchmark.inputs import INPUTS
    for name in names:
        if name not in INPUTS:
            continue
        cpu_args = INPUTS[name](0)
        for line in plan(fj.build(fj.script(PROGRAMS[name]), list(cpu_args))):
            print("  %s: %s" % (name, line))
        if name == "c1":
            a, b, n = cpu_args
            _plan_region(configs.build_c1(), b, n)
        elif name == "c2":
            _plan_region(configs.build_c2(), *cpu_args)
        elif name == "c5":
            _plan_region(configs.build_c5(cpu_args[0].size(0)), *cpu_args)
        elif name == "c3":
            loc, conf, priors = cpu_args
            _plan_region(configs.build_c3_decode(), *cpu_args)
            _plan_region(configs.build_c3_classes(80), torch.empty(priors.size(0), 4), torch.empty(priors.size(0), conf.size(-1)))
    if "variants" in names:
        # only their row-stream units: on the generic kernels these programs run interpreted
        _lib.lib.fx_spec_dump_what(2)
        preds, anchors, strides = INPUTS["c5"](0)
        for vname, kw in configs.HEAD_VARIANTS.items():
            r = configs.build_head_variant(batch=preds.size(0), **kw)
            _plan_region(r, preds, anchors, strides)
            info = r.rowstream_info(preds, anchors, strides)
            print("  head variant %s: row-stream key %016x%s" % (vname, info["key"], "" if info["ok"] else " (no row-stream form: %s)" % info["why"]))
        _lib.lib.fx_spec_dump_what(3)
    if "coverage" in names:
        _plan_region(configs.build_column_standardize(), torch.rand(*configs.COLUMN_STANDARDIZE_SHAPE))
        _plan_region(configs.build_row_filter(), *[torch.rand(*sh) - 0.5 for sh in configs.ROW_FILTER_SHAPES])
        for batch, levels in ((2, configs.GENERATED_ANCHOR_LEVELS), (16, configs.GENERATED_ANCHOR_LEVELS_C5)):
            # only the row-stream unit of the large instance: its program table is long, and the
            # generic kernels run it interpreted
            _lib.lib.fx_spec_dump_what(3 if batch == 2 else 2)
            _plan_region(configs.build_c5_generated_anchors(batch, levels), torch.empty(batch, sum(f * f * 3 for f, _ in levels), 85),
                         *[torch.empty(3, 4) for _ in levels])
        _lib.lib.fx_spec_dump_what(3)
    if "stream" in names:
        r = Region()
        xi = r.tensor_input(torch.float32, 2)
        r.output((xi * 2.0 + 1.0).sigmoid())
        _plan_region(r.finalize(), torch.empty(8192, 4096))


def _run_benchmark_programs(names):
    import torch
    import functs_amd.jit as fj
    from . import Region, configs
    from .benchmark import PROGRAMS
    from .benchmark.inputs import INPUTS
    dev = torch.device("cuda:0")

    def on_gpu(xs):
        return [x.to(dev) if isinstance(x, torch.Tensor) else x for x in xs]

    for name in names:
        if name not in INPUTS:
            continue
        cpu_args = INPUTS[name](0)
        # the TorchScript route: script -> build -> tssa::ParallelFunctor
        fn = fj.build(fj.script(PROGRAMS[name]), list(cpu_args))
        fn(*on_gpu(cpu_args))
        # the same configuration described through the Region API
        if name == "c1":
            a, b, n = cpu_args
            configs.build_c1()(*on_gpu((b, n)))
        elif name == "c2":
            configs.build_c2()(*on_gpu(cpu_args))
        elif name == "c5":
            configs.build_c5(cpu_args[0].size(0))(*on_gpu(cpu_args))
        elif name == "c3":
            decoded = configs.build_c3_decode()(*on_gpu(cpu_args))
            configs.build_c3_classes(80)(*decoded)
    if "coverage" in names:
        configs.build_column_standardize()(torch.rand(*configs.COLUMN_STANDARDIZE_SHAPE, device=dev))
    if "coverage" in names:
        configs.build_row_filter()(*[torch.rand(*sh, device=dev) - 0.5 for sh in configs.ROW_FILTER_SHAPES])
    if "stream" in names:
        x = torch.rand(8192, 4096, device=dev)
        r = Region()
        xi = r.tensor_input(torch.float32, 2)
        r.output((xi * 2.0 + 1.0).sigmoid())
        r.finalize()(x)
    torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--out", default=SPEC_DIR, help="directory the generated sources go to")
    ap.add_argument("--programs", default="c1,c2,c3,c4,c5,c5_nms,yolo_head,yolo_head_nms,attention,delta2bbox,variants,coverage,stream",
                    help="what to capture: benchmark programs, variants (other spellings of the detection head), "
                         "coverage, stream")
    ap.add_argument("--plan-only", action="store_true", help="plan the regions without running them: needs no GPU")
    args = ap.parse_args()
    names = [n for n in args.programs.split(",") if n]
    before = set(os.listdir(args.out)) if os.path.isdir(args.out) else set()
    with capture(args.out):
        if args.plan_only:
            _plan_benchmark_programs(names)
        else:
            _run_benchmark_programs([n for n in names if n != "variants"])
            if "variants" in names:
                _plan_benchmark_programs(["variants"])
    new = sorted(set(os.listdir(args.out)) - before)
    print("%d new specialised region(s) in %s" % (len(new), args.out))
    for f in new:
        print("  " + f)
    print("rebuild the library to link them: python -c \"import __graft_entry__ as g; g.build()\"")


if __name__ == "__main__":
    main()
