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

Use, for your own model (needs the GPU, because regions are planned when they first run)::

    import functs_amd.aot as aot
    with aot.capture():                 # default: functs_amd/csrc/fxhip/spec
        fn(*example_inputs)             # every region planned here leaves its source
    # then rebuild the library:  python -c "import __graft_entry__ as g; g.build()"

``python -m functs_amd.aot`` does this for the benchmark programs of
``functs_amd.benchmark`` (both routes: the Region API and the TorchScript operator).
"""
import argparse
import contextlib
import os

from . import _lib

SPEC_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "fxhip", "spec")


@contextlib.contextmanager
def capture(directory: str = SPEC_DIR):
    """Every region planned inside the block that has no compiled kernels linked in writes
    ``fx_spec_<key>.hip`` into ``directory``."""
    os.makedirs(directory, exist_ok=True)
    _lib.check(_lib.lib.fx_spec_dump_dir(directory.encode()))
    try:
        yield directory
    finally:
        _lib.check(_lib.lib.fx_spec_dump_dir(None))


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
    if "coverage" in names or len(names) == len(INPUTS):
        configs.build_column_standardize()(torch.rand(*configs.COLUMN_STANDARDIZE_SHAPE, device=dev))
    if "coverage" in names or len(names) == len(INPUTS):
        configs.build_row_filter()(*[torch.rand(*sh, device=dev) - 0.5 for sh in configs.ROW_FILTER_SHAPES])
    if "stream" in names or len(names) == len(INPUTS):
        x = torch.rand(8192, 4096, device=dev)
        r = Region()
        xi = r.tensor_input(torch.float32, 2)
        r.output((xi * 2.0 + 1.0).sigmoid())
        r.finalize()(x)
    torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--out", default=SPEC_DIR, help="directory the generated sources go to")
    ap.add_argument("--programs", default="c1,c2,c3,c4,c5", help="benchmark programs to capture")
    args = ap.parse_args()
    names = [n for n in args.programs.split(",") if n]
    before = set(os.listdir(args.out)) if os.path.isdir(args.out) else set()
    with capture(args.out):
        _run_benchmark_programs(names)
    new = sorted(set(os.listdir(args.out)) - before)
    print("%d new specialised region(s) in %s" % (len(new), args.out))
    for f in new:
        print("  " + f)
    print("rebuild the library to link them: python -c \"import __graft_entry__ as g; g.build()\"")


if __name__ == "__main__":
    main()
