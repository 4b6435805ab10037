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

Or at run time, where ``hipcc`` is at hand (the reference's way: code per subgraph when the
operator is first made): ``functs_amd.jit.build(..., compile_kernels=True)`` or
``aot.compile_missing(fn)`` plans the function's regions, compiles the units that are not linked
into small shared objects of their own and loads them; they register with the loaded library
like the linked ones (row-stream units take seconds; the general kernels instantiated for a
region's programs seconds to minutes, so by default only dense regions with short programs get
them: `tables`).  The objects are kept in ``kernel_cache_dir()`` and
loaded again by every later process (``load_cached_kernels``, called when the package is
imported).

``python -m functs_amd.aot`` does this for the benchmark programs of ``functs_amd.benchmark``
(both routes: the Region API and the TorchScript operator) and for the other spellings of the
detection head in ``functs_amd.configs.HEAD_VARIANTS``; with ``--plan-only`` it needs no GPU.
"""
import argparse
import contextlib
import ctypes
import glob
import hashlib
import os
import re
import shutil
import subprocess
import tempfile

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


# ---- kernels compiled at run time ---------------------------------------------------------------
_FXHIP_DIR = os.path.dirname(SPEC_DIR)
_HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]   # as csrc/fxhip/Makefile
_loaded = {}   # path -> CDLL (kept: the library calls into them)
AUTO_TABLE_INSNS = 256   # program tables up to this many instructions are compiled without being asked for (about 20 s)


def _abi_tag() -> str:
    """Kernels are compiled against the library's headers: a cache per state of those."""
    h = hashlib.sha1()
    for f in sorted(glob.glob(os.path.join(_FXHIP_DIR, "*.h"))):
        with open(f, "rb") as fh:
            h.update(os.path.basename(f).encode())
            h.update(fh.read())
    return h.hexdigest()[:16]


def kernel_cache_dir() -> str:
    """Where kernels compiled at run time are kept: ``$FUNCTS_AMD_KERNEL_CACHE`` or
    ``functs_amd/lib/jit``, in a directory per state of the library's headers."""
    base = os.environ.get("FUNCTS_AMD_KERNEL_CACHE") or os.path.join(os.path.dirname(_lib.LIB_PATH), "jit")
    return os.path.join(base, _abi_tag())


def hipcc_path():
    """The HIP compiler driver, or None."""
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _load_kernel_object(path: str) -> None:
    if path not in _loaded:
        # its static initialisers hand the kernels to the loaded library (fx_spec_register / fx_rs_register)
        _loaded[path] = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


def load_cached_kernels() -> int:
    """Loads every kernel object of kernel_cache_dir(); returns how many are loaded."""
    d = kernel_cache_dir()
    if os.path.isdir(d):
        for path in sorted(glob.glob(os.path.join(d, "fx_*.so"))):
            try:
                _load_kernel_object(path)
            except OSError:
                pass   # a stale or half-written object: compile_missing writes it again
    return len(_loaded)


def compile_sources(directory: str, verbose: bool = False, tables: str = "auto"):
    """Compiles the generated units of `directory` that have no object in the cache yet into
    shared objects there and loads them.  Every row-stream unit (``fx_rs_*.hip``: straight-line
    code, seconds) is compiled; of the program tables (``fx_spec_*.hip``: the general kernels
    instantiated for a region's programs: 5 s for a few instructions, 10 s for fifty, two minutes
    for 1 500) those of dense regions with at most AUTO_TABLE_INSNS instructions (`tables` =
    "auto", the default), of all dense regions ("dense"), all ("all") or none ("none").  Regions
    left out keep the interpreter.  Returns the names compiled."""
    cc = hipcc_path()
    if cc is None:
        raise RuntimeError("no hipcc found (PATH, $HIPCC, /opt/rocm/bin): generate the sources with aot.capture() and "
                           "build them into the library instead")
    out_dir = kernel_cache_dir()
    os.makedirs(out_dir, exist_ok=True)
    lib_dir = os.path.dirname(_lib.LIB_PATH)
    done = []
    for src in sorted(glob.glob(os.path.join(directory, "fx_*.hip"))):
        name = os.path.splitext(os.path.basename(src))[0]
        if name.startswith("fx_spec_"):
            with open(src) as fh:
                text = fh.read()
            dense = "FX_SPEC_DENSE" in text
            m = re.search(r"FxInsn code\[(\d+)\]", text)
            n_insn = int(m.group(1)) if m else 1 << 30
            if tables == "none" or (tables == "dense" and not dense) or (tables == "auto" and not (dense and n_insn <= AUTO_TABLE_INSNS)):
                continue
        obj = os.path.join(out_dir, name + ".so")
        if not os.path.isfile(obj):
            tmp = obj + ".%d.tmp" % os.getpid()
            cmd = [cc] + _HIPCC_FLAGS + ["-shared", "-I", SPEC_DIR, src, "-o", tmp, "-L", lib_dir, "-lfxhip", "-Wl,-rpath," + lib_dir]
            if verbose:
                print("[functs_amd.aot] compiling %s" % name, flush=True)
            res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
            if res.returncode != 0:
                if os.path.exists(tmp):
                    os.unlink(tmp)
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, res.stderr[-2000:]))
            os.replace(tmp, obj)
            done.append(name)
        _load_kernel_object(obj)
    return done


def compile_missing(fn=None, planner=None, verbose: bool = False, tables: str = "auto"):
    """Plans the regions of a built function (or whatever `planner()` plans) for the static types
    of its example, and compiles and loads the kernels that are not linked in.  Needs no GPU.
    Returns the names of the units compiled now."""
    tmp = tempfile.mkdtemp(prefix="functs_amd_src_")
    try:
        with capture(tmp):
            if fn is not None:
                plan(fn)
            if planner is not None:
                planner()
        return compile_sources(tmp, verbose=verbose, tables=tables)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


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
