"""TorchScript front end: functionalize a program and run its fused regions on
the GPU through ``tssa::ParallelFunctor``.

Same entry points as the reference's ``functs.jit`` (functs/jit/_script.py:12-110):
``script`` functionalizes, ``build`` forms regions and returns a callable,
``shape_infer`` refines the graph's argument types from example inputs.
"""
import inspect
import os
from typing import List, Sequence

import torch

from . import _C  # noqa: F401  (registers immut:: operators and tssa::ParallelFunctor)


def _shape_key(args):
    """Hash of the shapes and dtypes of the tensor arguments (lists of tensors element by element)."""
    return _C._shape_key(*args)


class AotScriptFunction(object):
    """Callable around the compiled graph (functs/jit/_script.py:12-26).

    The pipeline folds what the example's shapes answer (``x.size(0)``, ``len(xs)``, dtypes) into
    constants, as the reference's does: a graph built that way serves arguments of those shapes
    only.  Such a function keeps the functionalized script it was built from and builds a graph
    per set of argument shapes, the first one from the example; ``graph`` is that first one."""

    def __init__(self, aot_script_fn, source=None, key=None, lazy_lists=False, padded_outputs=False, **kwargs):
        self._aot_script_fn = aot_script_fn
        self._source = source
        self._lazy_lists = lazy_lists
        self._padded_outputs = padded_outputs
        self._call = _direct(aot_script_fn, lazy_lists)
        self._variants = {key: self._call} if source is not None else None

    @property
    def graph(self):
        return self._aot_script_fn.graph

    def __call__(self, *args, **kwargs):
        if kwargs:   # by name: through the ScriptFunction, which knows the argument names
            if self._variants is not None or self._lazy_lists:
                raise TypeError("this built function takes positional arguments only")
            return self._aot_script_fn(*args, **kwargs)
        if self._variants is None:
            return self._call(*args)
        key = _shape_key(args)
        fn = self._variants.get(key)
        if fn is None:
            fn = self._variants[key] = _direct(_compile(self._source, args, self._padded_outputs)[0], self._lazy_lists)
        return fn(*args)


def _direct(script_fn, lazy_lists=False):
    """What a call of a built function runs: a graph that is one tssa::ParallelFunctor over the
    arguments is called without the TorchScript interpreter (functs_amd._C.DirectFunctor: same
    operator, same results), any other graph through its ScriptFunction."""
    direct = _C._direct_functor(script_fn.graph)
    if direct is None:
        if lazy_lists:
            raise ValueError("lazy_lists needs a function that builds into one fused region")
        return script_fn
    direct.lazy_lists = lazy_lists
    return direct


def extract_type_hint_from_tensor(input_):
    """functs/jit/_script.py:29-49"""
    if isinstance(input_, bool):
        return torch.BoolType.get()
    if isinstance(input_, int):
        return torch.IntType.get()
    if isinstance(input_, float):
        return torch.FloatType.get()
    if isinstance(input_, torch.Tensor):
        return torch.TensorType.get().with_dtype(input_.dtype).with_sizes(list(input_.shape)).with_device(input_.device)
    if isinstance(input_, (list, tuple)):
        return torch.TupleType([extract_type_hint_from_tensor(e) for e in input_])
    raise TypeError("unsupported type {} at the type hint stage".format(type(input_)))


def _graph_of(fn):
    if isinstance(fn, AotScriptFunction):
        return fn.graph
    return fn.graph


def shape_infer(fn, example_input: Sequence[object], refined_types=None) -> None:
    """Give the graph's tensor arguments the dtype / rank / device of the examples
    (functs/jit/_script.py:52-55).  Regions specialise on the shapes they are
    called with, so nothing else has to be propagated ahead of time."""
    g = _graph_of(fn)
    hints = [extract_type_hint_from_tensor(i) for i in example_input]
    inputs = list(g.inputs())
    off = len(inputs) - len(hints)
    for v, t in zip(inputs[off:], hints):
        if isinstance(t, torch.TensorType):
            v.setType(t)


def _strip_self(g):
    inputs = list(g.inputs())
    if inputs and inputs[0].debugName().startswith("self") and not inputs[0].uses():
        g.eraseInput(0)


class GraphedFunction(AotScriptFunction):
    """A built function whose whole call is one HIP graph: for programs whose loops
    stay host loops (carried state, e.g. an LSTM) the per-launch host work of
    hundreds of small kernels is paid once, at capture.

    The first call with a given set of tensor shapes runs the function twice on a
    side stream (variants get compiled, workspaces allocated), then captures it with
    private input buffers; later calls copy the arguments into those buffers, replay
    and return clones of the captured outputs.  Non-tensor arguments are baked into
    the capture, so they are part of the key.  A function with a row-compacting
    region cannot be captured: its output shapes need a synchronisation per call.
    """

    def __init__(self, aot_script_fn, source=None, key=None):
        super().__init__(aot_script_fn, source=source, key=key)
        if "compact_rows=1" in str(aot_script_fn.graph):
            raise ValueError("a function with a row-compacting region cannot run as a HIP graph")
        self._captures = {}

    @staticmethod
    def _key(args):
        k = []
        for a in args:
            if isinstance(a, torch.Tensor):
                k.append((tuple(a.shape), a.dtype, a.device))
            elif isinstance(a, (list, tuple)) and a and isinstance(a[0], torch.Tensor):
                k.append(tuple((tuple(t.shape), t.dtype, t.device) for t in a))
            else:
                k.append(repr(a))
        return tuple(k)

    @staticmethod
    def _map(x, f):
        if isinstance(x, torch.Tensor):
            return f(x)
        if isinstance(x, (list, tuple)):
            return type(x)(GraphedFunction._map(e, f) for e in x)
        return x

    def __call__(self, *args):
        key = self._key(args)
        cap = self._captures.get(key)
        if cap is None:
            static = [self._map(a, lambda t: t.clone()) for a in args]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            run = super().__call__   # (builds the graph for these shapes first, if they are new)
            with torch.cuda.stream(side):
                for _ in range(2):
                    run(*static)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out = run(*static)
            cap = self._captures[key] = (graph, static, out)
        graph, static, out = cap

        def refill(dst, src):
            if isinstance(dst, torch.Tensor):
                dst.copy_(src)
            elif isinstance(dst, (list, tuple)):
                for d, s_ in zip(dst, src):
                    refill(d, s_)

        for d, a in zip(static, args):
            refill(d, a)
        graph.replay()
        return self._map(out, lambda t: t.clone())


def build(fn, example_input: List[object], hip_graph: bool = False, lazy_lists: bool = False,
          padded_outputs: bool = False, compile_kernels=None) -> AotScriptFunction:
    """Form fused regions in a functionalized script and return the callable
    (functs/jit/_script.py:58-73).  ``hip_graph=True`` returns a ``GraphedFunction``.
    ``lazy_lists=True`` (a function that builds into ONE fused region only): List[Tensor] results
    come back as ``functs_amd._C.TensorList`` - a sequence whose elements become Python tensors when
    they are read (len, indexing, iteration, ``tolist()``) - instead of Python lists, which cost a
    wrapper object per element on every call (a map over 80 tasks returns 160 tensors).
    ``padded_outputs=True``: row-compacting regions whose results the function returns hand them
    back at full size (a map: one tensor [tasks, rows, ...] per result) without waiting for the
    kept-row counts, which come as one more tensor at the end of the result tuple (int32, pinned
    host memory that the kernels write; rows from counts[task] on hold no values): for callers that
    pass the results on to work on the same stream.
    ``compile_kernels=True``: the regions of the built function that have no kernels linked into
    the library get theirs now: row compactions with a row-stream form their one-launch kernel,
    dense regions with programs of up to 256 instructions the compiled dense kernels (generated
    for the example's static types, compiled with hipcc into the kernel cache, 3 to 20 seconds per
    region the first time; later processes load them from the cache): where the reference
    generates and compiles code per subgraph when the operator is made
    (fait/fuser/graph_builder.cpp:259-712).  ``compile_kernels="dense"`` instantiates the general
    kernels for every dense region's programs (two minutes for 1 500 instructions), ``"all"`` for
    every region, ``"none"`` for none (row-stream kernels only).  Left
    at None the environment decides: ``FUNCTS_AMD_COMPILE_KERNELS=1`` (or ``dense`` / ``all``)
    switches it on for code that calls ``build`` the reference's way."""
    if not isinstance(fn, (torch.jit.ScriptFunction, torch.jit.ScriptModule)):
        raise AttributeError("only a functionalized jit script can be built")
    aot, specialized = _compile(fn, example_input, padded_outputs)
    source, key = (fn, _shape_key(example_input)) if specialized else (None, None)
    if compile_kernels is None:
        env = os.environ.get("FUNCTS_AMD_COMPILE_KERNELS", "0").strip().lower()
        compile_kernels = env if env in ("dense", "all", "none", "auto") else env not in ("", "0", "false", "no")
    if compile_kernels:
        from . import aot as _aot
        _aot.compile_missing(aot, tables=compile_kernels if isinstance(compile_kernels, str) else "auto")
    if hip_graph:
        return GraphedFunction(aot, source, key)
    return AotScriptFunction(aot, source, key, lazy_lists=lazy_lists, padded_outputs=padded_outputs)


def _compile(fn, example_input, padded_outputs=False):
    """(compiled function, whether its graph holds constants of the example's shapes)"""
    g = fn.graph.copy()
    if isinstance(fn, torch.jit.ScriptModule):
        _strip_self(g)
    hints = [extract_type_hint_from_tensor(i) for i in example_input]
    specialized = bool(_C._jit_pass_fait_pipeline(g, hints))
    if padded_outputs:
        _C._jit_pass_pad_compacted_results(g)
    return _C._create_function_from_graph("forward", g), specialized


def script(fn, backend="jit", remove_update=True, enable_dce_cse=True, add_clone=False):
    """TorchScript-compile ``fn`` and rewrite every tensor mutation into
    immut:: Access / Assign chains (functs/jit/_script.py:76-110)."""
    if backend not in ("jit", "aot"):
        raise AttributeError("No backend named {}".format(backend))
    jit_fn = torch.jit.script(fn)
    is_function = inspect.isfunction(fn)
    if is_function:
        # torch.jit.script hands out one cached ScriptFunction per Python function, and
        # its executor may already hold a plan: rewrite a private copy of the graph
        g = jit_fn.graph.copy()
    else:
        if torch.cuda.is_available():
            jit_fn = jit_fn.cuda()
        jit_fn = torch.jit.freeze(jit_fn.eval())
        g = jit_fn.graph
    if add_clone:
        _C._jit_pass_dumb_remove_inter_precedure_mutation(g)
    torch._C._jit_pass_inline(g)
    _C._jit_pass_convert_to_tensorssa(g)
    if remove_update:
        _C._jit_pass_tensorssa_remove_update(g)
    if enable_dce_cse:
        torch._C._jit_pass_dce(g)
        torch._C._jit_pass_cse(g)
        torch._C._jit_pass_constant_propagation(g)
    if is_function:
        return torch._C._create_function_from_graph(fn.__name__, g)
    return jit_fn
