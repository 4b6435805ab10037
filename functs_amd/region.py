"""Host-side mirror of the region interface on top of the C ABI.

A ``Region`` plays the role of the reference's ``GraphBuilder``
(fait/fuser/graph_builder.h:50-53): it is built once from the operators of a
fused functionalized subgraph, then called with the operator's run-time
arguments; it allocates the outputs (through torch, so they live in the
caching allocator on the current stream) and launches the HIP kernels.

Only device memory, streams and dtypes come from torch; all compute goes
through libfxhip.
"""
import ctypes

import torch

from . import _lib
from ._lib import C, FxArg, check, lib

_DT = {
    torch.float32: C["FX_DT_F32"],
    torch.int64: C["FX_DT_I64"],
    torch.int32: C["FX_DT_I32"],
    torch.uint8: C["FX_DT_U8"],
    torch.float16: C["FX_DT_F16"],
    torch.bfloat16: C["FX_DT_BF16"],
    torch.bool: C["FX_DT_BOOL"],
}
_DT_INV = {v: k for k, v in _DT.items()}


def fx_dtype(dt):
    if dt not in _DT:
        raise _lib.FxError(C["FX_E_UNSUPPORTED"], "dtype %s is not supported by fused regions" % dt)
    return _DT[dt]


class Val:
    """A value of a region under construction (tensor, scalar or list)."""

    __slots__ = ("region", "id")

    def __init__(self, region, vid):
        self.region = region
        self.id = vid

    # arithmetic sugar, so that tests read like the TorchScript they imitate
    def __add__(self, o): return self.region.op("ADD", self, o)
    def __radd__(self, o): return self.region.op("ADD", self, o)
    def __sub__(self, o): return self.region.op("SUB", self, o)
    def __rsub__(self, o): return self.region.op("RSUB", self, o)
    def __mul__(self, o): return self.region.op("MUL", self, o)
    def __rmul__(self, o): return self.region.op("MUL", self, o)
    def __truediv__(self, o): return self.region.op("DIV", self, o)
    def __neg__(self): return self.region.op("NEG", self)
    def __lt__(self, o): return self.region.op("LT", self, o)
    def __le__(self, o): return self.region.op("LE", self, o)
    def __gt__(self, o): return self.region.op("GT", self, o)
    def __ge__(self, o): return self.region.op("GE", self, o)
    def __and__(self, o): return self.region.op("AND", self, o)
    def __or__(self, o): return self.region.op("OR", self, o)

    def sigmoid(self): return self.region.op("SIGMOID", self)
    def exp(self): return self.region.op("EXP", self)
    def tanh(self): return self.region.op("TANH", self)
    def relu(self): return self.region.op("RELU", self)
    def clone(self): return self.region.op("CLONE", self)
    def select(self, dim, index): return self.region.op("SELECT", self, dim, index)
    def select_rev(self, src, dim, index): return self.region.op("SELECT_REV", self, src, dim, index)
    def slice(self, dim=0, start=None, end=None, step=1): return self.region.op("SLICE", self, dim, start, end, step)
    def slice_rev(self, src, dim=0, start=None, end=None, step=1):
        return self.region.op("SLICE_REV", self, src, dim, start, end, step)
    def squeeze(self, dim): return self.region.op("SQUEEZE", self, dim)
    def unsqueeze(self, dim): return self.region.op("UNSQUEEZE", self, dim)
    def view(self, *sizes): return self.region.op("VIEW", self, list(sizes[0]) if len(sizes) == 1 and isinstance(sizes[0], (list, tuple)) else list(sizes))
    reshape = view
    def permute(self, *dims): return self.region.op("PERMUTE", self, list(dims[0]) if len(dims) == 1 and isinstance(dims[0], (list, tuple)) else list(dims))
    def transpose(self, d0, d1): return self.region.op("TRANSPOSE", self, d0, d1)
    def expand(self, *sizes): return self.region.op("EXPAND", self, list(sizes[0]) if len(sizes) == 1 and isinstance(sizes[0], (list, tuple)) else list(sizes))
    def expand_as(self, other): return self.region.op("EXPAND_AS", self, other)
    def repeat(self, *reps): return self.region.op("REPEAT", self, list(reps[0]) if len(reps) == 1 and isinstance(reps[0], (list, tuple)) else list(reps))
    def index(self, idx): return self.region.op("INDEX", self, self.region.tensor_list([idx]))
    def clamp(self, min=None, max=None): return self.region.op("CLAMP", self, min, max)
    def softmax(self, dim): return self.region.op("SOFTMAX", self, dim)
    def to(self, dtype): return self.region.op("TO", self, dtype=dtype)


class _Plan:
    __slots__ = ("handle", "n_out", "out_meta", "scratch_bytes", "launches", "alg_bytes", "compact")


class Region:
    """Builder + runner of one fused region (``tssa::ParallelFunctor``)."""

    def __init__(self, parallel_degree=1, is_parallel_map=False):
        h = ctypes.c_void_p()
        check(lib.fx_region_create(int(parallel_degree), int(bool(is_parallel_map)), ctypes.byref(h)))
        self._h = h
        self.degree = int(parallel_degree)
        self.is_map = bool(is_parallel_map)
        self._inputs = []  # (kind, per_task)
        self._n_outputs = 0
        self._compact = False
        self._plans = {}
        self._scratch = {}
        self._totals = None

    def __del__(self):
        try:
            if self._h:
                lib.fx_region_destroy(self._h)
                self._h = None
        except Exception:
            pass

    # ---- values -------------------------------------------------------
    def _new(self, fn, *args):
        out = ctypes.c_int()
        check(fn(self._h, *args, ctypes.byref(out)))
        return Val(self, out.value)

    def tensor_input(self, dtype=torch.float32, rank=2, per_task=False):
        self._inputs.append(("tensor", bool(per_task)))
        return self._new(lib.fx_region_input_tensor, fx_dtype(dtype), int(rank), int(bool(per_task)))

    def scalar_input(self, kind, per_task=False):
        k = {"int": 1, "float": 2, "bool": 3}[kind]
        self._inputs.append((kind, bool(per_task)))
        return self._new(lib.fx_region_input_scalar, k, int(bool(per_task)))

    def task_index(self):
        return self._new(lib.fx_region_task_index)

    def loop_var(self):
        return self._new(lib.fx_region_loop_var)

    def const(self, x):
        if isinstance(x, Val):
            return x
        if x is None:
            return self._new(lib.fx_region_const_none)
        if isinstance(x, bool):
            return self._new(lib.fx_region_const_bool, int(x))
        if isinstance(x, int):
            return self._new(lib.fx_region_const_int, x)
        if isinstance(x, float):
            return self._new(lib.fx_region_const_float, x)
        if isinstance(x, (list, tuple)):
            return self.int_list(x)
        raise TypeError("cannot turn %r into a region value" % (x,))

    def _id_array(self, vals):
        ids = [self.const(v).id for v in vals]
        return (ctypes.c_int * max(len(ids), 1))(*ids), len(ids)

    def int_list(self, vals):
        arr, n = self._id_array(vals)
        return self._new(lib.fx_region_int_list, arr, n)

    def tensor_list(self, vals):
        arr, n = self._id_array(vals)
        return self._new(lib.fx_region_tensor_list, arr, n)

    def op(self, name, *args, dtype=None):
        code = C["FX_OP_" + name] if isinstance(name, str) else int(name)
        arr, n = self._id_array(args)
        return self._new(lib.fx_region_op, code, arr, n, -1 if dtype is None else fx_dtype(dtype))

    # creation ops
    def full(self, size, value, dtype=torch.float32):
        return self.op("FULL", self.int_list(size), value, dtype=dtype)

    def zeros(self, size, dtype=torch.float32):
        return self.full(size, 0, dtype)

    def arange(self, start, end, dtype=torch.int64):
        return self.op("ARANGE", start, end, dtype=dtype)

    def cat(self, tensors, dim=0):
        return self.op("CAT", self.tensor_list(tensors), dim)

    def stack(self, tensors, dim=0):
        return self.op("STACK", self.tensor_list(tensors), dim)

    def where(self, c, a, b):
        return self.op("WHERE", c, a, b)

    def output(self, v):
        check(lib.fx_region_output(self._h, v.id))
        self._n_outputs += 1

    def compact_rows(self, mask):
        check(lib.fx_region_compact_rows(self._h, mask.id))
        self._compact = True

    def finalize(self):
        check(lib.fx_region_finalize(self._h))
        return self

    # ---- run-time arguments -------------------------------------------
    def _flatten(self, args):
        """One FxArg per (input, task); returns (ctypes array, n, keep-alive list)."""
        if len(args) != len(self._inputs):
            raise _lib.FxError(C["FX_E_INVALID"], "region takes %d inputs, got %d" % (len(self._inputs), len(args)))
        flat = []
        for (kind, per_task), a in zip(self._inputs, args):
            items = list(a) if per_task else [a]
            if per_task and len(items) != self.degree:
                raise _lib.FxError(C["FX_E_INVALID"], "per-task input needs %d entries" % self.degree)
            for it in items:
                flat.append((kind, it))
        arr = (FxArg * max(len(flat), 1))()
        for i, (kind, it) in enumerate(flat):
            fa = arr[i]
            if kind == "tensor":
                if it.dim() > _lib.FX_ARG_MAX_RANK:
                    raise _lib.FxError(C["FX_E_UNSUPPORTED"], "tensor rank above %d" % _lib.FX_ARG_MAX_RANK)
                fa.kind = 0
                fa.dtype = fx_dtype(it.dtype)
                fa.ptr = it.data_ptr()
                fa.rank = it.dim()
                for d in range(it.dim()):
                    fa.sizes[d] = it.size(d)
                    fa.strides[d] = it.stride(d)
            elif kind == "int":
                fa.kind, fa.ival = 1, int(it)
            elif kind == "float":
                fa.kind, fa.fval = 2, float(it)
            else:
                fa.kind, fa.ival = 3, int(bool(it))
        return arr, len(flat), flat

    def plan(self, arr, n):
        h = ctypes.c_void_p()
        check(lib.fx_region_plan(self._h, arr, n, ctypes.byref(h)))
        p = self._plans.get(h.value)
        if p is None:
            p = _Plan()
            p.handle = h
            p.n_out = lib.fx_plan_num_outputs(h)
            p.out_meta = []
            dt, rk = ctypes.c_int32(), ctypes.c_int32()
            sizes = (ctypes.c_int64 * 8)()
            for o in range(p.n_out):
                per_task = []
                for t in range(self.degree):
                    check(lib.fx_plan_output(h, o, t, ctypes.byref(dt), ctypes.byref(rk), sizes))
                    per_task.append((_DT_INV[dt.value], tuple(sizes[i] for i in range(rk.value))))
                p.out_meta.append(per_task)
            p.scratch_bytes = lib.fx_plan_scratch_bytes(h)
            p.launches = lib.fx_plan_launches(h)
            p.alg_bytes = lib.fx_plan_algorithmic_bytes(h)
            p.compact = self._compact
            self._plans[h.value] = p
        return p

    def disasm(self, *args):
        arr, n, _ = self._flatten(args)
        p = self.plan(arr, n)
        buf = ctypes.create_string_buffer(1 << 20)
        check(lib.fx_plan_disasm(p.handle, buf, len(buf)))
        return buf.value.decode()

    def specialized(self, *args):
        """True if calls with these arguments run ahead-of-time compiled kernels
        (``python -m functs_amd.aot``) instead of the bytecode interpreter."""
        arr, n, _ = self._flatten(args)
        return bool(lib.fx_plan_specialized(self.plan(arr, n).handle))

    def spec_source(self, *args, label=""):
        """HIP translation unit that specialises the kernels for these arguments."""
        arr, n, _ = self._flatten(args)
        p = self.plan(arr, n)
        buf = ctypes.create_string_buffer(1 << 22)
        check(lib.fx_plan_spec_source(p.handle, label.encode(), buf, len(buf)))
        return buf.value.decode()

    def rowstream_info(self, *args):
        """Row-stream form of a compacting region for these arguments (fx_plan_rowstream_info):
        a dict with `ok` (the form exists), `active` (a generated kernel for it is linked and
        enabled), `key`, `row_elements`, `rows`, `tasks`, `inputs` and, when not ok, `why`."""
        arr, n, _ = self._flatten(args)
        p = self.plan(arr, n)
        out = (ctypes.c_int64 * 8)()
        check(lib.fx_plan_rowstream_info(p.handle, out, 8))
        why = ctypes.create_string_buffer(512)
        check(lib.fx_plan_rowstream_why(p.handle, why, len(why)))
        return {"ok": bool(out[0]), "active": bool(out[1]), "key": (int(out[3]) << 32) | int(out[2]), "row_elements": int(out[4]),
                "rows": int(out[5]), "tasks": int(out[6]), "inputs": int(out[7]), "why": why.value.decode()}

    def rowstream_source(self, *args, label=""):
        """HIP translation unit of the generated row-stream kernel for these arguments."""
        arr, n, _ = self._flatten(args)
        p = self.plan(arr, n)
        buf = ctypes.create_string_buffer(1 << 22)
        check(lib.fx_plan_rowstream_source(p.handle, label.encode(), buf, len(buf)))
        return buf.value.decode()

    def spec_key(self, *args):
        arr, n, _ = self._flatten(args)
        return int(lib.fx_plan_spec_key(self.plan(arr, n).handle))

    def bind(self, *args):
        """Resolve the plan for these arguments and allocate outputs; returns a
        ``BoundCall`` whose ``launch()`` only marshals and launches."""
        arr, n, keep = self._flatten(args)
        p = self.plan(arr, n)
        return BoundCall(self, p, arr, n, keep, args)

    def __call__(self, *args):
        bc = self.bind(*args)
        bc.launch()
        return bc.results()


class BoundCall:
    """A region bound to concrete arguments: outputs allocated, ready to launch."""

    def __init__(self, region, plan, arr, n, keep, args):
        self.region, self.plan, self.arr, self.n, self._keep, self.args = region, plan, arr, n, keep, args
        dev = None
        for kind, it in keep:
            if kind == "tensor":
                dev = it.device
                break
        if dev is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        if dev.type != "cuda":
            raise _lib.FxError(C["FX_E_NODEVICE"], "fused regions run on the GPU only (got %s tensors)" % dev)
        self.device = dev
        T = region.degree
        self.outs = []
        self._batched = []
        ptrs = (ctypes.c_void_p * max(plan.n_out * T, 1))()
        for o in range(plan.n_out):
            row = []
            metas = [plan.out_meta[o][t] for t in range(T)]
            if T > 1 and all(m == metas[0] for m in metas):
                # one allocation per output, the tasks' tensors at equal, 256-byte aligned distances
                # (what tssa::ParallelFunctor does as well): `batched` hands it on as [T, ...]
                dt, shape = metas[0]
                numel = 1
                for d in shape:
                    numel *= d
                per = 256 // torch.empty(0, dtype=dt).element_size()
                stride = max(-(-numel // per) * per, per)
                buf = torch.empty(T * stride, dtype=dt, device=dev)
                inner = torch.empty(shape, dtype=dt, device="meta").stride()
                whole = buf.as_strided((T,) + tuple(shape), (stride,) + tuple(inner))
                self._batched.append(whole)
                row = [whole[t] for t in range(T)]
            else:
                self._batched.append(None)
                row = [torch.empty(shape, dtype=dt, device=dev) for dt, shape in metas]
            for t, ten in enumerate(row):
                ptrs[o * T + t] = ten.data_ptr()
            self.outs.append(row)
        self.ptrs = ptrs
        self.scratch = torch.empty(max(plan.scratch_bytes, 1), dtype=torch.uint8, device=dev) if (plan.compact or plan.scratch_bytes > 0) else None
        self.totals = torch.zeros(T, dtype=torch.int32).pin_memory() if plan.compact else None
        self._stream = None

    def launch(self, stream=None):
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        self._stream = stream
        check(lib.fx_region_run(self.region._h, self.plan.handle, self.arr, self.n, self.ptrs,
                                self.scratch.data_ptr() if self.scratch is not None else None,
                                self.totals.data_ptr() if self.totals is not None else None,
                                ctypes.c_void_p(stream)))

    def launch_timed(self, stream=None, repeat=1):
        """launch() with HIP events around every kernel; returns the list of
        kernel durations in milliseconds (synchronises).  With repeat > 1 every kernel is
        launched that many times back to back inside its event pair and the mean is returned:
        the overhead of the pair (about 2 us) is spread over the batch."""
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        self._stream = stream
        ms = (ctypes.c_float * 4)()
        nk = ctypes.c_int()
        check(lib.fx_region_run_timed_batched(self.region._h, self.plan.handle, self.arr, self.n, self.ptrs,
                                              self.scratch.data_ptr() if self.scratch is not None else None,
                                              self.totals.data_ptr() if self.totals is not None else None,
                                              ctypes.c_void_p(stream), int(repeat), ms, 4, ctypes.byref(nk)))
        return [ms[i] for i in range(nk.value)]

    def batched(self, o):
        """Output `o` of a map whose tasks all have the same shape as one tensor [T, ...] over the
        tasks' buffers (dimension 0 strided), rows past a task's kept-row count unspecified; the
        counts are `totals` (pinned host memory, written by the kernels).  A consumer on the same
        stream that reads the counts from memory needs no synchronisation with the host."""
        if self._batched[o] is None:
            raise _lib.FxError(C["FX_E_INVALID"], "output %d is not one buffer (tasks of different shapes)" % o)
        return self._batched[o]

    def results(self):
        """Outputs as the operator returns them: a tensor per output, or a list
        of per-task tensors for a ParallelMap.  Compacted outputs are narrowed to
        the kept rows: this waits for the kept-row counts, which the kernels store
        early (ATen's nonzero waits for the whole stream); the outputs are valid in
        stream order."""
        if self.plan.compact:
            stream = self._stream if self._stream is not None else torch.cuda.current_stream(self.device).cuda_stream
            check(lib.fx_region_wait_totals(self.plan.handle, self.totals.data_ptr(), ctypes.c_void_p(stream)))
            totals = self.totals.tolist()
            outs = [[ten.narrow(0, 0, totals[t]) for t, ten in enumerate(row)] for row in self.outs]
        else:
            outs = self.outs
        if self.region.is_map:
            return [list(row) for row in outs]
        return [row[0] for row in outs]


def timed_sets(bound, which=-1, rounds=1, stream=None):
    """Mean duration in milliseconds of a call (which < 0) or of kernel `which` of a call,
    launched over the BoundCalls in `bound` in rotation inside one HIP event pair
    (fx_region_run_timed_sets).  All of them must come from the same region and plan."""
    b0 = bound[0]
    assert all(b.region is b0.region and b.plan.handle.value == b0.plan.handle.value for b in bound)
    if stream is None:
        stream = torch.cuda.current_stream(b0.device).cuda_stream
    k = len(bound)
    args = (ctypes.POINTER(FxArg) * k)(*[ctypes.cast(b.arr, ctypes.POINTER(FxArg)) for b in bound])
    outs = (ctypes.POINTER(ctypes.c_void_p) * k)(*[ctypes.cast(b.ptrs, ctypes.POINTER(ctypes.c_void_p)) for b in bound])
    scr = (ctypes.c_void_p * k)(*[b.scratch.data_ptr() if b.scratch is not None else None for b in bound])
    tot = (ctypes.c_void_p * k)(*[b.totals.data_ptr() if b.totals is not None else None for b in bound])
    ms = ctypes.c_float()
    check(lib.fx_region_run_timed_sets(b0.region._h, b0.plan.handle, k, args, b0.n, outs, scr, tot,
                                       ctypes.c_void_p(stream), int(which), int(rounds), ctypes.byref(ms)))
    for b in bound:
        b._stream = stream
    return ms.value


def compact_rows(mask, cols):
    """Stand-alone ``[c[mask] for c in cols]`` through fx_compact_rows."""
    n = mask.numel()
    m8 = mask.view(torch.uint8) if mask.dtype == torch.bool else mask
    dev = mask.device
    k = len(cols)
    src = (ctypes.c_void_p * max(k, 1))()
    dst = (ctypes.c_void_p * max(k, 1))()
    rowlen = (ctypes.c_int32 * max(k, 1))()
    elsize = (ctypes.c_int32 * max(k, 1))()
    outs = []
    for i, c in enumerate(cols):
        c = c.contiguous()
        o = torch.empty_like(c)
        outs.append(o)
        src[i], dst[i] = c.data_ptr(), o.data_ptr()
        rowlen[i] = max(c.numel() // max(n, 1), 1) if n else 1
        elsize[i] = c.element_size()
        cols[i] = c
    sb = lib.fx_compact_rows_scratch_bytes(n)
    scratch = torch.empty(sb, dtype=torch.uint8, device=dev)
    total = torch.zeros(1, dtype=torch.int32).pin_memory()
    check(lib.fx_compact_rows(m8.data_ptr(), n, src, dst, rowlen, elsize, k, scratch.data_ptr(), sb, total.data_ptr(),
                              ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))
    torch.cuda.current_stream(dev).synchronize()
    t = int(total[0])
    return [o.narrow(0, 0, t) for o in outs]
