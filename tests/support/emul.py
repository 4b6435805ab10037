"""Test-only: run a lowered region on the CPU through the scalar bytecode
emulator (tests/support/fx_emul.cpp).  Used to check the host lowering
against the oracle on machines without a GPU; never imported by the product."""
import ctypes
import os
import subprocess

import torch

from functs_amd import _lib
from functs_amd._lib import check, lib

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfx_emul.so")


_LSTM_SO = os.path.join(_HERE, "liblstm_emul.so")


def build():
    src = os.path.join(_HERE, "fx_emul.cpp")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", src, "-o", _SO])
    src = os.path.join(_HERE, "lstm_emul.cpp")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-pthread", src, "-o", _LSTM_SO])


def lstm_emul():
    """ctypes handle of the CPU build of the persistent LSTM kernel's schedule and barrier."""
    sources = [os.path.join(_HERE, "lstm_emul.cpp"), os.path.join(_HERE, "..", "..", "functs_amd", "csrc", "fxhip", "fx_lstm_sched.h")]
    if not os.path.exists(_LSTM_SO) or any(os.path.exists(s) and os.path.getmtime(s) > os.path.getmtime(_LSTM_SO) for s in sources):
        build()
    so = ctypes.CDLL(_LSTM_SO)
    fp = ctypes.c_void_p
    so.fx_lstm_emul.restype = ctypes.c_int
    so.fx_lstm_emul.argtypes = [fp] * 10 + [ctypes.c_int] * 4 + [ctypes.c_uint32, ctypes.c_int, ctypes.c_int, ctypes.c_uint32]
    so.fx_lstm_emul_give_up.restype = ctypes.c_int
    so.fx_lstm_emul_give_up.argtypes = [fp] * 10 + [ctypes.c_int] * 4 + [ctypes.c_uint32, ctypes.c_int]
    return so


def _load():
    sources = [os.path.join(_HERE, "fx_emul.cpp"), os.path.join(_HERE, "..", "..", "functs_amd", "csrc", "fxhip", "fx_bytecode.h")]
    if not os.path.exists(_SO) or any(os.path.exists(s) and os.path.getmtime(s) > os.path.getmtime(_SO) for s in sources):
        build()
    so = ctypes.CDLL(_SO)
    so.fx_emul_run.restype = ctypes.c_int
    so.fx_emul_run.argtypes = [ctypes.POINTER(ctypes.c_uint32), ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
    so.fx_emul_run_tables.restype = ctypes.c_int
    so.fx_emul_run_tables.argtypes = [ctypes.POINTER(ctypes.c_uint32), ctypes.c_size_t, ctypes.POINTER(ctypes.c_uint64),
                                      ctypes.POINTER(ctypes.c_uint32), ctypes.c_void_p]
    return so


_so = None


def run(region, *args):
    """Evaluate `region` on CPU tensors; returns what Region.__call__ returns."""
    global _so
    if _so is None:
        _so = _load()
    arr, n, keep = region._flatten(args)
    p = region.plan(arr, n)
    T = region.degree
    outs, ptrs = [], (ctypes.c_void_p * max(p.n_out * T, 1))()
    for o in range(p.n_out):
        row = []
        for t in range(T):
            dt, shape = p.out_meta[o][t]
            ten = torch.zeros(shape, dtype=dt)
            ptrs[o * T + t] = ten.data_ptr()
            row.append(ten)
        outs.append(row)
    scratch = torch.zeros(max(p.scratch_bytes, 1), dtype=torch.uint8)
    totals = torch.zeros(T, dtype=torch.int32)
    words = ctypes.POINTER(ctypes.c_uint32)()
    nw = ctypes.c_size_t()
    check(lib.fx_plan_blob(p.handle, ctypes.byref(words), ctypes.byref(nw)))
    n_p, n_s, uploaded = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_int()
    check(lib.fx_plan_table_sizes(p.handle, ctypes.byref(n_p), ctypes.byref(n_s), ctypes.byref(uploaded)))
    if uploaded.value:
        # a map of many tasks: the tables at their full length (on the device they are uploaded)
        tp, ts = (ctypes.c_uint64 * max(n_p.value, 1))(), (ctypes.c_uint32 * max(n_s.value, 1))()
        check(lib.fx_region_marshal_tables(region._h, p.handle, arr, n, ptrs, scratch.data_ptr(), totals.data_ptr(),
                                           tp, len(tp), ts, len(ts)))
        rc = _so.fx_emul_run_tables(words, nw.value, tp, ts, totals.data_ptr())
    else:
        dyn = ctypes.create_string_buffer(lib.fx_dyn_bytes())
        check(lib.fx_region_marshal(region._h, p.handle, arr, n, ptrs, scratch.data_ptr(), totals.data_ptr(), dyn, len(dyn)))
        rc = _so.fx_emul_run(words, nw.value, dyn, totals.data_ptr())
    assert rc == 0
    if p.compact:
        tl = totals.tolist()
        outs = [[ten.narrow(0, 0, tl[t]) for t, ten in enumerate(row)] for row in outs]
    if region.is_map:
        return [list(r) for r in outs]
    return [r[0] for r in outs]


# ---- generated row-stream kernels on the CPU ----------------------------------------------
_RS_SRC = os.path.join(_HERE, "fx_rs_host.cpp")
_RS_DIR = os.path.join(_HERE, "_rs_build")
_FXHIP = os.path.join(os.path.dirname(os.path.dirname(_HERE)), "functs_amd", "csrc", "fxhip")
_rs_cache = {}


def rowstream_host(region, *args, label="test"):
    """The row-stream unit the generator writes for `region` with these arguments, compiled for
    the CPU (tests/support/fx_rs_host.cpp); returns (ctypes handle, source text)."""
    src = region.rowstream_source(*args, label=label)
    key = region.rowstream_info(*args)["key"]
    if key in _rs_cache:
        return _rs_cache[key], src
    os.makedirs(_RS_DIR, exist_ok=True)
    gen = os.path.join(_RS_DIR, "fx_rs_%016x.hip" % key)
    so_path = os.path.join(_RS_DIR, "fx_rs_%016x.so" % key)
    with open(gen, "w") as f:
        f.write(src)
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-fPIC", "-shared", "-x", "c++", "-ffp-contract=off",
                           "-DFX_RS_GENERATED=\"%s\"" % gen, "-I", os.path.join(_FXHIP, "spec"), _RS_SRC, "-o", so_path])
    so = ctypes.CDLL(so_path)
    so.fx_rs_host_key.restype = ctypes.c_uint64
    so.fx_rs_host_launch_bytes.restype = ctypes.c_size_t
    so.fx_rs_host_run.restype = ctypes.c_int
    so.fx_rs_host_run.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32]
    assert so.fx_rs_host_key() == key
    _rs_cache[key] = so
    return so, src


def run_rowstream(region, *args, chunk_rows=100, sub_rows=None, threads=7):
    """Evaluate a compacting `region` on CPU tensors through its GENERATED row-stream code
    (compiled for the CPU); returns what Region.__call__ returns."""
    so, _ = rowstream_host(region, *args)
    arr, n, keep = region._flatten(args)
    p = region.plan(arr, n)
    T = region.degree
    outs, ptrs = [], (ctypes.c_void_p * max(p.n_out * T, 1))()
    for o in range(p.n_out):
        row = []
        for t in range(T):
            dt, shape = p.out_meta[o][t]
            ten = torch.zeros(shape, dtype=dt)
            ptrs[o * T + t] = ten.data_ptr()
            row.append(ten)
        outs.append(row)
    scratch = torch.zeros(max(p.scratch_bytes, 1), dtype=torch.uint8)
    totals = torch.zeros(T, dtype=torch.int32)
    dyn = ctypes.create_string_buffer(lib.fx_dyn_bytes())
    check(lib.fx_region_marshal(region._h, p.handle, arr, n, ptrs, scratch.data_ptr(), totals.data_ptr(), dyn, len(dyn)))
    la = ctypes.create_string_buffer(so.fx_rs_host_launch_bytes())
    info = region.rowstream_info(*args)
    max_sub = min(64, (6 * 256 * 4 - 6) // info["row_elements"])
    sub = max_sub if sub_rows is None else min(sub_rows, max_sub)
    check(lib.fx_plan_rowstream_launch(p.handle, min(chunk_rows, 256), sub, la, len(la)))
    rc = so.fx_rs_host_run(la, dyn, totals.data_ptr(), threads)
    assert rc == 0, rc
    tl = totals.tolist()
    outs = [[ten.narrow(0, 0, tl[t]) for t, ten in enumerate(row)] for row in outs]
    if region.is_map:
        return [list(r) for r in outs]
    return [r[0] for r in outs]
