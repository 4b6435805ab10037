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
    if not os.path.exists(_LSTM_SO):
        build()
    so = ctypes.CDLL(_LSTM_SO)
    fp = ctypes.c_void_p
    so.fx_lstm_emul.restype = ctypes.c_int
    so.fx_lstm_emul.argtypes = [fp] * 10 + [ctypes.c_int] * 4 + [ctypes.c_uint32, ctypes.c_int, ctypes.c_int, ctypes.c_uint32]
    return so


def _load():
    if not os.path.exists(_SO):
        build()
    so = ctypes.CDLL(_SO)
    so.fx_emul_run.restype = ctypes.c_int
    so.fx_emul_run.argtypes = [ctypes.POINTER(ctypes.c_uint32), ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
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
    dyn = ctypes.create_string_buffer(lib.fx_dyn_bytes())
    check(lib.fx_region_marshal(region._h, p.handle, arr, n, ptrs, scratch.data_ptr(), totals.data_ptr(), dyn, len(dyn)))
    words = ctypes.POINTER(ctypes.c_uint32)()
    nw = ctypes.c_size_t()
    check(lib.fx_plan_blob(p.handle, ctypes.byref(words), ctypes.byref(nw)))
    rc = _so.fx_emul_run(words, nw.value, dyn, totals.data_ptr())
    assert rc == 0
    if p.compact:
        tl = totals.tolist()
        outs = [[ten.narrow(0, 0, tl[t]) for t, ten in enumerate(row)] for row in outs]
    if region.is_map:
        return [list(r) for r in outs]
    return [r[0] for r in outs]
