"""ORACLE - test infrastructure only (see oracle/configs.py).

Element-by-element numpy restatement of the reference's index arithmetic for
the immut:: access / assign operators, one function per lowering:

  select      computeImmutSelect     functs/csrc/jit/tensorexpr/nnc_ext.cpp:166-185
              (+ negative index wrap, fait/fuser/custom_lowering_func.cpp:190-191)
  select_rev  computeImmutSelectRev  nnc_ext.cpp:187-212
  slice       computeSlice           custom_lowering_func.cpp:200-227
  slice_rev   computeImmutSliceRev   nnc_ext.cpp:112-164 (clamping variant)
  unsqueeze   computeImmutUnsqueeze  nnc_ext.cpp:214-229
  view        computeImmutView       nnc_ext.cpp:231-295
  permute     computeImmutPermute    nnc_ext.cpp:320-358
  expand      computeImmutExpand     nnc_ext.cpp:360-370, 32-53
  repeat      computeImmutRepeat     nnc_ext.cpp:297-318
  index       computeImmutIndex      nnc_ext.cpp:372-392
  cat / stack computeCat / Stack     custom_lowering_func.cpp:297-350
  triu        computeTriu            custom_lowering_func.cpp:41-49

Each function loops over OUTPUT coordinates and evaluates the load expression
the lowering builds - deliberately not a call to the matching numpy/torch
routine.  Pinned in tests/test_oracle.py against the ATen operators (library
routines, which the reference itself registers as the eager bodies:
functs/csrc/jit/ir/symbol_ext.cpp:17-117) over every dim / index / bound
combination of small shapes, and against the reference-held cases of
tests/golden/lowering_tests.json.
"""
import itertools

import numpy as np


def _coords(shape):
    return itertools.product(*[range(s) for s in shape])


def _norm_slice(size, start, end):
    s = 0 if start is None else start
    e = size if end is None else end
    s = min(s, size) if s >= 0 else s + size
    e = min(e, size) if e >= 0 else e + size
    s = max(s, 0)
    e = max(e, s)
    return s, e


def select(src, dim, index):
    dim %= src.ndim
    if index < 0:
        index += src.shape[dim]
    out_shape = src.shape[:dim] + src.shape[dim + 1:]
    out = np.empty(out_shape, src.dtype)
    for ax in _coords(out_shape):
        idx = ax[:dim] + (index,) + ax[dim:]
        out[ax] = src[idx]
    return out


def select_rev(self, src, dim, index):
    dim %= self.ndim
    if index < 0:
        index += self.shape[dim]
    out = np.empty(self.shape, self.dtype)
    for ax in _coords(self.shape):
        src_ax = ax[:dim] + ax[dim + 1:]
        out[ax] = src[src_ax] if ax[dim] == index else self[ax]
    return out


def slice_(src, dim, start, end, step):
    dim %= src.ndim
    s, e = _norm_slice(src.shape[dim], start, end)
    n = (e - s + step - 1) // step
    out_shape = src.shape[:dim] + (n,) + src.shape[dim + 1:]
    out = np.empty(out_shape, src.dtype)
    for ax in _coords(out_shape):
        idx = list(ax)
        idx[dim] = s + step * ax[dim]
        out[ax] = src[tuple(idx)]
    return out


def slice_rev(self, src, dim, start, end, step):
    dim %= self.ndim
    s, e = _norm_slice(self.shape[dim], start, end)
    out = np.empty(self.shape, self.dtype)
    for ax in _coords(self.shape):
        d = ax[dim]
        not_set = d < s or d >= e or (d - s) % step != 0
        if not_set:
            out[ax] = self[ax]
        else:
            idx = list(ax)
            idx[dim] = (d - s) // step
            out[ax] = src[tuple(idx)]
    return out


def unsqueeze(src, dim):
    if dim < 0:
        dim += src.ndim + 1
    out_shape = src.shape[:dim] + (1,) + src.shape[dim:]
    out = np.empty(out_shape, src.dtype)
    for ax in _coords(out_shape):
        out[ax] = src[ax[:dim] + ax[dim + 1:]]
    return out


def view(src, shape):
    shape = list(shape)
    if -1 in shape:
        known = int(np.prod([s for s in shape if s != -1]))
        shape[shape.index(-1)] = src.size // known
    out = np.empty(shape, src.dtype)
    ostr = [int(np.prod(shape[i + 1:])) for i in range(len(shape))]
    for ax in _coords(shape):
        flat = sum(a * s for a, s in zip(ax, ostr))
        idx, stride = [0] * src.ndim, 1
        for k in range(src.ndim - 1, -1, -1):
            idx[k] = (flat // stride) % src.shape[k] if k > 0 else flat // stride
            stride *= src.shape[k]
        out[ax] = src[tuple(idx)]
    return out


def permute(src, dims):
    dims = [d % src.ndim for d in dims]
    out_shape = tuple(src.shape[d] for d in dims)
    out = np.empty(out_shape, src.dtype)
    for ax in _coords(out_shape):
        new_axes = [0] * src.ndim
        for i, d in enumerate(dims):
            new_axes[d] = ax[i]
        out[ax] = src[tuple(new_axes)]
    return out


def expand(src, sizes):
    off = len(sizes) - src.ndim
    out_shape = tuple(src.shape[i - off] if (s == -1 and i >= off) else s for i, s in enumerate(sizes))
    out = np.empty(out_shape, src.dtype)
    for ax in _coords(out_shape):
        idx = tuple(0 if src.shape[i] == 1 else ax[i + off] for i in range(src.ndim))
        out[ax] = src[idx]
    return out


def repeat(src, repeats):
    repeats = [1] * max(src.ndim - len(repeats), 0) + list(repeats)
    off = len(repeats) - src.ndim
    out_shape = tuple(r * (src.shape[i - off] if i >= off else 1) for i, r in enumerate(repeats))
    out = np.empty(out_shape, src.dtype)
    for ax in _coords(out_shape):
        idx = tuple(ax[i + off] % src.shape[i] for i in range(src.ndim))
        out[ax] = src[idx]
    return out


def index(src, idx):
    out_shape = idx.shape + src.shape[1:]
    out = np.empty(out_shape, src.dtype)
    r = idx.ndim
    for ax in _coords(out_shape):
        out[ax] = src[(int(idx[ax[:r]]),) + ax[r:]]
    return out


def cat(tensors, dim):
    dim %= tensors[0].ndim
    bounds = np.cumsum([0] + [t.shape[dim] for t in tensors])
    out_shape = list(tensors[0].shape)
    out_shape[dim] = int(bounds[-1])
    out = np.empty(out_shape, tensors[0].dtype)
    for ax in _coords(out_shape):
        for i, t in enumerate(tensors):
            if ax[dim] < bounds[i + 1]:
                idx = list(ax)
                idx[dim] = ax[dim] - int(bounds[i])
                out[ax] = t[tuple(idx)]
                break
    return out


def stack(tensors, dim):
    if dim < 0:
        dim += tensors[0].ndim + 1
    out_shape = tensors[0].shape[:dim] + (len(tensors),) + tensors[0].shape[dim:]
    out = np.empty(out_shape, tensors[0].dtype)
    for ax in _coords(out_shape):
        out[ax] = tensors[ax[dim]][ax[:dim] + ax[dim + 1:]]
    return out


def triu(src, diagonal):
    out = np.empty(src.shape, src.dtype)
    for ax in _coords(src.shape):
        out[ax] = src[ax] if (ax[-1] - ax[-2]) >= diagonal else 0
    return out


def compact(mask, cols):
    """x[mask] for each x: kept rows in ascending source order."""
    kept = [i for i in range(len(mask)) if mask[i]]
    return [np.stack([c[i] for i in kept]) if kept else c[:0] for c in cols]
