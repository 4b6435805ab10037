"""ctypes binding of libfxhip.so (the C ABI declared in include/fxhip.h).

The library is built in-tree by ``__graft_entry__.build()`` (or ``make`` in
``functs_amd/csrc/fxhip``).  There is no fallback: if the shared object is
missing, importing this module raises.
"""
import ctypes
import os
import re

# torch ships its own HIP runtime; import it first so that libfxhip binds to
# the same libamdhip64 instance (streams and pointers are shared with torch).
import torch  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfxhip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "fxhip.h")

FX_ARG_MAX_RANK = 8


class FxArg(ctypes.Structure):
    _fields_ = [
        ("kind", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("ptr", ctypes.c_void_p),
        ("rank", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("sizes", ctypes.c_int64 * FX_ARG_MAX_RANK),
        ("strides", ctypes.c_int64 * FX_ARG_MAX_RANK),
        ("ival", ctypes.c_int64),
        ("fval", ctypes.c_double),
    ]


class FxNmsDesc(ctypes.Structure):
    """fx_nms_desc of include/fxhip.h."""
    _fields_ = [
        ("mode", ctypes.c_int32),
        ("n_tasks", ctypes.c_int32),
        ("rows", ctypes.c_uint32),
        ("n_classes", ctypes.c_uint32),
        ("boxes", ctypes.c_void_p),
        ("boxes_task_stride", ctypes.c_int64),
        ("scores", ctypes.c_void_p),
        ("scores_task_stride", ctypes.c_int64),
        ("scores_row_stride", ctypes.c_uint32),
        ("reserved0", ctypes.c_uint32),
        ("factors", ctypes.c_void_p),
        ("factors_task_stride", ctypes.c_int64),
        ("labels", ctypes.c_void_p),
        ("labels_task_stride", ctypes.c_int64),
        ("counts", ctypes.c_void_p),
        ("score_thr", ctypes.c_float),
        ("iou_thr", ctypes.c_float),
        ("max_num", ctypes.c_uint32),
        ("key_capacity", ctypes.c_uint32),
        ("dets", ctypes.c_void_p),
        ("out_labels", ctypes.c_void_p),
        ("out_index", ctypes.c_void_p),
        ("n_out", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
    ]


def _parse_header():
    """Opcode / dtype / error constants straight from the C header, so that the
    Python side can never drift from the ABI."""
    text = open(HEADER_PATH).read()
    consts = {}
    for m in re.finditer(r"#define\s+(FX_[A-Z0-9_]+)\s+\(?(-?\d+)\)?", text):
        consts[m.group(1)] = int(m.group(2))
    body = re.search(r"enum fx_opcode \{(.*?)\};", text, re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    val = 0
    for tok in body.split(","):
        tok = tok.strip()
        if not tok:
            continue
        if "=" in tok:
            name, v = [t.strip() for t in tok.split("=")]
            val = int(v)
        else:
            name = tok
        consts[name] = val
        val += 1
    return consts


C = _parse_header()


def exported_symbols():
    """Names of every function the header declares."""
    text = open(HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fx_[a-z0-9_]+)\s*\(", text)))


if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libfxhip.so is not built (%s). Run `python -c 'import __graft_entry__ as g; g.build()'` "
        "or `make -C functs_amd/csrc/fxhip`." % LIB_PATH
    )

lib = ctypes.CDLL(LIB_PATH)

_vp = ctypes.c_void_p
_i = ctypes.c_int
_ip = ctypes.POINTER(ctypes.c_int)


def _sig(name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_sig("fx_last_error", ctypes.c_char_p)
_sig("fx_api_version", _i)
_sig("fx_region_create", _i, _i, _i, ctypes.POINTER(_vp))
_sig("fx_region_destroy", None, _vp)
_sig("fx_region_input_tensor", _i, _vp, _i, _i, _i, _ip)
_sig("fx_region_input_scalar", _i, _vp, _i, _i, _ip)
_sig("fx_region_task_index", _i, _vp, _ip)
_sig("fx_region_loop_var", _i, _vp, _ip)
_sig("fx_region_const_int", _i, _vp, ctypes.c_int64, _ip)
_sig("fx_region_const_float", _i, _vp, ctypes.c_double, _ip)
_sig("fx_region_const_bool", _i, _vp, _i, _ip)
_sig("fx_region_const_none", _i, _vp, _ip)
_sig("fx_region_int_list", _i, _vp, _ip, _i, _ip)
_sig("fx_region_tensor_list", _i, _vp, _ip, _i, _ip)
_sig("fx_region_op", _i, _vp, _i, _ip, _i, _i, _ip)
_sig("fx_region_output", _i, _vp, _i)
_sig("fx_region_compact_rows", _i, _vp, _i)
_sig("fx_region_finalize", _i, _vp)
_sig("fx_region_plan", _i, _vp, ctypes.POINTER(FxArg), _i, ctypes.POINTER(_vp))
_sig("fx_plan_num_outputs", _i, _vp)
_sig("fx_plan_output", _i, _vp, _i, _i, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32),
     ctypes.POINTER(ctypes.c_int64))
_sig("fx_plan_scratch_bytes", ctypes.c_size_t, _vp)
_sig("fx_plan_launches", _i, _vp)
_sig("fx_plan_streaming", _i, _vp)
_sig("fx_plan_stream_info", _i, _vp, ctypes.POINTER(ctypes.c_int64), _i)
_sig("fx_set_streaming", None, _i)
_sig("fx_set_stream_spin_limit", None, ctypes.c_uint32)
_sig("fx_plan_algorithmic_bytes", ctypes.c_int64, _vp)
_sig("fx_plan_blob", _i, _vp, ctypes.POINTER(ctypes.POINTER(ctypes.c_uint32)), ctypes.POINTER(ctypes.c_size_t))
_sig("fx_plan_disasm", _i, _vp, ctypes.c_char_p, ctypes.c_size_t)
_sig("fx_plan_head_info", _i, _vp, ctypes.POINTER(ctypes.c_int64), _i)
_sig("fx_set_head_kernel", None, _i)
_sig("fx_plan_rowstream_info", _i, _vp, ctypes.POINTER(ctypes.c_int64), _i)
_sig("fx_plan_rowstream_why", _i, _vp, ctypes.c_char_p, ctypes.c_size_t)
_sig("fx_plan_rowstream_source", _i, _vp, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t)
_sig("fx_set_rowstream", None, _i)
_sig("fx_plan_rowstream_launch", _i, _vp, ctypes.c_uint32, ctypes.c_uint32, _vp, ctypes.c_size_t)
_sig("fx_rowstream_count", _i)
_sig("fx_plan_spec_key", ctypes.c_uint64, _vp)
_sig("fx_plan_specialized", _i, _vp)
_sig("fx_plan_spec_source", _i, _vp, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t)
_sig("fx_set_specialization", None, _i)
_sig("fx_specialization_count", _i)
_sig("fx_plan_dense_lean", _i, _vp)
_sig("fx_set_dense_lean", None, _i)
_sig("fx_spec_dump_dir", _i, ctypes.c_char_p)
_sig("fx_spec_dump_what", _i, _i)
_sig("fx_region_wait_totals", _i, _vp, _vp, _vp)
_sig("fx_region_poll_totals", _i, _vp, _vp, ctypes.c_uint32)
_sig("fx_launch_stats", None, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64))
_sig("fx_region_marshal", _i, _vp, _vp, ctypes.POINTER(FxArg), _i, ctypes.POINTER(_vp), _vp, _vp, _vp,
     ctypes.c_size_t)
_sig("fx_dyn_bytes", ctypes.c_size_t)
_sig("fx_plan_table_sizes", _i, _vp, ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(_i))
_sig("fx_region_marshal_tables", _i, _vp, _vp, ctypes.POINTER(FxArg), _i, ctypes.POINTER(_vp), _vp, _vp,
     ctypes.POINTER(ctypes.c_uint64), ctypes.c_size_t, ctypes.POINTER(ctypes.c_uint32), ctypes.c_size_t)
_sig("fx_region_run", _i, _vp, _vp, ctypes.POINTER(FxArg), _i, ctypes.POINTER(_vp), _vp, _vp, _vp)
_sig("fx_region_run_timed", _i, _vp, _vp, ctypes.POINTER(FxArg), _i, ctypes.POINTER(_vp), _vp, _vp, _vp,
     ctypes.POINTER(ctypes.c_float), _i, _ip)
_sig("fx_region_run_timed_batched", _i, _vp, _vp, ctypes.POINTER(FxArg), _i, ctypes.POINTER(_vp), _vp, _vp, _vp, _i,
     ctypes.POINTER(ctypes.c_float), _i, _ip)
_sig("fx_region_run_timed_sets", _i, _vp, _vp, _i, ctypes.POINTER(ctypes.POINTER(FxArg)), _i,
     ctypes.POINTER(ctypes.POINTER(_vp)), ctypes.POINTER(_vp), ctypes.POINTER(_vp), _vp, _i, _i,
     ctypes.POINTER(ctypes.c_float))
_sig("fx_compact_rows", _i, _vp, ctypes.c_int64, ctypes.POINTER(_vp), ctypes.POINTER(_vp),
     ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32), _i, _vp, ctypes.c_size_t, _vp, _vp)
_sig("fx_compact_rows_scratch_bytes", ctypes.c_size_t, ctypes.c_int64)
_sig("fx_compact_rows_static", _i, _vp, ctypes.c_int64, ctypes.POINTER(_vp), ctypes.POINTER(_vp),
     ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32), _i, _vp, _vp)
_sig("fx_async_error", _i, _i)
_sig("fx_async_error_take", _i, _i)
_sig("fx_async_error_report", None, _i)
_fp = ctypes.c_void_p
_sig("fx_sort_nms", ctypes.c_int, ctypes.POINTER(FxNmsDesc), ctypes.c_void_p)
_sig("fx_sort_nms_workspace_bytes", ctypes.c_size_t, ctypes.c_int, ctypes.c_uint32)
_sig("fx_sort_nms_workspace_clear_bytes", ctypes.c_size_t, ctypes.c_int)
_sig("fx_lstm_stack_fits", ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int)
_sig("fx_lstm_stack_workspace_bytes", ctypes.c_size_t, _i, _i, _i)
_sig("fx_lstm_stack", _i, _fp, _fp, _fp, _fp, _fp, _fp, _fp, _fp, _fp, _fp, _i, _i, _i, _i, _vp, ctypes.c_size_t, _vp)
_sig("fx_set_lstm_spin_limit", None, ctypes.c_uint32)
_sig("fx_set_totals_spin_us", None, ctypes.c_uint32)
_sig("fx_device_count", _i)
_sig("fx_copy_bytes", _i, _vp, _vp, ctypes.c_size_t, _vp)
_sig("fx_copy_bytes_timed_sets", _i, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p), _i, ctypes.c_size_t, _i, _vp,
     ctypes.POINTER(ctypes.c_float))


class FxError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("fxhip error %d: %s" % (code, msg))
        self.code = code


def check(rc):
    if rc < 0:
        raise FxError(rc, lib.fx_last_error().decode())
    return rc


def copy_bytes_timed_sets(pairs, rounds, stream=None):
    """Mean milliseconds per launch of the copy kernel over `rounds` passes through the (src, dst)
    pairs, launched back to back by the library (fx_copy_bytes_timed_sets)."""
    import torch
    nbytes = pairs[0][0].numel() * pairs[0][0].element_size()
    assert all(a.is_cuda and b.is_cuda and a.numel() * a.element_size() == nbytes == b.numel() * b.element_size() for a, b in pairs)
    src = (ctypes.c_void_p * len(pairs))(*[a.data_ptr() for a, _ in pairs])
    dst = (ctypes.c_void_p * len(pairs))(*[b.data_ptr() for _, b in pairs])
    st = torch.cuda.current_stream(pairs[0][0].device).cuda_stream if stream is None else stream
    ms = ctypes.c_float()
    check(lib.fx_copy_bytes_timed_sets(src, dst, len(pairs), nbytes, rounds, st, ctypes.byref(ms)))
    return float(ms.value)


def copy_bytes(src, dst, stream=None):
    """dst[:] = src with the library's plain 128-bit copy kernel (the known-size
    dispatch that hardware-counter readings are calibrated against)."""
    import torch
    assert src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()
    nbytes = src.numel() * src.element_size()
    assert nbytes == dst.numel() * dst.element_size()
    st = torch.cuda.current_stream(src.device).cuda_stream if stream is None else stream
    check(lib.fx_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes, st))
