"""Import names of the reference package (functs/__init__.py:1-2): ``functs``, ``functs.jit``,
``functs._C`` and ``functs.utils.prof`` resolve to the MI355X backend ``functs_amd``, so that a
script written against the reference (``import functs._C`` ...
``functs._C._jit_pass_rewrite_mutation(graph, info)``, ``functs.jit.script(fn)``,
``functs.jit.build(fn, example)``) runs unchanged."""
import sys as _sys
import types as _types

import functs_amd as _backend
import functs_amd._C as _C
import functs_amd.jit as jit
import functs_amd.prof as _prof

utils = _types.ModuleType(__name__ + ".utils")
utils.__doc__ = "functs.utils of the reference: the profiling harness (functs/utils/prof.py)."
utils.prof = _prof
_sys.modules[__name__ + "._C"] = _C
_sys.modules[__name__ + ".jit"] = jit
_sys.modules[__name__ + ".utils"] = utils
_sys.modules[__name__ + ".utils.prof"] = _prof

Region = _backend.Region
compact_rows = _backend.compact_rows
