"""MI355X (gfx950) execution backend for FuncTs/FAIT fused functionalized regions."""
from .region import Region, Val, BoundCall, compact_rows  # noqa: F401

# kernels that an earlier process compiled at run time (functs_amd.aot.compile_missing)
try:
    from . import aot as _aot
    _aot.load_cached_kernels()
except Exception:   # a cache that cannot be read is no reason not to import
    pass
