"""MI355X (gfx950) execution backend for FuncTs/FAIT fused functionalized regions."""
from .region import Region, Val, BoundCall, compact_rows  # noqa: F401
