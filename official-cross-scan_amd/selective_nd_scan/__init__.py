"""selective_nd_scan for AMD MI355X (gfx950): the 2D-CrossScan selective scan, forward + backward."""
from .interface import SelectiveNdScanFn, bwd, fwd, selective_nd_scan, set_schedule  # noqa: F401

__all__ = ["selective_nd_scan", "SelectiveNdScanFn", "fwd", "bwd", "set_schedule"]
