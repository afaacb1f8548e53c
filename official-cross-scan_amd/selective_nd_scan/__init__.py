"""selective_nd_scan for AMD MI355X (gfx950): the 2D-CrossScan selective scan, forward + backward."""
from .interface import (SelectiveNdScanFn, SelectiveNdScanMergedFn, bwd, fwd, init, selective_nd_scan,  # noqa: F401
                        selective_nd_scan_merged, get_schedule, set_debug, set_schedule)

__all__ = ["selective_nd_scan", "selective_nd_scan_merged", "SelectiveNdScanFn", "SelectiveNdScanMergedFn", "fwd", "bwd",
           "set_schedule", "get_schedule", "set_debug", "init"]
from .cross_scan import (cross_merge, cross_scan, cross_scan_2d, four_corner_scan,  # noqa: F401,E402
                         four_corner_scan_by_flips)

__all__ += ["cross_scan", "cross_merge", "cross_scan_2d", "four_corner_scan", "four_corner_scan_by_flips"]
from .vss_block import SS2DCrossScan, VSSBlock  # noqa: F401,E402

__all__ += ["SS2DCrossScan", "VSSBlock"]
