"""The reference's extension module name (kernels/selective_nd_scan/setup.py:80,
`selective_nd_scan_cuda_oflex`) on MI355X: code written for the reference does
`import selective_nd_scan_cuda_oflex` and calls `.fwd(...)` / `.bwd(...)` with the positional lists of
selective_scan_oflex.cpp:179-187,286-297.  This module is the gfx950 extension under that name; there is
no CUDA anywhere behind it."""
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
if _HERE not in sys.path:
    sys.path.insert(0, _HERE)
import torch  # noqa: E402,F401  (libtorch must be loaded before the extension)

try:
    from selective_nd_scan_hip_oflex import bwd, fwd, init, set_debug, set_schedule  # noqa: E402,F401
except ImportError as e:  # no fallback: a missing build must not look like a working GPU path
    raise ImportError("selective_nd_scan_hip_oflex is not built; run `python %s`" % os.path.join(_HERE, "build.py")) from e

__all__ = ["fwd", "bwd", "set_schedule", "set_debug", "init"]
