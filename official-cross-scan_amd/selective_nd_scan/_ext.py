"""Loads the in-tree PyTorch extension `selective_nd_scan_hip_oflex` (built by ../build.py).

There is no fallback: without the extension the operator raises, so a missing build is never
mistaken for a working GPU path.
"""
import importlib
import os
import sys

_PKG_PARENT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_mod = None


def ext():
    global _mod
    if _mod is None:
        import torch  # noqa: F401  (libtorch must be loaded before the extension)
        if _PKG_PARENT not in sys.path:
            sys.path.insert(0, _PKG_PARENT)
        try:
            _mod = importlib.import_module("selective_nd_scan_hip_oflex")
        except ImportError as e:
            raise ImportError(
                "selective_nd_scan_hip_oflex is not built; run `python %s`"
                % os.path.join(_PKG_PARENT, "build.py")) from e
    return _mod
