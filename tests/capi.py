"""The tests drive the C ABI through the package's ctypes binding."""
from selective_nd_scan.capi import *  # noqa: F401,F403
from selective_nd_scan.capi import (BwdParams, FwdParams, Plan, Shape, bwd, check, declared_symbols, fwd, lib,  # noqa: F401
                                    make_plan, make_shape)
