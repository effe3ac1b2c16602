"""polygrad_amd: MI355X (gfx950) device backend for polygrad.

The product is the C-ABI library polygrad_amd/lib/libpolygrad_hip.so (sources
in polygrad_amd/csrc, interface in include/polygrad_hip.h).  This package is the
thin Python host side: a ctypes binding and plan-level helpers.
"""
from . import _ffi
from .plan import HipPlan, PlanFile, save_schedule

__all__ = ["_ffi", "HipPlan", "PlanFile", "save_schedule"]
