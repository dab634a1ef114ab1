"""MI355X (gfx950) build of Accel-GCN's SpMM hot path: degree-sorted,
block-partitioned fp32 CSR x dense, behind the upstream operator interface.

The directory name is not a Python identifier; load it with
``__graft_entry__.load_package()`` (registers it as ``iccad_accel_gcn_amd``).
"""
from ._lib import AccelError, DeviceBuffer, device_count, lib  # noqa: F401
from .spmm import AccelSpMM, SpmmAccel  # noqa: F401
from .dense import GcnLayer, dense_xw, dense_xw_numpy  # noqa: F401
from . import block_level_partition, synthetic  # noqa: F401

__all__ = ["AccelError", "AccelSpMM", "DeviceBuffer", "GcnLayer", "SpmmAccel", "block_level_partition",
           "dense_xw", "dense_xw_numpy", "device_count", "lib", "synthetic"]
