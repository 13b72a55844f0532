"""recsdk_amd -- MI355X (gfx950) implementation of RecSDK's HSTU fused attention forward.

Importing the package loads the two shared libraries built by ``recsdk_amd._build``:

* ``lib/libhstu_hip.so``       C ABI (``include/hstu_hip.h``) + hand-written HIP kernels
* ``lib/libmxrec_hstu_ops.so`` registers ``torch.ops.mxrec.hstu_jagged`` (``.equal`` / ``.delta``),
  ``hstu_paged``, ``hstu_dense`` with the reference's schemas, plus ``hstu_jagged_table_bias`` and
  ``hstu_paged_fp8``

The loading convention is the reference's own: one ``torch.ops.load_library`` call
(cust_op/rec_cust_ops/__init__.py:134-183).  There is no fallback implementation: if a library is
missing the import fails.
"""
from __future__ import annotations

import os

import torch

from . import _build, _capi
from ._capi import HstuError  # noqa: F401

__all__ = ["load", "ops_library_path", "hip_library_path", "time_bucket_bounds", "HstuError"]

_loaded = False


def hip_library_path() -> str:
    return _build.hip_lib_path()


def ops_library_path() -> str:
    return _build.ops_lib_path()


def load() -> None:
    """Load both libraries (idempotent).  Raises if either is missing."""
    global _loaded
    if _loaded:
        return
    _capi.lib()
    path = ops_library_path()
    if not os.path.exists(path):
        raise HstuError(f"{path} is missing: build it with `python -m recsdk_amd._build`")
    torch.ops.load_library(path)
    _loaded = True


def time_bucket_bounds(num_buckets: int = 128, bucket_divisor: float = 0.301) -> torch.Tensor:
    """fp32 lower bound of every time bucket (``[num_buckets + 2]``, CPU): the ``ts_bounds`` argument of the C ABI."""
    load()
    return torch.ops.mxrec.hstu_time_bucket_bounds(num_buckets, bucket_divisor)


load()
