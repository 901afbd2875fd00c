"""Kernel backends behind the operators.

``hip``    the product path: hand-written gfx950 kernels in ``libkareus_hip.so``
           reached through its C ABI.  Selecting it without the built library, or
           handing it a tensor that is not bf16 on a HIP device, raises.
``eager``  the same primitive set written with eager PyTorch calls in the tensors'
           own dtype.  It exists for the fp32 host-side plumbing configuration
           (engine, scheduler and stream logic exercised without a GPU) and must be
           asked for by name; nothing selects it implicitly.
"""

from __future__ import annotations

from typing import Dict

_CACHE: Dict[str, object] = {}


def get_backend(name: str = "hip"):
    if name not in ("hip", "eager"):
        raise ValueError(f"unknown backend {name!r}; choose 'hip' or 'eager'")
    if name not in _CACHE:
        if name == "hip":
            from .hip import HipBackend

            _CACHE[name] = HipBackend()
        else:
            from .eager import EagerBackend

            _CACHE[name] = EagerBackend()
    return _CACHE[name]


# ---- compute-unit budget of the launches of the current thread ---------------------------------
# A schedule gives every partition a resource shape (kareus/megatron/core/partitions/
# partition_base.py:117-128: ``sm_num``, the compute units the work overlapping the partition is to
# get).  While a partition runs under such a shape the engine reserves that many units: kernels
# that would otherwise fill the device (the GEMMs, one persistent workgroup per unit) launch on the
# rest.  Thread-local because forward and backward run on different host threads.
import contextlib as _contextlib
import threading as _threading

_budget = _threading.local()


def reserved_compute_units() -> int:
    """Compute units the current partition leaves to the kernels of other nanobatch streams."""
    return getattr(_budget, "reserved", 0)


@_contextlib.contextmanager
def reserve_compute_units(count):
    old = getattr(_budget, "reserved", 0)
    _budget.reserved = max(int(count or 0), 0)
    try:
        yield
    finally:
        _budget.reserved = old
