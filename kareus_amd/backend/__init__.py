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
