"""GPU board power sampling -> joules per iteration.

Plays the part of the reference's Zeus measurement window
(tests/bayesian/common/hardware.py:121-132: energy and time of a repeated target
function over a fixed window).  Power is read from the amdgpu hwmon node
(``power1_input`` / ``power1_average``, microwatts) on a background thread and
integrated with the trapezoid rule; if the node is absent the ``amdsmi`` Python
binding is tried.  ``available`` is False when neither source works — callers
then report energy as unmeasured instead of guessing.
"""

from __future__ import annotations

import glob
import threading
import time
from typing import Callable, List, Optional, Tuple


def _sysfs_reader(device_index: int) -> Optional[Callable[[], float]]:
    for name in ("power1_input", "power1_average"):
        paths = sorted(glob.glob(f"/sys/class/drm/card*/device/hwmon/hwmon*/{name}"))
        if len(paths) > device_index:
            path = paths[device_index]

            def read(path=path) -> float:
                with open(path) as f:
                    return int(f.read().strip()) * 1e-6

            try:
                read()
                return read
            except (OSError, ValueError):
                continue
    return None


def _amdsmi_reader(device_index: int) -> Optional[Callable[[], float]]:
    try:
        import amdsmi  # type: ignore

        amdsmi.amdsmi_init()
        handle = amdsmi.amdsmi_get_processor_handles()[device_index]

        def read() -> float:
            info = amdsmi.amdsmi_get_power_info(handle)
            for key in ("socket_power", "current_socket_power", "average_socket_power"):
                val = info.get(key)
                if isinstance(val, (int, float)) and val > 0:
                    return float(val)
            raise RuntimeError("no power field")

        read()
        return read
    except Exception:
        return None


class PowerSampler:
    def __init__(self, device_index: int = 0, hz: float = 100.0) -> None:
        self._read = _sysfs_reader(device_index) or _amdsmi_reader(device_index)
        self.available = self._read is not None
        self.period = 1.0 / hz
        self.samples: List[Tuple[float, float]] = []
        self._stop = threading.Event()
        self._thread: Optional[threading.Thread] = None

    def _loop(self) -> None:
        while not self._stop.is_set():
            try:
                self.samples.append((time.perf_counter(), self._read()))
            except Exception:
                pass
            self._stop.wait(self.period)

    def start(self) -> None:
        if not self.available:
            return
        self.samples = []
        self._stop.clear()
        self._thread = threading.Thread(target=self._loop, daemon=True)
        self._thread.start()

    def stop(self) -> None:
        if self._thread is not None:
            self._stop.set()
            self._thread.join()
            self._thread = None

    def energy_joules(self, t0: float, t1: float) -> Optional[float]:
        """Trapezoid integral of the samples over [t0, t1] (perf_counter seconds)."""
        pts = [(t, p) for t, p in self.samples if t0 <= t <= t1]
        if len(pts) < 2:
            return None
        joules = sum(0.5 * (pa + pb) * (tb - ta) for (ta, pa), (tb, pb) in zip(pts, pts[1:]))
        # extend the first/last sample to the window edges
        joules += pts[0][1] * (pts[0][0] - t0) + pts[-1][1] * (t1 - pts[-1][0])
        return joules

    def mean_watts(self, t0: float, t1: float) -> Optional[float]:
        e = self.energy_joules(t0, t1)
        return None if e is None else e / (t1 - t0)
