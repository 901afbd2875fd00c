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
import os
import threading
import time
from typing import Callable, List, Optional, Tuple


def pci_bus_id(device_index: int = 0) -> Optional[str]:
    """``dddd:bb:dd.f`` of the HIP device with this index (the index already reflects
    HIP_VISIBLE_DEVICES / ROCR_VISIBLE_DEVICES), or None without a device."""
    try:
        import torch

        if not torch.cuda.is_available() or device_index >= torch.cuda.device_count():
            return None
        p = torch.cuda.get_device_properties(device_index)
        return f"{p.pci_domain_id:04x}:{p.pci_bus_id:02x}:{p.pci_device_id:02x}.0"
    except Exception:
        return None


def _card_number(path: str) -> int:
    digits = "".join(ch for ch in os.path.basename(path) if ch.isdigit())
    return int(digits) if digits else -1


def sysfs_device_dir(device_index: int = 0, sysfs_root: str = "/sys",
                     bus_id: Optional[str] = None) -> Optional[str]:
    """The amdgpu sysfs directory of the HIP device: ``/sys/bus/pci/devices/<bus id>`` or the
    ``/sys/class/drm/card*/device`` link that resolves to that bus id.  None when the device's bus
    id is unknown or no node matches it: the position of a card in a directory listing says
    nothing about which GPU this process was given, so it is never used to pick one."""
    bdf = bus_id if bus_id is not None else pci_bus_id(device_index)
    if bdf is None:
        return None
    direct = os.path.join(sysfs_root, "bus", "pci", "devices", bdf)
    if os.path.isdir(direct):
        return direct
    cards = glob.glob(os.path.join(sysfs_root, "class", "drm", "card[0-9]*", "device"))
    for dev in sorted(cards, key=lambda d: _card_number(os.path.dirname(d))):
        if os.path.basename(os.path.realpath(dev)) == bdf:
            return dev
    return None


def _sysfs_reader(device_index: int) -> Optional[Callable[[], float]]:
    dev = sysfs_device_dir(device_index)
    if dev is None:
        return None
    for name in ("power1_input", "power1_average"):
        for path in sorted(glob.glob(os.path.join(dev, "hwmon", "hwmon*", name))):

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
        bdf = pci_bus_id(device_index)
        handle = next((h for h in amdsmi.amdsmi_get_processor_handles()
                       if str(amdsmi.amdsmi_get_gpu_device_bdf(h)).lower() == bdf), None)
        if bdf is None or handle is None:
            return None

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
        self.bus_id = pci_bus_id(device_index)  # which GPU the readings belong to
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


class ClockReader:
    """Shader clock of the device sampled on a thread; ``values`` are MHz.  Sources, in order:
    hwmon ``freq1_input`` (Hz), else the starred line of ``pp_dpm_sclk`` (``"S: 1714Mhz *"`` is
    the clock in force when the driver lists a range instead of levels)."""

    def __init__(self, device_index: int = 0, hz: float = 100.0) -> None:
        dev = sysfs_device_dir(device_index)
        paths = sorted(glob.glob(os.path.join(dev, "hwmon", "hwmon*", "freq1_input"))) if dev else []
        self._hwmon = paths[0] if paths else None
        dpm = os.path.join(dev, "pp_dpm_sclk") if dev else None
        self._dpm = dpm if (self._hwmon is None and dpm and os.path.exists(dpm)) else None
        self.available = self._hwmon is not None or self._dpm is not None
        self.period = 1.0 / hz
        self.samples: List[Tuple[float, float]] = []
        self._stop = threading.Event()
        self._thread: Optional[threading.Thread] = None

    def read_mhz(self) -> Optional[float]:
        try:
            if self._hwmon is not None:
                with open(self._hwmon) as f:
                    return int(f.read().strip()) * 1e-6
            with open(self._dpm) as f:
                for line in f:
                    if line.rstrip().endswith("*"):
                        return parse_dpm_mhz(line)
        except (OSError, ValueError):
            pass
        return None

    def _loop(self) -> None:
        while not self._stop.is_set():
            mhz = self.read_mhz()
            if mhz is not None:
                self.samples.append((time.perf_counter(), mhz))
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

    def values(self, t0: float, t1: float) -> List[float]:
        return [v for t, v in self.samples if t0 <= t <= t1]


def parse_dpm_mhz(line: str) -> Optional[float]:
    """``"1: 2400Mhz *"`` or ``"S: 1714Mhz *"`` -> MHz."""
    for tok in line.replace("*", " ").split():
        low = tok.lower()
        if low.endswith("mhz"):
            try:
                return float(low[:-3])
            except ValueError:
                return None
    return None
