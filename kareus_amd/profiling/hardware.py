"""Time and energy of a repeated target function, and the sweep bookkeeping around it.

The measuring loop has the shape of the reference's
(tests/bayesian/common/hardware.py:76-137: per task set the clock, then
``zeus_measure(target_fn, measurement_duration=5 s, cooldown_duration=5 s)`` ->
``(energy_per_iter, time_per_iter)``) and the records are the reference's eval-log rows
(tests/bayesian/common/orchestration.py:65-147: one JSON object per line with ``freq,
overlap_start, overlap_end, sm, block, time_s, energy_j``; re-reading keeps the first row per
``(freq, overlap_start, overlap_end, sm)``).

Power comes from ``kareus_amd.energy.PowerSampler``.  Clock control writes the amdgpu sysfs
performance-level files; an ordinary user may not, in which case ``set_gpu_frequency`` returns
False and rows carry the requested value with ``freq_applied: false``.
"""

from __future__ import annotations

import json
import os
import time
from dataclasses import dataclass
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

from ..energy import PowerSampler, sysfs_device_dir


@dataclass(frozen=True)
class Trial:
    iterations: int
    time_per_iter: float            # seconds
    energy_per_iter: Optional[float]  # joules; None when no power source is readable
    mean_watts: Optional[float]


def _device_sync() -> None:
    import torch

    if torch.cuda.is_available():
        torch.cuda.synchronize()


def measure(
    target_function: Callable[[], object],
    sampler: Optional[PowerSampler] = None,
    measurement_duration: float = 5.0,
    cooldown_duration: float = 5.0,
    warmup_iterations: int = 3,
    sync: Callable[[], None] = _device_sync,
    clock: Callable[[], float] = time.perf_counter,
    sleep: Callable[[float], None] = time.sleep,
    batch: int = 8,
) -> Trial:
    """Cool down, warm up, then call ``target_function`` back to back until
    ``measurement_duration`` seconds have passed (device synchronised every ``batch`` calls and
    at both ends) while the sampler integrates board power over exactly that window."""
    if cooldown_duration > 0:
        sleep(cooldown_duration)
    for _ in range(warmup_iterations):
        target_function()
    sync()
    if sampler is not None:
        sampler.start()
    t0 = clock()
    iterations = 0
    while True:
        for _ in range(batch):
            target_function()
        iterations += batch
        sync()
        t1 = clock()
        if t1 - t0 >= measurement_duration:
            break
    energy = watts = None
    if sampler is not None:
        sampler.stop()
        if sampler.available:
            energy = sampler.energy_joules(t0, t1)
            watts = None if energy is None else energy / (t1 - t0)
    return Trial(
        iterations=iterations,
        time_per_iter=(t1 - t0) / iterations,
        energy_per_iter=None if energy is None else energy / iterations,
        mean_watts=watts,
    )


# ---- clock control (best effort) -------------------------------------------------------------
def _device_dir(device_index: int) -> Optional[str]:
    """sysfs directory of the HIP device, found by its PCI bus id; None (no clock is touched)
    when it cannot be matched."""
    d = sysfs_device_dir(device_index)
    return d if d is not None and os.path.exists(os.path.join(d, "pp_dpm_sclk")) else None


def available_frequencies_mhz(device_index: int = 0) -> List[int]:
    """Shader-clock levels the driver lists (``pp_dpm_sclk`` lines ``"<n>: <MHz>Mhz [*]"``)."""
    d = _device_dir(device_index)
    if d is None:
        return []
    out = []
    try:
        with open(os.path.join(d, "pp_dpm_sclk")) as f:
            for line in f:
                parts = line.split()
                # "<level>: <MHz>Mhz [*]"; a line "S: <MHz>Mhz *" is the clock in force, not a level
                if len(parts) >= 2 and parts[0][:-1].isdigit() and parts[1].lower().endswith("mhz"):
                    out.append(int(float(parts[1][:-3])))
    except OSError:
        return []
    return out


def nominal_frequency_mhz(device_index: int = 0) -> int:
    """The clock a sweep records when it leaves the clock alone: the device's rated shader clock
    (the same number on every run and box), else the highest listed level, else 0.  The listed
    levels are no stable label: the driver shows the clock in force as a level of its own, so
    their maximum moves by a few MHz between reads."""
    try:
        import torch

        if torch.cuda.is_available():
            from ..backend.hip import load_library

            with torch.cuda.device(device_index):
                mhz = int(load_library().kr_device_clock_mhz())
            if mhz > 0:
                return mhz
    except (ImportError, OSError, RuntimeError, AttributeError):
        pass
    return max(available_frequencies_mhz(device_index) or [0])


def set_gpu_frequency(target_freq_mhz: int, device_index: int = 0, settle_s: float = 0.5) -> bool:
    """Pin the shader clock to the listed level closest to ``target_freq_mhz``.  Returns False
    (and changes nothing) when the files are missing or not writable by this user.  ``settle_s``:
    pause after the write (a measurement wants the clock settled, a per-instruction switch in
    a training loop passes 0)."""
    d = _device_dir(device_index)
    levels = available_frequencies_mhz(device_index)
    if d is None or not levels:
        return False
    level = min(range(len(levels)), key=lambda i: abs(levels[i] - target_freq_mhz))
    try:
        with open(os.path.join(d, "power_dpm_force_performance_level"), "w") as f:
            f.write("manual")
    except OSError:
        return False
    try:
        with open(os.path.join(d, "pp_dpm_sclk"), "w") as f:
            f.write(str(level))
    except OSError:
        reset_gpu_clocks(device_index)  # do not leave the card in manual mode without a level
        return False
    if settle_s > 0:
        time.sleep(settle_s)
    return True


def reset_gpu_clocks(device_index: int = 0) -> bool:
    d = _device_dir(device_index)
    if d is None:
        return False
    try:
        with open(os.path.join(d, "power_dpm_force_performance_level"), "w") as f:
            f.write("auto")
    except OSError:
        return False
    return True


# ---- sweeps ------------------------------------------------------------------------------------
BLOCK_SIZE = 1024  # tests/bayesian/common/encoding.py:13


def all_configurations(freq_values: Sequence[int], sm_values: Sequence[int],
                       overlap_windows: Sequence[Tuple]) -> List[Dict]:
    """Full grid in the reference's order: frequency, then SM count, then overlap window
    (tests/bayesian/common/encoding.py:60-69)."""
    return [
        {"freq": f, "sm": sm, "block": BLOCK_SIZE, "overlap": tuple(w)}
        for f in freq_values for sm in sm_values for w in overlap_windows
    ]


def build_eval_record(cfg: Dict, time_s: float, energy_j: Optional[float],
                      freq_applied: Optional[bool] = None) -> Dict:
    rec = {
        "freq": int(cfg["freq"]),
        "overlap_start": cfg["overlap"][0],
        "overlap_end": cfg["overlap"][1],
        "sm": int(cfg["sm"]),
        "block": int(cfg["block"]),
        "time_s": time_s,
        "energy_j": energy_j,
    }
    if freq_applied is not None:
        rec["freq_applied"] = bool(freq_applied)
    return rec


def append_eval_log(path: str, records: Iterable[Dict]) -> None:
    with open(path, "a") as f:
        for rec in records:
            f.write(json.dumps(rec) + "\n")


def load_eval_log(path: str) -> List[Dict]:
    """Rows of a JSONL eval log, first occurrence per configuration; ``[]`` if unreadable."""
    if not os.path.exists(path):
        return []
    try:
        with open(path) as f:
            rows = [json.loads(line) for line in f if line.strip()]
    except (OSError, ValueError):
        return []
    seen, unique = set(), []
    for r in rows:
        key = (int(r["freq"]), r["overlap_start"], r["overlap_end"], int(r["sm"]))
        if key not in seen:
            seen.add(key)
            unique.append(r)
    return unique


def measure_batch(partition_test, configs: Sequence[Dict], sampler: Optional[PowerSampler] = None,
                  measurement_duration: float = 5.0, cooldown_duration: float = 5.0,
                  device_index: int = 0, **measure_kwargs) -> List[Dict]:
    """Evaluate configurations one after another on this GPU; returns eval-log records.
    ``partition_test.test_config(overlap_window, (sm, block))`` is the unit being repeated."""
    records = []
    current_freq = None
    pinned = False
    try:
        for cfg in configs:
            if cfg["freq"] != current_freq:
                pinned = set_gpu_frequency(int(cfg["freq"]), device_index)
                current_freq = cfg["freq"]
            window, shape = tuple(cfg["overlap"]), (int(cfg["sm"]), int(cfg["block"]))
            trial = measure(lambda: partition_test.test_config(window, shape), sampler,
                            measurement_duration, cooldown_duration, **measure_kwargs)
            records.append(build_eval_record(cfg, trial.time_per_iter, trial.energy_per_iter, pinned))
    finally:
        if pinned:
            reset_gpu_clocks(device_index)
    return records
