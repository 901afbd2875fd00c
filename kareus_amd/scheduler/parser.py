"""Reader for the planner's per-instruction schedule files (``scheds_pipeline_*.py``)
and frequency files (``freqs_pipeline_*.py``).

A schedule file is one Python list literal: one inner list per pipeline stage, one
entry per instruction (or per microbatch).  Each partition kind gets a string
``"<start>-<end>-<sm>-<block>"``; start/end are op indices (possibly negative) or
slot names (``norm_0``, ``rope_0``, ..., ``none``).  Grammar and error messages
follow kareus/scheduler/parser.py: config string ``:66-101``, activation-
checkpointing format (``('forward', attn, mlp)`` / ``('backward', rec_attn, rec_mlp,
attn, mlp)``) ``:122-165``, context-parallel formats ``:166-226,275-316``, per-
microbatch pair format ``:228-274``, default trail config ``:30``.

The file is read with ``ast.literal_eval``: the grammar is a pure literal, so
nothing in it needs to be executed.
"""

from __future__ import annotations

import ast
import re
from dataclasses import dataclass
from pathlib import Path
from typing import List, Optional, Sequence, Tuple, Union

__all__ = [
    "CommConfig",
    "ScheduleItem",
    "ScheduleItemCP",
    "MicrobatchPair",
    "OverlapWindow",
    "ResourceShape",
    "parse_schedule_file",
    "parse_frequency_file",
]

OverlapWindow = Tuple[Union[int, str], Union[int, str]]
ResourceShape = Tuple[int, int]


@dataclass(frozen=True)
class CommConfig:
    overlap_window: OverlapWindow
    resource_shape: ResourceShape


_TRAIL_CONFIG = CommConfig(overlap_window=("norm_0", "none"), resource_shape=(20, 1024))


@dataclass(frozen=True)
class ScheduleItem:
    fwd_attn: Optional[CommConfig]
    fwd_mlp: Optional[CommConfig]
    bwd_attn: Optional[CommConfig]
    bwd_mlp: Optional[CommConfig]
    fwd_trail: Optional[CommConfig] = _TRAIL_CONFIG
    bwd_trail: Optional[CommConfig] = _TRAIL_CONFIG


_CP_FWD = ("fwd_qkv_ar", "fwd_qkv_ag", "fwd_ao_ag", "fwd_ao_ar", "fwd_mlp")
_CP_BWD = ("bwd_qkv_ar", "bwd_qkv_rs", "bwd_a_rs", "bwd_a_ag", "bwd_o_ag", "bwd_o_ar", "bwd_mlp")


@dataclass(frozen=True)
class ScheduleItemCP:
    fwd_qkv_ar: Optional[CommConfig]
    fwd_qkv_ag: Optional[CommConfig]
    fwd_ao_ag: Optional[CommConfig]
    fwd_ao_ar: Optional[CommConfig]
    fwd_mlp: Optional[CommConfig]
    bwd_qkv_ar: Optional[CommConfig]
    bwd_qkv_rs: Optional[CommConfig]
    bwd_a_rs: Optional[CommConfig]
    bwd_a_ag: Optional[CommConfig]
    bwd_o_ag: Optional[CommConfig]
    bwd_o_ar: Optional[CommConfig]
    bwd_mlp: Optional[CommConfig]
    fwd_trail: Optional[CommConfig] = _TRAIL_CONFIG
    bwd_trail: Optional[CommConfig] = _TRAIL_CONFIG


MicrobatchPair = Tuple[ScheduleItem, ScheduleItem]

_ALL_INT = re.compile(r"^(-?\d+)-(-?\d+)-(-?\d+)-(-?\d+)$")


def _parse_config_string(cfg: str) -> CommConfig:
    """``"0-8-16-1024"``, ``"-1--1-16-1024"``, ``"norm_0-linear_1-16-1024"``,
    ``"none-none-16-1024"`` -> ``CommConfig``."""
    m = _ALL_INT.match(cfg)
    if m:
        a, b, sm, blk = (int(g) for g in m.groups())
        return CommConfig((a, b), (sm, blk))
    pieces = cfg.rsplit("-", 2)
    if len(pieces) != 3:
        raise ValueError(
            "Config string must have format "
            f"'overlap_start-overlap_end-sm_num-block_size', got: {cfg}"
        )
    window, sm, blk = pieces
    sm_num, block_size = int(sm), int(blk)
    # Slot names are "<group>_<n>": no '-' inside, so the first '-' separates them.
    start, dash, end = window.partition("-")
    if not dash:
        raise ValueError(f"Overlap part must contain 'start-end', got: {window!r}")
    return CommConfig((start, end), (sm_num, block_size))


def _load_literal(path: Union[str, Path]):
    text = Path(path).read_text(encoding="utf-8")
    parsed = ast.literal_eval(text.strip() or "None")
    if not isinstance(parsed, list):
        raise TypeError("Top-level config must be a list")
    return parsed


def _configs(fields: Sequence[str]) -> List[CommConfig]:
    return [_parse_config_string(f) for f in fields]


def _item_ac(tup) -> ScheduleItem:
    if not isinstance(tup, tuple) or len(tup) < 3:
        raise TypeError("Instruction tuple must be ('name', ...) with at least 3 elements")
    name = tup[0]
    if name == "forward":
        if len(tup) != 3:
            raise TypeError("Forward tuple must be ('forward', attn:str, mlp:str)")
        attn, mlp = _configs(tup[1:])
        return ScheduleItem(fwd_attn=attn, fwd_mlp=mlp, bwd_attn=None, bwd_mlp=None)
    if name == "backward":
        if len(tup) != 5:
            raise TypeError(
                "Backward tuple must be ('backward', rec_attn:str, rec_mlp:str, attn:str, mlp:str)"
            )
        rec_attn, rec_mlp, attn, mlp = _configs(tup[1:])
        # The recompute pass of a backward instruction reads the fwd_* fields.
        return ScheduleItem(fwd_attn=rec_attn, fwd_mlp=rec_mlp, bwd_attn=attn, bwd_mlp=mlp)
    raise ValueError(f"Unknown instruction name: {name}")


def _item_ac_cp(tup) -> ScheduleItemCP:
    if not isinstance(tup, tuple) or len(tup) < 2:
        raise TypeError("Instruction tuple must be ('name', ...) with at least 2 elements")
    name = tup[0]
    if name == "forward":
        if len(tup) != 1 + len(_CP_FWD):
            raise TypeError(
                "Forward tuple must be ('forward', qkv_ar:str, qkv_ag:str, ao_ag:str, ao_ar:str, mlp:str)"
            )
        kw = dict(zip(_CP_FWD, _configs(tup[1:])))
        kw.update({k: None for k in _CP_BWD})
        return ScheduleItemCP(**kw)
    if name == "backward":
        if len(tup) != 1 + len(_CP_FWD) + len(_CP_BWD):
            raise TypeError(
                "Backward tuple must be ('backward', <5 recompute fields>, qkv_ar:str, qkv_rs:str, "
                "a_rs:str, a_ag:str, o_ag:str, o_ar:str, mlp:str)"
            )
        return ScheduleItemCP(**dict(zip(_CP_FWD + _CP_BWD, _configs(tup[1:]))))
    raise ValueError(f"Unknown instruction name: {name}")


def _split_pair(item):
    if not (isinstance(item, tuple) and len(item) == 2):
        raise TypeError("Each microbatch entry must be a tuple of two tuples: (forward, backward)")
    return item


def _check_names(fwd, bwd) -> None:
    if fwd[0] != "forward" or bwd[0] != "backward":
        raise ValueError(f"Expected ('forward', ...), ('backward', ...), got: {fwd[0]}, {bwd[0]}")


def _item_pair(item) -> ScheduleItem:
    fwd, bwd = _split_pair(item)
    for raw, label in ((fwd, "Forward"), (bwd, "Backward")):
        if not (isinstance(raw, tuple) and len(raw) == 3 and all(isinstance(f, str) for f in raw)):
            raise TypeError(f"{label} entry must be (name:str, attn:str, mlp:str)")
    _check_names(fwd, bwd)
    fa, fm = _configs(fwd[1:])
    ba, bm = _configs(bwd[1:])
    return ScheduleItem(fwd_attn=fa, fwd_mlp=fm, bwd_attn=ba, bwd_mlp=bm)


def _item_pair_cp(item) -> ScheduleItemCP:
    fwd, bwd = _split_pair(item)
    if len(fwd) != 1 + len(_CP_FWD):
        raise TypeError(
            "Forward entry must be (name:str, qkv_ar:str, qkv_ag:str, ao_ag:str, ao_ar:str, mlp:str)"
        )
    if len(bwd) != 1 + len(_CP_BWD):
        raise TypeError(
            "Backward entry must be (name:str, qkv_ar:str, qkv_rs:str, a_rs:str, a_ag:str, "
            "o_ag:str, o_ar:str, mlp:str)"
        )
    _check_names(fwd, bwd)
    kw = dict(zip(_CP_FWD, _configs(fwd[1:])))
    kw.update(zip(_CP_BWD, _configs(bwd[1:])))
    return ScheduleItemCP(**kw)


def parse_schedule_file(
    path: Union[str, Path],
    use_activation_checkpointing: bool,
    context_parallel: bool,
) -> List[List[Union[ScheduleItem, ScheduleItemCP]]]:
    """File -> one list of schedule items per pipeline stage."""
    parsed = _load_literal(path)
    if use_activation_checkpointing:
        convert = _item_ac_cp if context_parallel else _item_ac
        what = "instruction tuples in 1F1B order"
    else:
        convert = _item_pair_cp if context_parallel else _item_pair
        what = "microbatch pairs ((forward_tuple),(backward_tuple))"
    stages = []
    for idx, per_stage in enumerate(parsed):
        if not isinstance(per_stage, list):
            raise TypeError(f"Entry {idx} must be a list of {what}")
        stages.append([convert(entry) for entry in per_stage])
    return stages


def parse_frequency_file(path: Union[str, Path]) -> List[List[Tuple[str, int]]]:
    """``freqs_pipeline_*.py`` -> per stage ``[("forward"|"backward", MHz), ...]`` in the
    same instruction order as the schedule file (format: the shipped plans under
    tests/kareus/schedules/.../frontier/freqs_pipeline_*.py of the reference)."""
    parsed = _load_literal(path)
    stages = []
    for idx, per_stage in enumerate(parsed):
        if not isinstance(per_stage, list):
            raise TypeError(f"Entry {idx} must be a list of (instruction, MHz) tuples")
        items = []
        for entry in per_stage:
            if not (isinstance(entry, tuple) and len(entry) == 2):
                raise TypeError("Frequency entry must be (name:str, mhz:int)")
            name, mhz = entry
            if name not in ("forward", "backward"):
                raise ValueError(f"Unknown instruction name: {name}")
            if not isinstance(mhz, int) or isinstance(mhz, bool) or mhz <= 0:
                raise ValueError(f"Frequency must be a positive integer MHz value, got: {mhz!r}")
            items.append((name, mhz))
        stages.append(items)
    return stages
