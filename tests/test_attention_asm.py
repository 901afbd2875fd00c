"""The dQ kernel with one wave per SIMD issues its score MFMAs as inline assembly, so the compiler inserts
none of the wait states a reader of an MFMA result needs (on gfx950 an 8-pass MFMA's result may be read by
a vector, memory or LDS instruction eleven issue slots later at the earliest).  The kernel keeps that
distance by construction; this test reads the compiled kernel and checks that it does — after a compiler
update, a change of flags or an edit that makes the register allocator copy or spill such a register
early, it fails instead of the kernel silently reading half-written values.  No GPU needed."""

import os
import re
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "kareus_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
WAIT_SLOTS = 12
OPERAND_SLOTS = 4


def _regs(token, kind):
    token = token.strip().strip(",")
    m = re.match(kind + r"\[(\d+):(\d+)\]$", token)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(kind + r"(\d+)$", token)
    return {int(m.group(1))} if m else set()


def _kernel_body(text, kernel):
    lines, on = [], False
    for line in text.split("\n"):
        if re.match(r"^_Z\w*" + kernel + r"\w*:", line):
            on = True
        if on:
            lines.append(line)
            if "s_endpgm" in line:
                break
    return lines


def early_readers(lines, need=WAIT_SLOTS):
    """(number of inline-assembly MFMAs, [(line, text, distance)] of instructions that read a VGPR less than
    `need` issue slots after an inline-assembly MFMA wrote it, and of inline-assembly MFMAs that take an operand
    a vector instruction wrote fewer than OPERAND_SLOTS slots before).  Every instruction counts as one slot
    (they take at least that), `s_nop n` as n + 1.  An MFMA accumulating onto its own earlier result is the
    hardware's business and is not a reader here."""
    stores = ("ds_write", "global_store", "buffer_store", "scratch_store")
    in_asm, slot, written, bad, n_asm, fresh = False, 0, {}, [], 0, {}
    for i, line in enumerate(lines):
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not t or t[0] in ";." or t.endswith(":"):
            continue
        code = t.split(";")[0].strip()
        op, _, rest = code.partition(" ")
        args = [a.strip() for a in rest.split(",") if a.strip()]
        slot += 1
        if op == "s_nop":
            slot += int(args[0])
            continue
        if in_asm and op.startswith("v_mfma"):
            n_asm += 1
            # its operands must not have been written by a vector instruction just before it either: the
            # compiler would separate such a pair if it knew what the assembly is
            for a in args[1:]:
                for kind in "va":
                    for r in _regs(a, kind):
                        if slot - fresh.get((kind, r), -10 ** 9) < OPERAND_SLOTS:
                            bad.append((i, t, slot - fresh[(kind, r)]))
            for r in _regs(args[0], "v"):
                written[r] = slot
            continue
        if op.startswith("v_") and args:
            for kind in "va":
                for r in _regs(args[0], kind):
                    fresh[(kind, r)] = slot
        for a in (args if op.startswith(stores) else args[1:]):
            for r in _regs(a, "v"):
                if r in written and slot - written[r] < need:
                    bad.append((i, t, slot - written[r]))
        if args and not op.startswith(stores) and not op.startswith("s_"):
            for r in _regs(args[0], "v"):
                written.pop(r, None)          # rewritten by an instruction the compiler knows
    return n_asm, bad


def test_checker_sees_an_early_reader_and_accepts_a_late_one():
    mfma = [";;#ASMSTART", "\tv_mfma_f32_32x32x16_bf16 v[0:15], v[20:23], a[0:3], 0", ";;#ASMEND"]
    early = mfma + ["\tv_add_f32_e32 v40, v3, v41"]
    late = mfma + ["\ts_nop 15", "\tv_add_f32_e32 v40, v3, v41"]
    chained = mfma + [";;#ASMSTART", "\tv_mfma_f32_32x32x16_bf16 v[0:15], v[24:27], a[4:7], v[0:15]", ";;#ASMEND"]
    spilled = mfma + ["\tscratch_store_dwordx4 off, v[12:15], off offset:16"]
    assert early_readers(early) == (1, [(3, "v_add_f32_e32 v40, v3, v41", 1)])
    assert early_readers(late) == (1, [])
    assert early_readers(chained) == (2, [])
    assert len(early_readers(spilled)[1]) == 4
    copied = ["\tv_accvgpr_write_b32 a0, v9"] + mfma
    assert early_readers(copied) == (1, [(2, "v_mfma_f32_32x32x16_bf16 v[0:15], v[20:23], a[0:3], 0", 1)])


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc is not installed")
def test_no_instruction_reads_a_hand_placed_mfma_result_too_early(tmp_path):
    out = tmp_path / "kr_attention.s"
    subprocess.run(["make", "-C", CSRC, f"HIPCC={HIPCC}", f"ASMDIR={tmp_path}", str(out)], check=True,
                   stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=600)
    text = out.read_text()
    body = _kernel_body(text, "attn_bwd_dq_w64_kernel")
    assert body, "kernel not found in the assembly"
    n_asm, bad = early_readers(body)
    # prologue 32 + two steps of the loop 64 + the diagonal tile's first step 32
    assert n_asm == 128
    assert not bad, bad[:5]
    meta = text[text.index("attn_bwd_dq_w64_kernel", text.index("amdhsa.kernels")):]
    spills = re.search(r"\.vgpr_spill_count:\s*(\d+)", meta)
    assert spills and int(spills.group(1)) == 0
