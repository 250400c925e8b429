"""Scan of gfx950 assembly for the one hazard the compiler cannot see in this library's kernels.

The four-wave GEMM kernels and the direct convolution kernel issue their MFMAs from inline assembly
(so that every accumulator stays in its registers).  To the compiler such a statement is opaque: it does not know that the
result arrives some passes later, and inserts none of the wait states that an ordinary instruction
reading (or overwriting) the result registers needs behind an MFMA -- the kernels carry them
themselves.  This scan checks that they do: for every MFMA inside an inline-assembly region it
follows the instruction stream and reports any non-MFMA instruction that names one of the MFMA's
destination registers before enough wait states have gone by (every instruction
counts one, ``s_nop N`` counts N + 1).  The stream is read in layout order, branches are not
followed: a block laid out behind an MFMA but reached another way can give a false alarm, never a
miss on the fall-through path.

Wait states (XDL write of a VGPR followed by a VALU / VMEM / LDS access, gfx940 and later):
passes + 3, with 4 passes for v_mfma_i32_16x16x64_i8, 8 for the 4-bit and 16 for the 8-bit forms
of v_mfma[_scale]_f32_32x32x64_f8f6f4.
"""
import re

_RANGE = re.compile(r"^([av])\[(\d+):(\d+)\]$")
_ONE = re.compile(r"^([av])(\d+)$")
_LABEL = re.compile(r"^([A-Za-z_][\w$]*):")


def _acc_regs(token):
    """The registers a token names, as (file, index) pairs: accumulation registers and ordinary vector
    registers both (the direct convolution kernel accumulates in the latter)."""
    m = _RANGE.match(token)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = _ONE.match(token)
    if m:
        return {(m.group(1), int(m.group(2)))}
    return set()


def _wait_states_needed(line):
    if "i32_16x16x64_i8" in line:
        return 4 + 3
    if "32x32x64_f8f6f4" in line:
        return (8 if "cbsz:4" in line and "blgp:4" in line else 16) + 3
    if "16x16x128_f8f6f4" in line:
        return (4 if "cbsz:4" in line and "blgp:4" in line else 8) + 3
    return 16 + 3   # unknown form: the longest


def scan(path, only=None):
    """Returns (number of inline-assembly MFMAs seen, list of hazard descriptions).  ``only``: a
    substring that a kernel's mangled name must contain to be scanned."""
    hazards, seen = [], 0
    kernel, in_asm, pending = None, False, []
    with open(path) as f:
        for number, raw in enumerate(f, 1):
            text = raw.strip()
            if text.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if text.startswith(";;#ASMEND"):
                in_asm = False
                continue
            label = _LABEL.match(text)   # a function's label (block labels start with a dot)
            if label:
                kernel, pending = label.group(1), []
                continue
            if not text or text[0] in ".;":
                continue
            if only is not None and (kernel is None or only not in kernel):
                continue
            text = text.split(";")[0].strip()
            parts = text.replace(",", " ").split()
            op, operands = parts[0], parts[1:]
            states = int(operands[0]) + 1 if op == "s_nop" else 1
            if op.startswith("v_mfma") or op.startswith("v_smfmac"):
                # an MFMA that accumulates into the registers of the one before it is interlocked
                pending = [(r, w - states, n) for (r, w, n) in pending if w - states > 0]
                if in_asm:
                    seen += 1
                    pending.append((_acc_regs(operands[0]), _wait_states_needed(text), number))
                continue
            touched = set()
            for token in operands:
                touched |= _acc_regs(token)
            for regs, left, at in pending:
                if touched & regs:
                    first = min(touched & regs)
                    hazards.append(f"{kernel}: line {number} `{text}` touches {first[0]}{first[1]}.. "
                                   f"{left} wait states early (MFMA at line {at})")
            pending = [(r, w - states, n) for (r, w, n) in pending if w - states > 0]
    return seen, hazards


def scan_assembly_loads(path, only=None):
    """The second hazard of this kind: vector-memory loads issued from inline assembly.

    The int4 GEMV over reordered weights issues its global loads as assembly statements and waits
    for them with counted ``s_waitcnt vmcnt(N)`` statements of its own; the compiler believes a
    load's destination registers hold their value from the load on and may copy them
    (``v_mov``) before the wait, which reads whatever the registers held before.  For every
    ``global_load`` inside an inline-assembly region this scan follows the stream in layout order and
    reports any instruction that names one of its destination registers before a
    ``s_waitcnt vmcnt(N)`` with N at most the number of assembly loads issued since (a wave's loads
    return in order).  A load into the same registers ends the watch as well.  Branches are not
    followed.  Returns (loads seen, hazards)."""
    hazards, seen = [], 0
    kernel, in_asm, pending = None, False, []   # pending: [registers, loads issued behind, line]
    with open(path) as f:
        for number, raw in enumerate(f, 1):
            text = raw.strip()
            if text.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if text.startswith(";;#ASMEND"):
                in_asm = False
                continue
            label = _LABEL.match(text)
            if label:
                kernel, pending = label.group(1), []
                continue
            if not text or text[0] in ".;":
                continue
            if only is not None and (kernel is None or only not in kernel):
                continue
            text = text.split(";")[0].strip()
            parts = text.replace(",", " ").split()
            op, operands = parts[0], parts[1:]
            if op == "s_waitcnt":
                m = re.search(r"vmcnt\((\d+)\)", text)
                if m:
                    pending = [p for p in pending if p[1] < int(m.group(1))]
                continue
            if op == "s_endpgm":
                pending = []
                continue
            touched = set()
            for token in operands:
                touched |= _acc_regs(token)
            is_load = op.startswith("global_load") or op.startswith("buffer_load") or op.startswith("scratch_load")
            dest = _acc_regs(operands[0]) if is_load and operands else set()
            for regs, behind, at in pending:
                hit = (touched - dest) & regs if is_load else touched & regs
                if hit:
                    first = min(hit)
                    hazards.append(f"{kernel}: line {number} `{text}` names {first[0]}{first[1]} before the load "
                                   f"at line {at} has been waited for")
            if is_load:
                pending = [p for p in pending if not (p[0] & dest)]
                for p in pending:
                    p[1] += 1
                if in_asm:
                    seen += 1
                    pending.append([dest, 0, number])
    return seen, hazards


def scan_m0_writes(path, only=None):
    """A third hazard the compiler cannot see: inside inline assembly, a write of M0 needs one wait
    state (any instruction) before a direct-to-LDS load reads it as its LDS destination.  The
    twelve-slab loops of the four-wave GEMM kernels write M0 themselves.  Returns (M0 writes seen
    inside assembly regions, hazards): a hazard is an assembly M0 write whose next instruction is a
    ``global_load_lds_*`` / ``buffer_load_* ... lds``."""
    hazards, seen = [], 0
    kernel, in_asm, m0_just_written = None, False, None
    with open(path) as f:
        for number, raw in enumerate(f, 1):
            text = raw.strip()
            if text.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if text.startswith(";;#ASMEND"):
                in_asm = False
                continue
            label = _LABEL.match(text)
            if label:
                kernel, m0_just_written = label.group(1), None
                continue
            if not text or text[0] in ".;":
                continue
            if only is not None and (kernel is None or only not in kernel):
                continue
            text = text.split(";")[0].strip()
            parts = text.replace(",", " ").split()
            op, operands = parts[0], parts[1:]
            is_lds_load = op.startswith("global_load_lds") or (op.startswith("buffer_load") and "lds" in operands)
            if is_lds_load and m0_just_written is not None:
                hazards.append(f"{kernel}: line {number} `{text}` reads M0 written by the instruction before it "
                               f"(line {m0_just_written})")
            m0_just_written = None
            if in_asm and op.startswith("s_") and operands and operands[0] == "m0":
                seen += 1
                m0_just_written = number
    return seen, hazards
