"""Reads the generated gfx950 ISA of dscuda_amd/csrc/mla_decode.hip and checks the one property of the
hand-issued score MFMAs that neither the compiler nor the hardware enforces.

Those MFMAs (inline asm, destination in ordinary vector registers) form dependent chains.  The hardware
interlocks MFMA-after-MFMA on the same accumulator, but a vector-ALU, LDS or memory instruction that reads or
writes the accumulator's registers needs software wait states after the last MFMA that wrote them (8 passes + 3
on this part).  To the compiler the accumulator is an ordinary value after each asm statement, so it may place
a register move in the middle of a chain; this test fails if the built code contains any such access:

    for every MFMA whose destination is a VGPR tuple (the compiler's own MFMAs write AGPRs), no instruction
    other than an MFMA accumulating into exactly that tuple may name a register of the tuple until at least
    MIN_WAIT_STATES wait states (instructions issued, ``s_nop N`` counting N + 1) have passed.

It needs hipcc, not a GPU."""

import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
MIN_WAIT_STATES = 12

REGISTER = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def _registers(text):
    for match in REGISTER.finditer(text):
        if match.group(3) is not None:
            yield int(match.group(3)), int(match.group(3))
        else:
            yield int(match.group(1)), int(match.group(2))


def check_isa(text):
    """Returns a list of (kernel, line number, instruction, tuple) violations."""
    violations = []
    kernel = None
    pending = {}   # (low, high) of a VGPR accumulator -> wait states since the last MFMA that wrote it
    for number, raw in enumerate(text.splitlines(), 1):
        line = raw.split(";")[0].strip()
        if not line:
            continue
        if re.match(r"^_Z\w+:", line):
            kernel, pending = line[:-1], {}
            continue
        if line.startswith(".") or line.endswith(":"):
            continue   # directives and labels; state is carried across labels on purpose
        mnemonic, _, operands = line.partition(" ")
        if mnemonic == "s_endpgm":
            pending = {}
            continue
        if mnemonic.startswith("v_mfma"):
            fields = [field.strip() for field in operands.split(",")]
            destination = next(_registers(fields[0]), None)
            if fields[0].startswith("v") and destination is not None:
                # operands A and B may not be registers of an accumulator in flight
                for low, high in pending:
                    for operand in fields[1:3]:
                        for a, b in _registers(operand):
                            if a <= high and b >= low and (low, high) != destination:
                                violations.append((kernel, number, line, (low, high)))
                source_c = next(_registers(fields[3]), None) if len(fields) > 3 else None
                for low, high in list(pending):
                    overlaps = destination[0] <= high and destination[1] >= low
                    if overlaps and (low, high) != destination:
                        violations.append((kernel, number, line, (low, high)))
                    if source_c and source_c[0] <= high and source_c[1] >= low and source_c != destination:
                        violations.append((kernel, number, line, (low, high)))
                for key in pending:
                    pending[key] += 1
                pending[destination] = 0
                continue
        else:
            for low, high in pending:
                if pending[(low, high)] >= MIN_WAIT_STATES:
                    continue
                for a, b in _registers(operands):
                    if a <= high and b >= low:
                        violations.append((kernel, number, line, (low, high)))
                        break
        states = 1
        if mnemonic == "s_nop":
            states = int(operands.strip()) + 1
        for key in list(pending):
            pending[key] += states
            if pending[key] >= 64:
                del pending[key]
    return violations


def test_checker_on_hand_written_cases():
    safe = """
_Zkernel:
    v_mfma_f32_32x32x16_bf16 v[16:31], v[192:195], v[36:39], 0
    ds_read_b128 v[192:195], v218
    v_mfma_f32_32x32x16_bf16 v[16:31], v[188:191], v[40:43], v[16:31]
    s_nop 15
    s_nop 7
    v_mov_b64_e32 v[0:1], v[16:17]
    s_endpgm
"""
    assert check_isa(safe) == []
    early_move = safe.replace("    s_nop 15\n    s_nop 7\n", "")
    assert len(check_isa(early_move)) == 1
    move_inside_chain = """
_Zkernel:
    v_mfma_f32_32x32x16_bf16 v[16:31], v[192:195], v[36:39], 0
    v_mov_b64_e32 v[0:1], v[16:17]
    v_mfma_f32_32x32x16_bf16 v[0:15], v[188:191], v[40:43], v[0:15]
    s_endpgm
"""
    assert len(check_isa(move_inside_chain)) >= 1
    load_into_accumulator = """
_Zkernel:
    v_mfma_f32_32x32x16_bf16 v[16:31], v[192:195], v[36:39], 0
    ds_read_b64_tr_b16 v[18:19], v191 offset:9536
    s_endpgm
"""
    assert len(check_isa(load_into_accumulator)) == 1
    compiler_mfma = """
_Zkernel:
    v_mfma_f32_32x32x16_bf16 a[0:15], v[192:195], v[4:7], a[0:15]
    v_accvgpr_read_b32 v0, a0
    s_endpgm
"""
    assert check_isa(compiler_mfma) == []


def test_no_access_to_score_accumulators_in_flight(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(hipcc).exists():
        pytest.skip("no hipcc")
    from dscuda_amd.build import COMMON_FLAGS, CSRC

    target = tmp_path / "mla_decode.s"
    flags = [flag for flag in COMMON_FLAGS if flag != "-fPIC"]
    result = subprocess.run([hipcc, *flags, "--cuda-device-only", "-S", str(CSRC / "mla_decode.hip"), "-o", str(target)],
                            capture_output=True, text=True, timeout=900)
    assert result.returncode == 0, result.stderr[-3000:]
    text = target.read_text()
    assert "v_mfma_f32_32x32x16_bf16 v[" in text, "the hand-issued MFMAs should show up with VGPR destinations"
    violations = check_isa(text)
    report = "\n".join(f"{kernel} line {number}: `{line}` touches v[{low}:{high}] in flight"
                       for kernel, number, line, (low, high) in violations[:20])
    assert not violations, report
