"""A check on the compiled code of kernels whose loads are issued from inline assembly.

The weight-streaming kernels of ``csrc/skinny_resident_kernels.h`` request their weights with ``asm volatile`` loads
and wait for them with explicit ``s_waitcnt vmcnt(N)``.  The compiler does not know that a register named as the
output of such a load is still being written: given a reason (a loop-carried value, a register budget that makes it
spill) it will copy, move or store that register between the request and the wait, and the kernel then computes on
whatever the register held before the load landed.  The kernels are written so that this does not happen
(straight-line code, one definition per request); this module replays the load / wait order of the compiled code and
reports any instruction that touches a vector register while an earlier load into it may still be in flight, so that
a compiler change or an edit that brings the hazard back is caught without a GPU.

Loads retire in issue order, so after ``s_waitcnt vmcnt(n)`` only the youngest n loads are in flight.  The scan is
linear (branches are not followed), which is exact for straight-line kernels and a single pass over each loop body
otherwise.
"""

from __future__ import annotations

import re
import shutil
import subprocess
import tempfile
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
_REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def _registers(text: str) -> set[int]:
    out: set[int] = set()
    for m in _REG.finditer(text):
        if m.group(1) is not None:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def scan_kernel(lines: list[str]) -> list[str]:
    """Findings (one string per offending instruction) for the instructions of one kernel."""
    in_flight: list[set[int]] = []  # destination registers of the loads in flight, oldest first
    findings = []
    for number, line in enumerate(lines, 1):
        text = line.split(";")[0].strip()
        if not text or text.startswith(".") or text.endswith(":"):
            continue
        op = text.split()[0]
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", text)
            if m:
                del in_flight[: max(0, len(in_flight) - int(m.group(1)))]
            continue
        live = set().union(*in_flight) if in_flight else set()
        if op.startswith(("global_load", "buffer_load")):
            operands = text[len(op):].split(",")
            dst = set() if "lds" in op else _registers(operands[0])
            touched = (dst | _registers(",".join(operands[1:]))) & live
            in_flight.append(dst)
        else:
            if op.startswith(("global_store", "global_atomic", "buffer_store")):
                in_flight.append(set())  # stores count in vmcnt as well
            touched = _registers(text) & live
        if touched:
            findings.append(f"line {number}: {text}  (in flight: v{sorted(touched)[0]} ...)")
    return findings


def scan(asm: str, name_contains: str = "") -> dict[str, list[str]]:
    """Kernel symbol -> findings, for every kernel of a device assembly listing whose symbol contains the filter."""
    result: dict[str, list[str]] = {}
    current, body = None, []
    for line in asm.splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            current, body = m.group(1), []
            continue
        if current is not None:
            body.append(line)
            if "s_endpgm" in line:
                if name_contains in current:
                    result[current] = scan_kernel(body)
                current = None
    return result


def compile_device_asm(source: str) -> str:
    """gfx950 device assembly of a HIP translation unit, with the flags the library is built with."""
    from .build import HIPCC_FLAGS

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    flags = [f for f in HIPCC_FLAGS if f not in ("-fPIC", "-shared")]
    with tempfile.TemporaryDirectory() as tmp:
        src, out = Path(tmp) / "unit.hip", Path(tmp) / "unit.s"
        src.write_text(source)
        proc = subprocess.run([hipcc, *flags, f"-I{CSRC}", "--cuda-device-only", "-S", str(src), "-o", str(out)],
                              capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stderr[-2000:]}")
        return out.read_text()
