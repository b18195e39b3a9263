"""Build libmoespresso_amd.so from the HIP sources in ``csrc/`` with hipcc for gfx950.

``python -m moespresso_amd.build`` compiles every source to an object file (in
parallel) and links the shared library in-tree next to this file. hipcc
cross-compiles without a GPU.
"""

from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "_obj")
LIB_PATH = os.path.join(HERE, "libmoespresso_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the asynchronous LDS loads set M0 by hand inside inline asm
    "-Wno-inline-asm",
]


def sources() -> list[str]:
    return sorted(
        os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip") or f.endswith(".cpp")
    )


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    cmd = [HIPCC, *COMMON_FLAGS, "-c", src, "-o", obj]
    if src.endswith(".cpp"):
        cmd = [HIPCC, "-O2", "-std=c++17", "-fPIC", "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


def device_assembly(src: str) -> str:
    """gfx950 assembly of one HIP source (device-only compile, nothing runs)."""
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "kernels.s")
        cmd = [HIPCC, *COMMON_FLAGS, "-S", "--cuda-device-only", "-o", out, src]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stderr}")
        return open(out).read()


def kernel_resources(src: str, text: str | None = None) -> dict[str, dict[str, int]]:
    """Registers and scratch of every kernel in one HIP source, from the code object metadata of a device-only
    compile to assembly: ``{kernel symbol: {"vgprs", "sgprs", "scratch_bytes", "vgpr_spills", "sgpr_spills"}}``.

    The kernels that count their own vector-memory operations (asynchronous tile copies awaited with
    ``s_waitcnt vmcnt(n)``) rely on the compiler adding none: a register spilled to scratch is one more
    vector-memory operation in the middle of the count, and its reload drains every copy in flight.
    """
    import re

    text = device_assembly(src) if text is None else text
    fields = {"vgprs": "vgpr_count", "sgprs": "sgpr_count", "scratch_bytes": "private_segment_fixed_size",
              "vgpr_spills": "vgpr_spill_count", "sgpr_spills": "sgpr_spill_count"}
    kernels: dict[str, dict[str, int]] = {}
    # one metadata record per kernel: "- .agpr_count: ..." up to the next record; ".name:" carries the symbol
    for record in re.split(r"\n  - \.", text[text.index("amdhsa.kernels:"):])[1:]:
        name = re.search(r"\.name:\s+(\S+)", record)
        if not name:
            continue
        kernels[name.group(1)] = {
            key: int(m.group(1)) if (m := re.search(rf"\.{field}:\s+(\d+)", record)) else 0
            for key, field in fields.items()
        }
    return kernels


def kernel_bodies(text: str) -> dict[str, list[str]]:
    """Instruction lines of every kernel of an assembly text: ``{kernel symbol: [line, ...]}``."""
    import re

    bodies: dict[str, list[str]] = {}
    for m in re.finditer(r"^(\w+):[^\n]*\n(.*?)^\s*\.end_amdhsa_kernel", text, flags=re.S | re.M):
        if ".amdhsa_kernel " + m.group(1) in m.group(2):
            bodies[m.group(1)] = m.group(2).split(".section")[0].splitlines()
    return bodies


def inline_asm_register_loads(lines: list[str]) -> list[str]:
    """Memory loads with a register destination that come from inline asm statements (the compiler brackets those
    with ``;;#ASMSTART`` / ``;;#ASMEND``). The compiler takes the outputs of an asm statement for valid the moment
    the statement ends, so a load issued that way may see its destination register moved, reused or spilled while
    the data is still in flight; loads whose destination is LDS write no register and are exempt."""
    import re

    found, inside = [], False
    for line in lines:
        if "#ASMSTART" in line:
            inside = True
        elif "#ASMEND" in line:
            inside = False
        elif inside and re.search(r"\b(global|buffer|flat|scratch)_load|\bs_(buffer_)?load", line) and "_lds_" not in line:
            found.append(line.strip())
    return found


if __name__ == "__main__":
    build()
