"""Build libcornserve_amd.so (the C-ABI kernel library) in-tree with hipcc for gfx950.

Usage: ``python -m cornserve_amd.build`` or ``cornserve_amd.build.build_library()``.  The library is
written next to the sources so that it travels with the tree; nothing is JIT-compiled at import.
"""

from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_PATH = PKG_DIR / "libcornserve_amd.so"
OBJ_DIR = CSRC / "build"

ARCH = "gfx950"
# Packed-FP32 instructions are disabled for every device translation unit (see the project notes on
# v_pk_*_f32); the host pass prints a harmless "not a recognized feature" note for the same flag.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libcornserve_amd.so")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(line for line in proc.stdout.splitlines() if "packed-fp32-ops" not in line and "--hip-link" not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


# Sources with this marker keep their accumulators in accumulation registers that only inline assembly
# touches; the compiler does not know they are occupied, so its output is checked after every build.
HAND_MANAGED_ACC_MARKER = "CS_ALL_ACC_REGS"
_ACC_REG = re.compile(r"\ba(\d+|\[)")


def check_hand_managed_acc_registers(asm_text: str) -> list[str]:
    """Return the kernels that use inline-assembly accumulation registers AND in which compiler-generated
    code touches an accumulation register too (a register spill or a staging copy would corrupt the
    accumulators).  An empty list means the convention holds."""
    offenders = []
    for m in re.finditer(r"^(_Z\S+):.*?s_endpgm", asm_text, re.S | re.M):
        in_asm, uses_inline, outside = False, False, 0
        for line in m.group(0).splitlines():
            if "#ASMSTART" in line:
                in_asm = True
                continue
            if "#ASMEND" in line:
                in_asm = False
                continue
            code = line.split(";")[0]
            if _ACC_REG.search(code):
                if in_asm:
                    uses_inline = True
                else:
                    outside += 1
        if uses_inline and outside:
            offenders.append(f"{m.group(1)}: {outside} compiler-generated accumulation-register references")
    return offenders


def _check_source(hipcc: str, src: Path) -> None:
    asm = OBJ_DIR / (src.stem + ".gfx950.s")
    _run([hipcc, *HIPCC_FLAGS, "-S", "--cuda-device-only", str(src), "-o", str(asm)])
    offenders = check_hand_managed_acc_registers(asm.read_text())
    asm.unlink()
    if offenders:
        # the object of a source that fails this check must not survive for a later incremental build to link
        (OBJ_DIR / (src.stem + ".o")).unlink(missing_ok=True)
        raise RuntimeError(f"{src.name}: the compiler used accumulation registers that inline assembly owns:\n  "
                           + "\n  ".join(offenders))


def _check_no_missing_kernels(lib: Path) -> None:
    """A shared library links with undefined symbols; a kernel whose host-side launch stub the compiler
    dropped would only show up as a load error on the GPU box.  Every undefined symbol must be external
    (HIP runtime, libc/libstdc++): none may come from this library's own (anonymous) namespaces."""
    nm = shutil.which("nm")
    if nm is None:
        return
    out = subprocess.run([nm, "-D", "--undefined-only", str(lib)], stdout=subprocess.PIPE, text=True).stdout
    own = [line.split()[-1] for line in out.splitlines() if "GLOBAL__N" in line or " cs_" in line]
    if own:
        raise RuntimeError(f"{lib.name} has undefined symbols of its own (dropped kernels?):\n  " + "\n  ".join(own))


def build_library(force: bool = True, jobs: int = 8) -> Path:
    """Compile every .hip source under csrc/ and link the shared library. Returns its path."""
    hipcc = _hipcc()
    OBJ_DIR.mkdir(exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    headers = list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h"))
    newest_hdr = max(h.stat().st_mtime for h in headers)
    objs = []
    todo = []
    for src in sources:
        obj = OBJ_DIR / (src.stem + ".o")
        objs.append(obj)
        stale = force or not obj.exists() or obj.stat().st_mtime < max(src.stat().st_mtime, newest_hdr)
        if stale:
            todo.append(lambda cmd=[hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]: _run(cmd))
            if HAND_MANAGED_ACC_MARKER in src.read_text():
                todo.append(lambda src=src: _check_source(hipcc, src))
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo) or 1))) as pool:
        list(pool.map(lambda job: job(), todo))
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB_PATH), *map(str, objs)])
    _check_no_missing_kernels(LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    incremental = "--incremental" in sys.argv
    print(build_library(force=not incremental))
