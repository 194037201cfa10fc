"""Build the host execution model of the kernels: ``tests/hostsim/libkfold_hostsim.so``.

TEST INFRASTRUCTURE.  The kernel sources of ``kfold_amd/csrc`` are compiled as plain C++ for
x86-64 with ``tests/hostsim/hip/hip_runtime.h`` standing where HIP's header stands in the GPU
build, and linked with the fiber runtime ``hostsim.cpp``.  The library exports the same C ABI as
``libkfold_hip.so`` (pointers are host pointers) plus the ``hostsim_*`` controls.  Only tests load
it; the product never does.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
CSRC = ROOT / "kfold_amd" / "csrc"
LIB = HERE / "libkfold_hostsim.so"
OBJ = HERE / "_obj"

CXX = os.environ.get("HOSTSIM_CXX", "/opt/rocm/llvm/bin/clang++")
FLAGS = ["-x", "c++", "-std=c++17", "-O2", "-march=x86-64-v3", "-fPIC", "-pthread", "-w",
         f"-I{HERE}", "-ffp-contract=off"]
# HOSTSIM_EXTRA_FLAGS: extra host-compiler flags for a checking build of this library: clang's
# undefined-behaviour checks in trapping mode (alignment of every typed load and store; signed and
# unsigned overflow and 64 -> 32 bit truncation of index arithmetic, with ubsan_ignore.txt listing
# the one intended wrap; bounds of the per-lane arrays).  hostsim.cpp reports the kernel, workgroup,
# thread and library offset of a trap; the README lists the command lines.
FLAGS += os.environ.get("HOSTSIM_EXTRA_FLAGS", "").split()


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip")) + [HERE / "hostsim.cpp"]


def up_to_date() -> bool:
    if not LIB.exists():
        return False
    t = LIB.stat().st_mtime
    deps = list(CSRC.glob("*.hip")) + list(CSRC.glob("*.hpp")) + [HERE / "hostsim.cpp",
            HERE / "hip" / "hip_runtime.h", ROOT / "include" / "kfold_hip.h"]
    return all(d.stat().st_mtime <= t for d in deps)


def _compile(src: Path) -> Path:
    obj = OBJ / (src.stem + ".o")
    res = subprocess.run([CXX, *FLAGS, "-c", str(src), "-o", str(obj)], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"host build failed for {src.name}:\n{res.stderr[-4000:]}")
    return obj


def build(force: bool = False) -> Path:
    if not force and up_to_date():
        return LIB
    OBJ.mkdir(exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(len(srcs), os.cpu_count() or 4, 16)) as ex:
        objs = list(ex.map(_compile, srcs))
    res = subprocess.run([CXX, "-shared", "-fPIC", "-pthread", "-o", str(LIB), *map(str, objs)],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"host link failed:\n{res.stderr[-4000:]}")
    return LIB


if __name__ == "__main__":
    print(build(force="-f" in sys.argv))
