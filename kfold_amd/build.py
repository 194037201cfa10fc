"""Build libkfold_hip.so (gfx950) in-tree with hipcc.

``python -m kfold_amd.build`` or ``kfold_amd.build.build()``.  Objects are compiled in
parallel into ``kfold_amd/csrc/_obj`` and linked into ``kfold_amd/libkfold_hip.so``.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
LIB = ROOT / "libkfold_hip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 VALU forms are disabled for all device code (device-only feature flag; the
# host pass prints a harmless "not a recognized feature" note)
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unused-command-line-argument",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, obj: Path, verbose: bool) -> None:
    cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)


# kernel files whose machine code the committed profiles were measured on
ISA_FILES = ("trimul", "contract", "triattn", "flash", "transition", "pairbias")
ISA_JSON = ROOT / "kernel_isa.json"


RESOURCES_JSON = ROOT / "kernel_resources.json"
_RESOURCE_KEYS = ("vgpr_count", "agpr_count", "sgpr_count", "group_segment_fixed_size",
                  "private_segment_fixed_size", "vgpr_spill_count", "max_flat_workgroup_size")


def _asm_of(src: Path) -> str:
    """gfx950 assembly (with the code object's metadata) of one source file."""
    res = subprocess.run([HIPCC, *FLAGS, "--cuda-device-only", "-S", str(src), "-o", "-"],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src.name}:\n{res.stderr[-2000:]}")
    return res.stdout


def _resources_of(asm: str) -> dict[str, dict[str, int]]:
    """{mangled kernel name: registers, LDS bytes, scratch bytes per lane, spilled registers, largest
    workgroup} as the compiler records them in the code object's metadata."""
    import re

    out = {}
    for m in re.finditer(r"- \.agpr_count:.*?\.wavefront_size", asm, re.S):
        block = m.group(0)
        name = re.search(r"\.name:\s+(\S+)", block).group(1)
        out[name] = {k: int(re.search(rf"\.{k}:\s+(\d+)", block).group(1)) for k in _RESOURCE_KEYS}
    return out


def _isa_of(asm: str) -> dict[str, str]:
    """{mangled kernel name: digest of its gfx950 instruction stream} for one file's assembly.  Labels,
    directives and comments are dropped, so the digest changes only when an instruction does."""
    import hashlib
    import re

    out: dict[str, list[str]] = {}
    cur = None
    for line in asm.splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            cur = m.group(1)
            out[cur] = []
            continue
        if cur is None:
            continue
        code = line.split(";")[0].strip()
        if code.startswith(".Lfunc_end"):
            cur = None
        elif code and not code.startswith("."):
            out[cur].append(code)
    return {k: hashlib.sha256("\n".join(v).encode()).hexdigest()[:16] for k, v in out.items()}


def isa_digests(jobs: int = 8) -> dict[str, str]:
    """Digest of the compiled instruction stream of every kernel of the hot-path files: what a
    measurement (a rocprofv3 summary under profiles/) is valid for.  Edits that leave a kernel's
    machine code unchanged (comments, new helpers, other kernels) keep its digest."""
    return kernel_facts(jobs, [CSRC / f"{name}.hip" for name in ISA_FILES])[0]


def kernel_facts(jobs: int = 8, srcs: list[Path] | None = None) -> tuple[dict[str, str], dict[str, dict[str, int]]]:
    """(instruction-stream digests of the hot-path files' kernels, compiler-reported resources of
    every kernel) from one assembly pass over the sources."""
    srcs = sources() if srcs is None else srcs
    hot = {CSRC / f"{name}.hip" for name in ISA_FILES}
    isa: dict[str, str] = {}
    res: dict[str, dict[str, int]] = {}
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, asm in zip(srcs, ex.map(_asm_of, srcs)):
            if src in hot:
                isa.update(_isa_of(asm))
            res.update(_resources_of(asm))
    return dict(sorted(isa.items())), dict(sorted(res.items()))


def build(verbose: bool = False, jobs: int | None = None) -> Path:
    objdir = CSRC / "_obj"
    objdir.mkdir(exist_ok=True)
    srcs = sources()
    objs = [objdir / (s.stem + ".o") for s in srcs]
    jobs = jobs or min(len(srcs), os.cpu_count() or 4, 16)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _compile(so[0], so[1], verbose), zip(srcs, objs)))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    import json

    isa, resources = kernel_facts(jobs)
    ISA_JSON.write_text(json.dumps(isa, indent=1) + "\n")
    RESOURCES_JSON.write_text(json.dumps(resources, indent=1) + "\n")
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
