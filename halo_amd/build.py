"""Builds ``halo_amd/lib/libhalo_moe.so``: every ``csrc/*.hip`` compiled by hipcc for gfx950 and linked into one
shared library with a plain C ABI (``include/halo_moe.h``).  No torch in the build; hipcc cross-compiles without a
GPU.  ``python -m halo_amd.build`` rebuilds unconditionally."""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PACKAGE_DIR)
CSRC = os.path.join(PACKAGE_DIR, "csrc")
LIB_DIR = os.path.join(PACKAGE_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libhalo_moe.so")
ARCH = "gfx950"

HIPCC_FLAGS = [
    "-O3",
    f"--offload-arch={ARCH}",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed fp32 arithmetic stays off: scalar float code must not be fused into v_pk_*_f32
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the direct-to-LDS loads set m0 inside inline assembly and say so in their clobber lists; clang notes that m0 is
    # a reserved register on every instantiation
    "-Wno-inline-asm",
    f"-I{os.path.join(REPO_ROOT, 'include')}",
]


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if candidate and (os.path.sep not in candidate or os.path.exists(candidate)):
            return candidate
    raise RuntimeError("hipcc not found")


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = _hipcc()
    jobs = []
    for src in sources():
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        jobs.append((src, obj))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        list(pool.map(lambda job: _run([hipcc, *HIPCC_FLAGS, "-c", job[0], "-o", job[1]]), jobs))
    # -z defs: a kernel whose host stub went missing must fail the link, not the first dlopen
    _run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wl,-z,defs", "-o", LIB_PATH,
          *[obj for _, obj in jobs]])
    if verbose:
        print(f"built {LIB_PATH} from {len(jobs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build()
