"""Ahead-of-time build of the HIP kernels into ``ssm_amd/lib/libssm_amd.so``.

Run as ``python -m ssm_amd.build``.  The library exposes only the C ABI of
``include/ssm_amd.h``; it does not link against torch.

A second library, ``libssm_amd_testhooks.so``, is linked from the same objects
except that the sources which pick between kernels are compiled once more with
``-DSSM_TEST_HOOKS`` (``include/ssm_amd_testing.h``): the test suite uses it to
run a chosen kernel where the shipped library would pick another.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = PKG / "lib" / "obj"
LIB = PKG / "lib" / "libssm_amd.so"
HOOKS_LIB = PKG / "lib" / "libssm_amd_testhooks.so"
# the sources that read a kernel selector (SSM_RESERVED) or record the kernel taken
HOOKED = ("scan_fwd.hip", "scan_bwd.hip", "dscan_bwd.hip", "ssd.hip")

ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-cuda-version",
]


def hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, extra: list[str], suffix: str = "") -> Path:
    obj = OBJ / (src.stem + suffix + ".o")
    cmd = [hipcc(), *FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True, extra: list[str] | None = None, jobs: int | None = None) -> Path:
    """Compile every ``csrc/*.hip`` for gfx950 and link the shared library."""
    OBJ.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError("no HIP sources found")
    jobs = jobs or min(8, len(srcs))
    extra = extra or []
    hooked = [s for s in srcs if s.name in HOOKED]
    tasks = [(s, extra, "") for s in srcs] + [(s, [*extra, "-DSSM_TEST_HOOKS"], "_hooks") for s in hooked]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        done = list(pool.map(lambda t: _compile(*t), tasks))
    objs, hook_objs = done[:len(srcs)], dict(zip((s.name for s in hooked), done[len(srcs):]))
    for lib, parts in ((LIB, objs), (HOOKS_LIB, [hook_objs.get(s.name, o) for s, o in zip(srcs, objs)])):
        cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(lib), *map(str, parts)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB} and {HOOKS_LIB.name} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build(extra=sys.argv[1:])
