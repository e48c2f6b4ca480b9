"""Compile the HIP sources into ``coffin_amd/libcoffin_mi355.so`` for gfx950.

Run as ``python -m coffin_amd.build``.  hipcc cross-compiles without a GPU, so
the library is built once where the sources live and shipped next to them; no
JIT cache is involved and nothing here imports torch.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
SRC_DIR = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libcoffin_mi355.so"
OBJ_DIR = SRC_DIR / "build"

ARCH = "gfx950"

#: Device and host flags.  Packed-fp32 VALU ops are switched off, division and
#: sqrt stay correctly rounded, and a*b+c is fused only where the source says
#: fmaf(): the integer paths are checked bit for bit against a CPU oracle.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-ffp-contract=off", "-fno-fast-math",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def hipcc() -> str:
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(path).exists():
        raise RuntimeError("hipcc not found; the gfx950 kernels cannot be built")
    return path


def sources() -> list[Path]:
    return sorted(SRC_DIR.glob("*.hip"))


def _compile(src: Path) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stderr[-4000:]}")
    return obj


def build_library(jobs: int | None = None, verbose: bool = False) -> Path:
    """Compile every ``csrc/*.hip`` and link the shared library; always rebuilds."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {SRC_DIR}")
    jobs = jobs or min(len(srcs), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp),
           *map(str, objs)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr[-4000:]}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build_library(verbose=True)
