"""Build libg4b_attn.so (HIP kernels for gfx950 + the C ABI) in-tree with hipcc.

    python -m g4b_amd.build            # compile every translation unit, link
    python -m g4b_amd.build --verbose  # also print the per-kernel register / LDS usage remarks

The shared library lands next to this file so that it travels with the source tree; nothing
is installed.  hipcc cross-compiles for gfx950 without a GPU present.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
BUILD_DIR = PKG_DIR / "build"
LIB_PATH = PKG_DIR / "libg4b_attn.so"
ARCH = "gfx950"

SOURCES = ["api.hip", "attn_decode.hip", "attn_prefill.hip", "attn_prefill_wide.hip", "cache_ops.hip", "rope.hip"]

# packed-fp32 VALU forms are kept off: the compiler must not form v_pk_{add,mul,fma}_f32
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fno-honor-nans", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-variable", "-Wno-unknown-pragmas"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build g4b_amd")
    return exe


def _compile(src: str, verbose: bool) -> Path:
    obj = BUILD_DIR / (src + ".o")
    cmd = [hipcc(), *COMMON_FLAGS, *DEVICE_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    if verbose:
        cmd.insert(1, "-Rpass-analysis=kernel-resource-usage")
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = False, jobs: int | None = None) -> Path:
    BUILD_DIR.mkdir(exist_ok=True)
    jobs = jobs or min(len(SOURCES), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose="--verbose" in sys.argv)
    print(path)
