"""The share-out of decode tiles over workers (g4b::TileShares, attn_decode.hpp) brute-forced on the CPU: the workers
compute their ranges with begin(), the merge kernel finds the workers of a pair with owner(), and a disagreement between
the two would read partial rows nobody wrote.  The header's own code is compiled host-only (no device pass, no GPU)."""

import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def test_begin_and_owner_agree(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(hipcc).exists():
        pytest.skip("hipcc not found")
    obj, exe = tmp_path / "check.o", tmp_path / "check"
    subprocess.run([hipcc, "--cuda-host-only", "-O2", "-std=c++17", "-fPIE", "-Wno-inline-asm", "-I", str(ROOT / "g4b_amd" / "csrc"), "-c",
                    str(ROOT / "tests" / "tile_shares_check.hip"), "-o", str(obj)], check=True, capture_output=True)
    subprocess.run(["g++", str(obj), "-o", str(exe)], check=True, capture_output=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-2000:]
    lines = res.stdout.strip().splitlines()
    assert lines[-1].endswith(" 0 bad") and int(lines[-1].split()[0]) > 1_000_000, res.stdout[-500:]
    even, odd = (int(x) for x in (lines[-2].split()[5], lines[-2].split()[7]))
    assert even > odd  # the weighting is on at the benchmark's size
