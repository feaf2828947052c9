"""The walk that cuts the key tiles of a pair of query tiles into spans (g4b::pf_pair_spans, prefill_map.hpp) brute-forced
on the CPU: the workgroups of a pair each run it and keep their own span, so the spans have to tile the list exactly.
The header's own code is compiled host-only (no device pass, no GPU)."""

import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def test_spans_tile_the_list(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(hipcc).exists():
        pytest.skip("hipcc not found")
    obj, exe = tmp_path / "check.o", tmp_path / "check"
    subprocess.run([hipcc, "--cuda-host-only", "-O2", "-std=c++17", "-fPIE", "-Wno-inline-asm", "-I", str(ROOT / "g4b_amd" / "csrc"), "-c",
                    str(ROOT / "tests" / "pair_spans_check.hip"), "-o", str(obj)], check=True, capture_output=True)
    subprocess.run(["g++", str(obj), "-o", str(exe)], check=True, capture_output=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-2000:]
    last = res.stdout.strip().splitlines()[-1]
    assert last.endswith(" 0 bad") and int(last.split()[0]) > 10_000, res.stdout[-500:]
