"""Host code of the C ABI under AddressSanitizer and UndefinedBehaviorSanitizer (GPU sanitizers are not available on
this pool; the debug counterpart of the reference's ``tl.device_assert`` / ``G4B_DBG`` switches,
g4b/kernels/add_kv_to_cache.py:139, g4b/utils.py:120-123).  ``python -m g4b_amd.build --asan`` builds two programs:
the entry points and their validation driven through a few hundred refused argument blocks, with stand-in launchers
that abort if anything gets as far as a launch, and the share-out arithmetic of the decode workers.  No GPU needed."""

import os
import shutil
import subprocess
from pathlib import Path

import pytest


def test_host_code_is_clean_under_asan_and_ubsan():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(hipcc).exists():
        pytest.skip("hipcc not found")
    from g4b_amd.build import build_asan

    for exe in build_asan():
        syms = subprocess.run(["nm", str(exe)], capture_output=True, text=True).stdout
        assert "__asan_init" in syms and "__ubsan_handle" in syms, f"{exe.name} was built without the sanitizers"
        res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600,
                             env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0"))
        assert res.returncode == 0, (exe.name, res.stdout[-1500:], res.stderr[-3000:])
        last = res.stdout.strip().splitlines()[-1]
        assert last.endswith(" 0 bad") and int(last.split()[0]) > 500, last
        assert "runtime error" not in res.stderr and "AddressSanitizer" not in res.stderr, res.stderr[-3000:]
