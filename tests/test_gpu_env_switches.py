"""The environment switches of the library (counterparts of the reference's G4B_FA_FORCE_CONFIG / G4B_FA_PRINT_CONFIG,
g4b/kernels/fa2.py:148-150,691-700) and the XCC-id probe behind the weighted work shares.  The switches are read when
the library is first used, so every case runs in a child process of its own: a batched decode launch there is
compared with the same launch without a key split, and the plan lines on stderr are read back here."""

import os
import subprocess
import sys
import textwrap

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = textwrap.dedent("""
    import sys
    import torch
    sys.path.insert(0, %r)
    sys.path.insert(0, %r)
    from g4b_amd.kernels import fa2
    from helpers import i32, make_case, u8
    B, H, G, D, W = 12, 8, 2, 256, 9000
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=4)
    tds, phase = i32([W - 611 * b for b in range(B)]), u8([2] * B)
    ws = torch.empty(fa2.workspace_bytes(B, H, G, 1, D), dtype=torch.uint8, device="cuda")
    print("workspace", ws.numel(), flush=True)
    fa2.flash_attention(q, k, v, o, tds, phase, W, 2, scale=0.0625, workspace=ws)
    o1 = torch.empty_like(o)
    fa2.flash_attention(q, k, v, o1, tds, phase, W, 2, scale=0.0625, workspace=False)
    torch.cuda.synchronize()
    d = (o.float() - o1.float()).abs().max().item()
    assert d <= 5e-4, d
    print("ok", d, flush=True)
""") % (ROOT, os.path.join(ROOT, "tests"))


def run_child(extra_env):
    env = dict(os.environ, G4B_ATTN_PRINT_PLAN="1", **extra_env)
    res = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "ok" in res.stdout
    return res.stdout, res.stderr


def test_probe_reports_the_xcc_ids_and_picks_the_shares(gpu_device):
    out, err = run_child({})
    line = next(l for l in err.splitlines() if "XCC ids of workgroups" in l)
    ids = [int(x) for x in line.split("->")[0].rsplit(":", 1)[1].split()]
    assert len(ids) == 16 and all(0 <= x < 8 for x in ids), line
    expect = "weighted" if all((x & 1) == (i & 1) for i, x in enumerate(ids)) else "equal"
    assert line.rstrip().endswith(expect + " shares"), line
    plan = next(l for l in err.splitlines() if "g4b_attn plan: decode" in l and "flat tile list" in l)
    assert f"1024 workers, {expect} shares" in plan, plan
    print(line)


def test_equal_shares_and_worker_count_can_be_forced(gpu_device):
    out, err = run_child({"G4B_ATTN_XCD_SHARES": "0", "G4B_ATTN_NUM_WORKERS": "200"})
    assert "XCC ids" not in err  # nothing was asked of the hardware
    plan = next(l for l in err.splitlines() if "g4b_attn plan: decode" in l and "flat tile list" in l)
    assert "200 workers, equal shares" in plan, plan
    # the workspace size follows the forced worker count: (200 + B*G) partial slots of 4 rows x (256 + 2) floats
    assert f"workspace {(200 + 12 * 2) * 4 * 258 * 4}" in out, out
    out, err = run_child({"G4B_ATTN_XCD_SHARES": "1"})
    plan = next(l for l in err.splitlines() if "g4b_attn plan: decode" in l and "flat tile list" in l)
    assert "1024 workers, weighted shares" in plan, plan
