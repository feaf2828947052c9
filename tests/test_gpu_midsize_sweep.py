"""Seeded random sweep of mid-size prefill-shaped launches (40 .. 5000 query tokens on 0 .. 20000 tokens of context,
one to four slots, head dimensions 128 / 256 / 512): the sizes where the launch is split over key splits, key spans or
pairs of query tiles and the merge kernel takes its wider variants.  Every case runs unsplit, split through a poisoned
workspace and through the library's static scratch; the three must agree, and sampled rows of each are held against an
fp64 reference computed on the device (on the unrounded query where use_fp32_dot asks for it).  G4B_TEST_SEED_SHIFT=<k>
runs other draws.
"""

import os

import numpy as np
import pytest
import torch

from helpers import ATOL_BF16, ATOL_F16, RTOL_BF16, RTOL_F16, ix

pytestmark = pytest.mark.gpu
N_CASES = 48
SHIFT = 100000 * int(os.environ.get("G4B_TEST_SEED_SHIFT", "0"))


def draw(rng):
    D = int(rng.choice([128, 256, 256, 512]))
    R = int(rng.choice([1, 2, 4, 4, 8]))
    G = int(rng.choice([1, 2, 2, 4]))
    Tq = int(rng.choice([rng.integers(40, 400), rng.integers(400, 1500), rng.integers(1500, 5000)]))
    ctx = int(rng.choice([0, 0, rng.integers(1, 3000), rng.integers(3000, 20000)]))
    B = int(rng.integers(1, 5))
    kv = ctx + Tq
    kv_ctx = kv + int(rng.integers(0, 100))
    qf32 = rng.random() < 0.3
    return dict(D=D, R=R, G=G, H=R * G, Tq=Tq, B=B, n_in=int(rng.integers(1, B + 1)), kv=kv, kv_ctx=kv_ctx,
                W=int(rng.choice([kv_ctx, kv_ctx, max(Tq, int(rng.integers(Tq, kv_ctx + 1)))])),
                qwin=None if rng.random() < 0.6 else int(rng.choice([64, 256, 512, 1000])),
                stage=ix.STAGE_FULL if rng.random() < 0.15 else ix.STAGE_CAUSAL, bf16=rng.random() < 0.25, qf32=qf32,
                dot32=qf32 and rng.random() < 0.6, scale=float(rng.choice([1 / 16, 0.25 / np.sqrt(D)])))


@pytest.mark.parametrize("n", range(N_CASES))
def test_random_midsize_prefill(gpu_device, n):
    from g4b_amd.kernels import fa2

    rng = np.random.default_rng(31000 + n + SHIFT)
    c = draw(rng)
    print(c, flush=True)
    B, H, G, R, Tq, D, kv_ctx, W, n_in = c["B"], c["H"], c["G"], c["R"], c["Tq"], c["D"], c["kv_ctx"], c["W"], c["n_in"]
    cdt = torch.bfloat16 if c["bf16"] else torch.float16
    qdt = torch.float32 if c["qf32"] else cdt
    g = torch.Generator(device="cuda").manual_seed(32000 + n + SHIFT)
    q = torch.randn(B, H, Tq, D, generator=g, device="cuda", dtype=torch.float32).to(qdt)
    k = torch.randn(B, G, kv_ctx, D, generator=g, device="cuda", dtype=torch.float32).to(cdt)
    v = torch.randn(B, G, kv_ctx, D, generator=g, device="cuda", dtype=torch.float32).to(cdt)
    kv = c["kv"]
    tds_list = [int(rng.choice([kv, max(Tq, kv - int(rng.integers(0, 50))), kv + int(rng.integers(0, 3 * kv_ctx))])) for _ in range(B)]
    tds = torch.tensor(tds_list, dtype=torch.int32, device="cuda")
    phases = torch.tensor([1] * n_in + [2] * (B - n_in), dtype=torch.uint8, device="cuda")
    kw = dict(scale=c["scale"], query_window=c["qwin"], stage=c["stage"], use_fp32_dot=c["dot32"])

    def run(**how):
        o = torch.full((B, H, Tq, D), 777.0, dtype=qdt, device="cuda")
        fa2.flash_attention(q, k, v, o, tds, phases, W, 1, **how, **kw)
        return o

    outs = {"unsplit": run(workspace=False), "static scratch": run()}
    need = fa2.workspace_bytes(B, H, G, Tq, D)
    if need:
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        ws.fill_(0xFF)  # reads as NaN in every type
        outs["workspace"] = run(workspace=ws)
    torch.cuda.synchronize()

    atol, rtol = (ATOL_BF16, RTOL_BF16) if c["bf16"] else (ATOL_F16, RTOL_F16)
    rows = sorted(set([0, Tq - 1] + rng.integers(0, Tq, 6).tolist()))
    for b in range(n_in):
        win, start = ix.window_size(tds_list[b], W), ix.ring_start(tds_list[b], W, kv_ctx)
        idx = (torch.arange(win, device="cuda") + start) % kv_ctx
        for i in rows:
            lo, hi = ix.visible_range(i, tds_list[b], W, Tq, c["stage"], c["qwin"])
            for h in range(0, H, max(1, H // 3)):
                # the query as the kernel takes it: unrounded with use_fp32_dot, else rounded to the cache's type
                qq = q[b, h, i].double() if (c["dot32"] or not c["qf32"]) else q[b, h, i].to(cdt).double()
                ref = torch.zeros(D, dtype=torch.float64, device="cuda")
                if hi > lo:
                    kk, vv = k[b, h // R][idx[lo:hi]].double(), v[b, h // R][idx[lo:hi]].double()
                    s = (kk @ qq) * c["scale"]
                    p = torch.exp(s - s.max())
                    ref = (p / p.sum()) @ vv
                for name, o in outs.items():
                    d = (o[b, h, i].double() - ref).abs()
                    assert bool(torch.isfinite(o[b, h, i]).all()), (name, b, h, i)
                    assert bool((d <= atol + rtol * ref.abs()).all()), (name, b, h, i, d.max().item())
    ref = outs["unsplit"][:n_in].double()
    tol = (8e-3 if c["bf16"] else 1e-3) + (2e-2 if c["bf16"] else 4e-3) * ref.abs()
    for name, o in outs.items():
        assert bool(torch.isfinite(o[:n_in]).all()), name
        assert bool((o[n_in:] == 777.0).all()), f"{name}: rows of slots that are not in phase were written"
        assert bool(((o[:n_in].double() - ref).abs() <= tol).all()), f"{name} against unsplit"


def draw_decode(rng):
    D = int(rng.choice([128, 256, 256, 512]))
    R = int(rng.choice([1, 2, 4, 4, 8, 16]))
    G = int(rng.choice([1, 2, 2, 4]))
    Tq = int(rng.choice([1, 1, 1, 2, 3, 4]))
    while R * Tq > 16:
        Tq -= 1
    kv_ctx = int(rng.choice([rng.integers(40, 600), rng.integers(600, 5000), rng.integers(5000, 20000)]))
    qf32 = rng.random() < 0.3
    return dict(D=D, R=R, G=G, H=R * G, Tq=Tq, B=int(rng.choice([1, 2, 5, 17, 33, 64])), kv_ctx=kv_ctx,
                W=int(rng.choice([kv_ctx, kv_ctx, int(rng.integers(max(Tq, 1), kv_ctx + 1)), min(kv_ctx, 512)])),
                per_slot=rng.random() < 0.3, bf16=rng.random() < 0.25, qf32=qf32, dot32=qf32 and rng.random() < 0.6,
                scale=float(rng.choice([1 / 16, 0.25 / np.sqrt(D)])), nw=int(rng.choice([0, 0, 0, 7, 100, 3000])))


@pytest.mark.parametrize("n", range(N_CASES))
def test_random_midsize_decode(gpu_device, n):
    """Decode-shaped launches of 1 .. 64 slots on rings of 40 .. 20000 rows (empty, filling, full and wrapped slots,
    slots of other phases, per-slot windows, short windows that take the one-kernel path, worker counts from 7 to 3000):
    one wave per pair, workers + merge through a poisoned workspace and through the static scratch, all against fp64
    rows."""
    from g4b_amd.kernels import fa2

    rng = np.random.default_rng(41000 + n + SHIFT)
    c = draw_decode(rng)
    print(c, flush=True)
    B, H, G, R, Tq, D, kv_ctx, W = c["B"], c["H"], c["G"], c["R"], c["Tq"], c["D"], c["kv_ctx"], c["W"]
    win_list = [int(rng.integers(Tq, W + 1)) for _ in range(B)] if c["per_slot"] else None
    tds_list = [int(rng.choice([0, Tq, int(rng.integers(Tq, W + 1)), W, int(rng.integers(W, 4 * kv_ctx))])) for _ in range(B)]
    tds_list = [t if t >= Tq or t == 0 else Tq for t in tds_list]
    ph_list = [2 if rng.random() < 0.85 else int(rng.choice([0, 1])) for _ in range(B)]
    cdt = torch.bfloat16 if c["bf16"] else torch.float16
    qdt = torch.float32 if c["qf32"] else cdt
    g = torch.Generator(device="cuda").manual_seed(42000 + n + SHIFT)
    q = torch.randn(B, H, Tq, D, generator=g, device="cuda", dtype=torch.float32).to(qdt)
    k = torch.randn(B, G, kv_ctx, D, generator=g, device="cuda", dtype=torch.float32).to(cdt)
    v = torch.randn(B, G, kv_ctx, D, generator=g, device="cuda", dtype=torch.float32).to(cdt)
    tds = torch.tensor(tds_list, dtype=torch.int32, device="cuda")
    phases = torch.tensor(ph_list, dtype=torch.uint8, device="cuda")
    win = torch.tensor(win_list, dtype=torch.int32, device="cuda") if win_list else None
    kw = dict(scale=c["scale"], use_fp32_dot=c["dot32"], window_sizes=win)

    def run(**how):
        o = torch.full((B, H, Tq, D), 777.0, dtype=qdt, device="cuda")
        fa2.flash_attention(q, k, v, o, tds, phases, W, 2, **how, **kw)
        return o

    need = fa2.workspace_bytes(B, H, G, Tq, D, c["nw"])
    ws = torch.empty(max(16, need), dtype=torch.uint8, device="cuda")
    ws.fill_(0xFF)
    outs = {"one wave per pair": run(workspace=False), "workspace": run(workspace=ws, num_workers=c["nw"])}
    if need <= fa2._native.load().g4b_static_scratch_bytes():
        outs["static scratch"] = run(workspace="static", num_workers=c["nw"])
    torch.cuda.synchronize()

    atol, rtol = (ATOL_BF16, RTOL_BF16) if c["bf16"] else (ATOL_F16, RTOL_F16)
    for b in range(B):
        if ph_list[b] != 2:
            for name, o in outs.items():
                assert bool((o[b] == 777.0).all()), f"{name}: slot {b} is not in phase and was written"
            continue
        Wb = win_list[b] if win_list else W
        wsz, start = ix.window_size(tds_list[b], Wb), ix.ring_start(tds_list[b], Wb, kv_ctx)
        idx = (torch.arange(wsz, device="cuda") + start) % kv_ctx
        for i in range(Tq):
            lo, hi = ix.visible_range(i, tds_list[b], Wb, Tq, ix.STAGE_CAUSAL, None)
            for h in range(0, H, max(1, H // 3)):
                qq = q[b, h, i].double() if (c["dot32"] or not c["qf32"]) else q[b, h, i].to(cdt).double()
                ref = torch.zeros(D, dtype=torch.float64, device="cuda")
                if hi > lo:
                    kk, vv = k[b, h // R][idx[lo:hi]].double(), v[b, h // R][idx[lo:hi]].double()
                    s = (kk @ qq) * c["scale"]
                    p = torch.exp(s - s.max())
                    ref = (p / p.sum()) @ vv
                for name, o in outs.items():
                    d = (o[b, h, i].double() - ref).abs()
                    assert bool(torch.isfinite(o[b, h, i]).all()), (name, b, h, i)
                    assert bool((d <= atol + rtol * ref.abs()).all()), (name, b, h, i, tds_list[b], Wb, d.max().item())


N_MIXED = 36


@pytest.mark.parametrize("n", range(N_MIXED))
def test_random_midsize_mixed_launch(gpu_device, n):
    """Prefill-phase and decode-phase slots in one launch at mid sizes (chunks of 64 .. 1024 tokens, 2 .. 40 slots, rings
    up to 20000 rows, both head dimensions) against the two separate launches of the same arguments, which the sweeps
    above hold against fp64 rows."""
    from g4b_amd.kernels import fa2

    rng = np.random.default_rng(51000 + n + SHIFT)
    D = int(rng.choice([256, 512]))
    R = int(rng.choice([1, 2, 4, 4, 8]))
    G = int(rng.choice([1, 2, 2, 4]))
    H = R * G
    t = int(rng.choice([64, 128, 200, 512, 1024]))
    td = 1 if R > 8 or rng.random() < 0.7 else 2
    B = int(rng.choice([2, 3, 9, 33, 40]))
    kv_ctx = int(rng.choice([rng.integers(t + 8, 3000), rng.integers(3000, 20000)]))
    W = int(rng.choice([kv_ctx, kv_ctx, int(rng.integers(t, kv_ctx + 1)), max(t, min(kv_ctx, 512))]))
    phase = [int(rng.choice([1, 2, 2, 2, 2, 0])) for _ in range(B)]
    phase[int(rng.integers(0, B))] = 1
    if 2 not in phase:
        phase[(phase.index(1) + 1) % B] = 2
    tds = [int(rng.choice([t if p == 1 else td, int(rng.integers(t, max(t, W) + 1)), int(rng.integers(W, 4 * kv_ctx))])) for p in phase]
    bf16, q_f32 = rng.random() < 0.25, rng.random() < 0.3
    fp32_dot = q_f32 and rng.random() < 0.5
    scale = float(rng.choice([1 / 16, 0.25 / np.sqrt(D)]))
    print(dict(D=D, H=H, G=G, t=t, td=td, B=B, kv_ctx=kv_ctx, W=W, phase=phase, tds=tds, bf16=bf16, q_f32=q_f32, fp32_dot=fp32_dot),
          flush=True)
    cdt = torch.bfloat16 if bf16 else torch.float16
    qdt = torch.float32 if q_f32 else cdt
    g = torch.Generator(device="cuda").manual_seed(52000 + n + SHIFT)
    qp = torch.randn(B, H, t, D, generator=g, device="cuda", dtype=torch.float32).to(qdt)
    qd = torch.randn(B, H, td, D, generator=g, device="cuda", dtype=torch.float32).to(qdt)
    k = torch.randn(B, G, kv_ctx, D, generator=g, device="cuda", dtype=torch.float32).to(cdt)
    v = torch.randn(B, G, kv_ctx, D, generator=g, device="cuda", dtype=torch.float32).to(cdt)
    tds_t = torch.tensor(tds, dtype=torch.int32, device="cuda")
    ph_t = torch.tensor(phase, dtype=torch.uint8, device="cuda")
    kw = dict(scale=scale, use_fp32_dot=fp32_dot)

    def fresh(tok):
        return torch.full((B, H, tok, D), 777.0, dtype=qdt, device="cuda")

    ref_p, ref_d = fresh(t), fresh(td)
    fa2.flash_attention(qp, k, v, ref_p, tds_t, ph_t, W, 1, workspace=False, **kw)
    fa2.flash_attention(qd, k, v, ref_d, tds_t, ph_t, W, 2, workspace=False, **kw)
    nbytes = fa2.mixed_workspace_bytes(B, H, G, t, td, D, kv_ctx, W)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    for how in ("workspace", "no workspace"):
        ws.fill_(0xFF)
        op, od = fresh(t), fresh(td)
        fa2.flash_attention(qp, k, v, op, tds_t, ph_t, W, 1, decode_q=qd, decode_o=od, workspace=ws if how == "workspace" else False, **kw)
        torch.cuda.synchronize()
        for got, ref, what in ((op, ref_p, "chunk"), (od, ref_d, "decode")):
            assert bool(torch.isfinite(got).all()), (how, what)
            d = (got.double() - ref.double()).abs()
            tol = (8e-3 if bf16 else 1e-3) + (2e-2 if bf16 else 4e-3) * ref.double().abs()
            assert bool((d <= tol).all()), (how, what, d.max().item())
