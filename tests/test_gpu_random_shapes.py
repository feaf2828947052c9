"""Seeded random sweep of small launches against the fp64 oracle: every combination the boundary accepts of head
dimension, group size, query tokens, ring length, window, per-query window, stage, per-slot windows, dtypes, phases
and lengths (empty slots, lengths below / at / beyond the window, wrapped rings), split and unsplit.  The fixed cases
elsewhere follow the reference's shape list; this one looks for the corner nobody listed.
"""

import os

import numpy as np
import pytest
import torch

from helpers import ATOL_BF16, RTOL_BF16, assert_close, i32, ix, oracle, u8

pytestmark = pytest.mark.gpu

N_CASES = 240
# G4B_TEST_SEED_SHIFT=<k> runs the same sweeps on other draws (every seed below moved by k * 100000); the committed cases
# are those of shift 0
SHIFT = 100000 * int(os.environ.get("G4B_TEST_SEED_SHIFT", "0"))


def draw_case(rng):
    D = int(rng.choice([128, 256, 512]))
    R = int(rng.choice([1, 2, 4, 8, 16]))
    G = int(rng.choice([1, 2, 3]))
    H = R * G
    Tq = int(rng.choice([1, 1, 2, 3, 5, 16, 33, 64, 100]))
    kv_ctx = int(rng.integers(max(Tq, 8), 260))
    W = int(rng.integers(max(Tq, 1), kv_ctx + 1))
    B = int(rng.integers(1, 7))
    phase_id = 2 if Tq == 1 and rng.random() < 0.7 else 1
    phase = [phase_id if rng.random() < 0.75 else int(rng.choice([0, 3 - phase_id])) for _ in range(B)]
    tds = []
    for _ in range(B):
        kind = rng.integers(0, 5)
        if kind == 0:
            tds.append(0 if Tq == 1 else Tq)  # nothing but the chunk itself (or an empty decode slot)
        elif kind == 1:
            tds.append(int(rng.integers(Tq, W + 1)))  # window not yet full
        elif kind == 2:
            tds.append(W)
        else:
            tds.append(int(rng.integers(W, 4 * kv_ctx)))  # ring wrapped
    stage = ix.STAGE_FULL if rng.random() < 0.2 else ix.STAGE_CAUSAL
    qwin = int(rng.integers(1, 2 * W)) if rng.random() < 0.3 else None
    win = [int(rng.integers(Tq, W + 1)) for _ in range(B)] if rng.random() < 0.25 else None  # the caller keeps window >= Tq
    bf16 = rng.random() < 0.25
    q_f32 = rng.random() < 0.3
    engine = rng.random() < 0.5
    split = rng.random() < 0.5
    scale = float(rng.choice([1.0, 1 / 16, 0.3]))
    fp32_dot = rng.random() < 0.5  # drawn last: the cases keep the parameters they had before this switch existed
    return dict(D=D, H=H, G=G, Tq=Tq, kv_ctx=kv_ctx, W=W, B=B, phase_id=phase_id, phase=phase, tds=tds, stage=stage, qwin=qwin,
                win=win, bf16=bf16, q_f32=q_f32, engine=engine, split=split, scale=scale, fp32_dot=fp32_dot)


@pytest.mark.parametrize("n", range(N_CASES))
def test_random_launch(gpu_device, n):
    from g4b_amd.kernels import fa2

    rng = np.random.default_rng(1000 + n + SHIFT)
    c = draw_case(rng)
    print({k: v for k, v in c.items()}, flush=True)
    B, H, G, Tq, D = c["B"], c["H"], c["G"], c["Tq"], c["D"]
    cdt = torch.bfloat16 if c["bf16"] else torch.float16
    qdt = torch.float32 if c["q_f32"] else cdt
    gen = torch.Generator().manual_seed(2000 + n + SHIFT)
    if c["engine"]:
        q = torch.randn(B, Tq, H, D, generator=gen).to(qdt).cuda().permute(0, 2, 1, 3)
        o = torch.full((B, Tq, H, D), 777.0, dtype=qdt, device="cuda").permute(0, 2, 1, 3)
    else:
        q = torch.randn(B, H, Tq, D, generator=gen).to(qdt).cuda()
        o = torch.full((B, H, Tq, D), 777.0, dtype=qdt, device="cuda")
    k = torch.randn(B, G, c["kv_ctx"], D, generator=gen).to(cdt).cuda()
    v = torch.randn(B, G, c["kv_ctx"], D, generator=gen).to(cdt).cuda()
    kw = dict(stage=c["stage"], scale=c["scale"], query_window=c["qwin"])
    # use_fp32_dot=False: the kernels feed the MFMA with q rounded to the cache's 16-bit type (fa2.py:88);
    # use_fp32_dot=True: with the query as a hi + lo pair of operands, i.e. the oracle on the query as it is
    ref = oracle(q if c["fp32_dot"] else q.to(cdt), k, v, c["tds"], c["phase"], c["W"], c["phase_id"], window_sizes=c["win"], **kw)
    kw["use_fp32_dot"] = c["fp32_dot"]
    if c["win"] is not None:
        kw["window_sizes"] = i32(c["win"])
    if c["split"]:
        kw["workspace"] = torch.empty(max(fa2.workspace_bytes(B, H, G, Tq, D), 16), dtype=torch.uint8, device="cuda")
    elif (H // G) * Tq > 16:
        kw["workspace"] = False
    fa2.flash_attention(q, k, v, o, i32(c["tds"]), u8(c["phase"]), c["W"], c["phase_id"], **kw)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    tol = dict(atol=ATOL_BF16, rtol=RTOL_BF16) if c["bf16"] else {}
    sentinel = torch.tensor(777.0, dtype=qdt).float().item()  # 776 in bf16
    for b in range(B):
        if c["phase"][b] == c["phase_id"]:
            assert_close(got[b], ref[b], what=f"case {n} slot {b}", **tol)
        else:
            assert (got[b] == sentinel).all(), f"case {n}: off-phase slot {b} was written"


N_ROPE_CASES = 60


@pytest.mark.parametrize("n", range(N_ROPE_CASES))
def test_random_rope_append(gpu_device, n):
    """RoPE + q/k RMSNorm + ring append in one launch against the oracle's composition: random head dimensions (the
    value heads may differ), token counts up to the ring length, offsets that wrap, scratchpad layouts and dtypes,
    cache dtypes, phase skip."""
    from g4b_amd.kernels import rope
    from oracle import rope_ref as rr

    rng = np.random.default_rng(5000 + n + SHIFT)
    D = int(rng.choice([64, 128, 256, 512]))
    Dv = int(rng.choice([D, D, 128, 512]))
    G = int(rng.choice([1, 2, 4]))
    H = G * int(rng.choice([1, 2, 4, 8]))
    B = int(rng.integers(1, 5))
    T = int(rng.integers(1, 70))
    t = int(rng.integers(1, T + 1))
    offs = [int(rng.integers(0, 100000)) if rng.random() < 0.7 else int(rng.integers(0, T)) for _ in range(B)]
    phase_id = int(rng.choice([1, 2]))
    phase = [phase_id if rng.random() < 0.75 else 0 for _ in range(B)]
    xdt = [torch.float32, torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 4))]
    cdt = torch.float16 if rng.random() < 0.6 else torch.bfloat16
    engine = rng.random() < 0.6
    print(dict(D=D, Dv=Dv, G=G, H=H, B=B, T=T, t=t, offs=offs, phase=phase, xdt=xdt, cdt=cdt, engine=engine), flush=True)
    gen = torch.Generator().manual_seed(6000 + n + SHIFT)

    def pad(heads, d):
        if engine:
            return torch.randn(B, t, heads, d, generator=gen).to(xdt).cuda().permute(0, 2, 1, 3)
        return torch.randn(B, heads, t, d, generator=gen).to(xdt).cuda()

    q, k, v = pad(H, D), pad(G, D), pad(G, Dv)
    q_rsos, k_rsos, v_rsos = ((x.float() ** 2).sum(-1) for x in (q, k, v))
    freqs = torch.from_numpy(rr.populate_rope_frequencies_ref(D // 2, 1e6).astype(np.float32)).cuda()
    qw = (1 + 0.1 * torch.randn(D, generator=gen)).cuda()
    kw = (1 + 0.1 * torch.randn(D, generator=gen)).cuda()
    kc = torch.randn(B, G, T, D, generator=gen).to(cdt).cuda()
    vc = torch.randn(B, G, T, Dv, generator=gen).to(cdt).cuda()
    f = lambda x: x.float().cpu().numpy()  # noqa: E731
    kc_ref, vc_ref = f(kc).copy(), f(vc).copy()
    q_ref, _ = rr.rope_append_ref(f(q), f(k), f(v), f(freqs), np.array(offs), f(q_rsos), f(k_rsos), f(v_rsos), f(qw), f(kw), 1e-6,
                                  kc_ref, vc_ref, np.array(phase), phase_id)
    q0, k0 = q.clone(), k.clone()
    rope.apply_rope_and_append(q, k, v, freqs, i32(offs), q_rsos, k_rsos, v_rsos, qw, kw, 1e-6, kc, vc, u8(phase), phase_id)
    torch.cuda.synchronize()
    x_tol = {torch.float32: 2e-4, torch.float16: 4e-3, torch.bfloat16: 3e-2}[xdt]
    c_tol = 4e-3 if cdt == torch.float16 else 3e-2
    # angles of up to 1e5 radians: the oracle's fp32 angle product is the reference, as in the kernel
    np.testing.assert_allclose(f(q), q_ref, rtol=x_tol, atol=x_tol * 4)
    np.testing.assert_allclose(f(kc), kc_ref, rtol=c_tol, atol=c_tol * 4)
    np.testing.assert_allclose(f(vc), vc_ref, rtol=c_tol, atol=c_tol * 4)
    assert torch.equal(k, k0)  # the K scratchpad is left alone
    del q0


@pytest.mark.parametrize("n", range(40))
def test_random_kv_append_is_bit_exact(gpu_device, n):
    """Plain append (no normalisation): every ring row holds exactly the token the index formula puts there, in the
    cache's dtype, and nothing else moved -- for random shapes, offsets (int32 or int64), phases and layouts."""
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache

    rng = np.random.default_rng(7000 + n + SHIFT)
    D = 8 * int(rng.integers(1, 70))
    G, B = int(rng.integers(1, 5)), int(rng.integers(1, 6))
    T = int(rng.integers(1, 90))
    t = int(rng.integers(1, T + 1))
    offs = [int(rng.integers(0, 1 << 20)) for _ in range(B)]
    use_phase = rng.random() < 0.6
    phase = [1 if rng.random() < 0.7 else 2 for _ in range(B)]
    xdt = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
    cdt = [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(0, 3))]
    odt = torch.int64 if rng.random() < 0.5 else torch.int32
    gen = torch.Generator().manual_seed(8000 + n + SHIFT)
    if rng.random() < 0.5:
        x = torch.randn(B, t, G, D, generator=gen).to(xdt).cuda().permute(0, 2, 1, 3)
    else:
        x = torch.randn(B, G, t, D, generator=gen).to(xdt).cuda()
    cache0 = torch.randn(B, G, T, D, generator=gen).to(cdt).cuda()
    cache = cache0.clone()
    kw = dict(user_phase=u8(phase), phase=1) if use_phase else {}
    add_kv_to_cache(x, cache, torch.tensor(offs, dtype=odt, device="cuda"), 1e-6, **kw)
    torch.cuda.synchronize()
    exp = cache0.clone()
    for b in range(B):
        if use_phase and phase[b] != 1:
            continue
        rows = (torch.arange(t) + offs[b]) % T
        exp[b][:, rows.cuda(), :] = x[b].to(cdt)
    assert torch.equal(cache, exp), dict(D=D, G=G, B=B, T=T, t=t, offs=offs, phase=phase if use_phase else None)


N_MIXED_CASES = 60


@pytest.mark.parametrize("n", range(N_MIXED_CASES))
def test_random_mixed_launch(gpu_device, n):
    """Prefill-phase and decode-phase slots in one launch (decode_q= / decode_o=): random group sizes, chunk lengths,
    rings, windows, phases (including slots of neither phase), lengths, dtypes, with and without a workspace, against
    the oracle run once per phase."""
    from g4b_amd.kernels import fa2

    rng = np.random.default_rng(9000 + n + SHIFT)
    D = int(rng.choice([256, 512]))
    R = int(rng.choice([1, 2, 4, 8, 16]))
    G = int(rng.choice([1, 2, 3]))
    H = R * G
    t = int(rng.choice([17, 33, 64, 100, 130]))
    td = int(rng.choice([1, 1, 1, 2, 3]))
    if R * td > 16:
        td = 1
    kv_ctx = int(rng.integers(t + 8, 400))
    W = int(rng.integers(t, kv_ctx + 1)) if rng.random() < 0.7 else kv_ctx
    B = int(rng.integers(2, 8))
    phase = [int(rng.choice([1, 2, 2, 2, 0])) for _ in range(B)]
    tds = []
    for b in range(B):
        lo = t if phase[b] == 1 else td
        kind = rng.integers(0, 4)
        if kind == 0:
            tds.append(lo if phase[b] == 1 else int(rng.choice([0, td])))
        elif kind == 1:
            tds.append(int(rng.integers(lo, max(lo, W) + 1)))
        else:
            tds.append(int(rng.integers(W, 4 * kv_ctx)))
    win = [int(rng.integers(t, W + 1)) for _ in range(B)] if rng.random() < 0.25 else None
    bf16, q_f32, fp32_dot = rng.random() < 0.25, rng.random() < 0.4, rng.random() < 0.5
    with_ws = rng.random() < 0.7
    scale = float(rng.choice([1.0, 1 / 16, 0.3]))
    print(dict(D=D, H=H, G=G, t=t, td=td, kv_ctx=kv_ctx, W=W, B=B, phase=phase, tds=tds, win=win, bf16=bf16, q_f32=q_f32,
               fp32_dot=fp32_dot, with_ws=with_ws, scale=scale), flush=True)
    cdt = torch.bfloat16 if bf16 else torch.float16
    qdt = torch.float32 if q_f32 else cdt
    gen = torch.Generator().manual_seed(9500 + n + SHIFT)
    qp = torch.randn(B, t, H, D, generator=gen).to(qdt).cuda().permute(0, 2, 1, 3)
    qd = torch.randn(B, td, H, D, generator=gen).to(qdt).cuda().permute(0, 2, 1, 3)
    op = torch.full((B, t, H, D), 777.0, dtype=qdt, device="cuda").permute(0, 2, 1, 3)
    od = torch.full((B, td, H, D), 777.0, dtype=qdt, device="cuda").permute(0, 2, 1, 3)
    k = torch.randn(B, G, kv_ctx, D, generator=gen).to(cdt).cuda()
    v = torch.randn(B, G, kv_ctx, D, generator=gen).to(cdt).cuda()
    kw = dict(scale=scale, use_fp32_dot=fp32_dot)
    if win is not None:
        kw["window_sizes"] = i32(win)
    if with_ws:
        nbytes = fa2.mixed_workspace_bytes(B, H, G, t, td, D, kv_ctx, W, win is not None)
        kw["workspace"] = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    fa2.flash_attention(qp, k, v, op, i32(tds), u8(phase), W, 1, decode_q=qd, decode_o=od, **kw)
    torch.cuda.synchronize()
    rq = (lambda x: x) if fp32_dot else (lambda x: x.to(cdt))
    ref_p = oracle(rq(qp), k, v, tds, phase, W, 1, scale=scale, window_sizes=win)
    ref_d = oracle(rq(qd), k, v, tds, phase, W, 2, scale=scale, window_sizes=win)
    tol = dict(atol=ATOL_BF16, rtol=RTOL_BF16) if bf16 else {}
    sentinel = torch.tensor(777.0, dtype=qdt).float().item()
    gp, gd = op.float().cpu().numpy(), od.float().cpu().numpy()
    for b in range(B):
        if phase[b] == 1:
            assert_close(gp[b], ref_p[b], what=f"mixed case {n} chunk slot {b}", **tol)
            assert (gd[b] == sentinel).all()
        elif phase[b] == 2:
            if tds[b] >= td:  # a decode slot shorter than its query block is the caller's to avoid (scheduler.py:167-172)
                assert_close(gd[b], ref_d[b], what=f"mixed case {n} decode slot {b}", **tol)
            assert (gp[b] == sentinel).all()
        else:
            assert (gp[b] == sentinel).all() and (gd[b] == sentinel).all(), f"mixed case {n}: idle slot {b} was written"


N_GENERIC_CASES = 100


@pytest.mark.parametrize("n", range(N_GENERIC_CASES))
def test_random_launch_outside_the_tuned_shapes(gpu_device, n):
    """The same sweep over what the tuned kernels do not cover and the plain fp32 kernel serves: head dimensions that
    are any multiple of 8, group sizes with odd factors, fp32 caches, STAGE_ON_BAND alone with a random block size."""
    from g4b_amd.kernels import fa2

    rng = np.random.default_rng(9000 + n + SHIFT)
    D = int(rng.choice([8, 16, 40, 64, 72, 96, 128, 192, 256, 320, 512, 640, 1024]))
    R = int(rng.choice([1, 2, 3, 5, 6, 7, 12]))
    G = int(rng.choice([1, 2, 3]))
    H = R * G
    Tq = int(rng.choice([1, 1, 2, 7, 16, 33, 80]))
    kv_ctx = int(rng.integers(max(Tq, 8), 200))
    W = int(rng.integers(max(Tq, 1), kv_ctx + 1))
    B = int(rng.integers(1, 5))
    phase_id = int(rng.choice([1, 2]))
    phase = [phase_id if rng.random() < 0.75 else 0 for _ in range(B)]
    tds = [int(rng.choice([0 if Tq == 1 else Tq, int(rng.integers(Tq, W + 1)), W, int(rng.integers(W, 4 * kv_ctx))])) for _ in range(B)]
    stage = int(rng.choice([ix.STAGE_CAUSAL, ix.STAGE_CAUSAL, ix.STAGE_FULL, ix.STAGE_ON_BAND]))
    block = int(rng.integers(1, Tq + 4)) if stage == ix.STAGE_ON_BAND else None
    qwin = int(rng.integers(1, 2 * W)) if rng.random() < 0.3 else None
    win = [int(rng.integers(Tq, W + 1)) for _ in range(B)] if rng.random() < 0.25 else None
    cdt = [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(0, 3))]
    qdt = torch.float32 if (cdt == torch.float32 or rng.random() < 0.4) else cdt
    engine = rng.random() < 0.5
    scale = float(rng.choice([1 / 16, 0.3, D**-0.5]))
    print(dict(D=D, H=H, G=G, Tq=Tq, kv_ctx=kv_ctx, W=W, B=B, phase_id=phase_id, phase=phase, tds=tds, stage=stage, block=block,
               qwin=qwin, win=win, cdt=cdt, qdt=qdt, engine=engine, scale=scale), flush=True)
    gen = torch.Generator().manual_seed(9500 + n + SHIFT)
    if engine:
        q = torch.randn(B, Tq, H, D, generator=gen).to(qdt).cuda().permute(0, 2, 1, 3)
        o = torch.full((B, Tq, H, D), 777.0, dtype=qdt, device="cuda").permute(0, 2, 1, 3)
    else:
        q = torch.randn(B, H, Tq, D, generator=gen).to(qdt).cuda()
        o = torch.full((B, H, Tq, D), 777.0, dtype=qdt, device="cuda")
    k = torch.randn(B, G, kv_ctx, D, generator=gen).to(cdt).cuda()
    v = torch.randn(B, G, kv_ctx, D, generator=gen).to(cdt).cuda()
    kw = dict(stage=stage, scale=scale, query_window=qwin, on_band_block=block)
    ref = oracle(q, k, v, tds, phase, W, phase_id, window_sizes=win, **kw)
    if win is not None:
        kw["window_sizes"] = i32(win)
    fa2.flash_attention(q, k, v, o, i32(tds), u8(phase), W, phase_id, use_fp32_dot=True, **kw)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    tol = dict(atol=ATOL_BF16, rtol=RTOL_BF16) if cdt == torch.bfloat16 else {}
    sentinel = torch.tensor(777.0, dtype=qdt).float().item()
    for b in range(B):
        if phase[b] == phase_id:
            assert_close(got[b], ref[b], what=f"case {n} slot {b}", **tol)
        else:
            assert (got[b] == sentinel).all(), f"case {n}: off-phase slot {b} was written"


N_WORK_CASES = 40


@pytest.mark.parametrize("n", range(N_WORK_CASES))
def test_random_prefill_work_distribution(gpu_device, n):
    """Prefill launches large enough to reach every way the query tiles are dealt to workgroups: one tile each, pairs,
    pairs cut into key spans, uniform key splits, with any number of slots in phase -- against the fp64 oracle."""
    from g4b_amd.kernels import fa2

    rng = np.random.default_rng(12000 + n + SHIFT)
    D = int(rng.choice([128, 256]))
    R = int(rng.choice([4, 8, 16]))
    G = int(rng.choice([1, 2, 4])) if R < 16 else int(rng.choice([1, 2]))
    H = R * G
    Tq = int(rng.integers(200, 1101))
    kv_ctx = int(rng.integers(Tq, Tq + 500))
    W = int(rng.integers(Tq, kv_ctx + 1))
    B = int(rng.integers(1, 7))
    phase = [1 if rng.random() < 0.7 else 2 for _ in range(B)]
    phase[int(rng.integers(0, B))] = 1
    tds = [int(rng.choice([Tq, int(rng.integers(Tq, W + 1)), int(rng.integers(W, 3 * kv_ctx))])) for _ in range(B)]
    stage = ix.STAGE_FULL if rng.random() < 0.15 else ix.STAGE_CAUSAL
    qwin = int(rng.integers(50, 2 * Tq)) if rng.random() < 0.25 else None
    mode = int(rng.integers(0, 3))  # explicit workspace, the library's own scratch, no scratch
    print(dict(D=D, H=H, G=G, Tq=Tq, kv_ctx=kv_ctx, W=W, B=B, phase=phase, tds=tds, stage=stage, qwin=qwin, mode=mode), flush=True)
    gen = torch.Generator().manual_seed(13000 + n + SHIFT)
    q = torch.randn(B, Tq, H, D, generator=gen).half().cuda().permute(0, 2, 1, 3)
    o = torch.full((B, Tq, H, D), 777.0, dtype=torch.float16, device="cuda").permute(0, 2, 1, 3)
    k = torch.randn(B, G, kv_ctx, D, generator=gen).half().cuda()
    v = torch.randn(B, G, kv_ctx, D, generator=gen).half().cuda()
    kw = dict(stage=stage, scale=D**-0.5, query_window=qwin)
    ref = oracle(q, k, v, tds, phase, W, 1, **kw)
    if mode == 0:
        kw["workspace"] = torch.empty(max(fa2.workspace_bytes(B, H, G, Tq, D), 16), dtype=torch.uint8, device="cuda")
    elif mode == 2:
        kw["workspace"] = False
    fa2.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 1, **kw)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    for b in range(B):
        if phase[b] == 1:
            assert_close(got[b], ref[b], what=f"case {n} slot {b}")
        else:
            assert (got[b] == 777.0).all(), f"case {n}: off-phase slot {b} was written"
