"""The plain fp32 kernel that serves what the tuned kernels are not built for: head dimensions other than
128 / 256 / 512, query-head groups that do not divide a workgroup's rows, an fp32 KV cache (the reference's
G4B_DTKV_FP32 switch, g4b/models/gemma4e.py:32) and STAGE_ON_BAND on its own (g4b/kernels/fa2.py:15,399-435).

Every case is compared with the fp64 oracle on the values the GPU sees, at the fp16 tolerance (the path computes in
fp32, so only the output's rounding to its dtype separates it from the oracle); off-phase slots must stay untouched.
"""

import numpy as np
import pytest
import torch

from helpers import ATOL_BF16, RTOL_BF16, assert_close, i32, ix, make_case, oracle, u8

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


def run_and_check(fa, q, k, v, o, tds, phase_arr, W, phase, tol=None, **kw):
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase_arr), W, phase, **kw)
    torch.cuda.synchronize()
    okw = {n: kw[n] for n in ("stage", "scale", "query_window", "on_band_block") if n in kw}
    if "window_sizes" in kw:
        okw["window_sizes"] = [int(x) for x in kw["window_sizes"].cpu()]
    ref = oracle(q, k, v, tds, phase_arr, W, phase, **okw)
    got = o.float().cpu().numpy()
    for b in range(q.shape[0]):
        if phase_arr[b] == phase:
            assert_close(got[b], ref[b], what=f"slot {b}", **(tol or {}))
        else:
            assert (got[b] == 777.0).all(), f"off-phase slot {b} was written"


@pytest.mark.parametrize("D", [8, 64, 96, 160, 320, 1024])
@pytest.mark.parametrize("Tq", [1, 40])
def test_other_head_dims(fa, D, Tq):
    print(f"generic D={D} Tq={Tq}", flush=True)
    B, H, G, kv_ctx, W = 4, 6, 2, 300, 200
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=D + Tq)
    # beyond the ring (wraps), short, an off-phase slot, an empty in-phase slot (Tq = 1 only: a chunk needs tds >= Tq)
    tds = [777, 3 + Tq, 150, 0 if Tq == 1 else Tq]
    phase_arr = [1, 1, 0, 1]
    run_and_check(fa, q, k, v, o, tds, phase_arr, W, 1, scale=D**-0.5)


@pytest.mark.parametrize("H,G", [(3, 1), (10, 2), (7, 7), (24, 2)])
def test_group_sizes_that_do_not_divide_a_workgroups_rows(fa, H, G):
    """Prefill-shaped launches with H/G of 3, 5, 1 and 12 at head dimension 256 (1 divides: the tuned kernel runs; the
    others take the plain kernel)."""
    print(f"generic H={H} G={G}", flush=True)
    B, Tq, D, kv_ctx = 2, 70, 256, 400
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=H)
    run_and_check(fa, q, k, v, o, [333, 70], [2, 2], kv_ctx, 2, scale=1 / 16)


@pytest.mark.parametrize("D", [128, 256, 512])
@pytest.mark.parametrize("Tq", [1, 130])
def test_fp32_cache(fa, D, Tq):
    """G4B_DTKV_FP32: fp32 caches under the engine's fp32 q / o views, scale 1.0 on normed-size values."""
    print(f"generic fp32 cache D={D} Tq={Tq}", flush=True)
    B, H, G, kv_ctx = 3, 8, 2, 500 + Tq
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=7 * D + Tq, dtype=torch.float32, engine_layout=True)
    q.mul_(0.25)  # |q.k| around D/4 * ... keeps exp2 arguments of scale 1.0 in a sane range
    tds = [kv_ctx + 60, 200 + Tq, 90 + Tq]
    run_and_check(fa, q, k, v, o, tds, [1, 0, 1], kv_ctx, 1, scale=1.0 / 8, use_fp32_dot=True,
                  tol=dict(atol=2e-5, rtol=2e-5))


@pytest.mark.parametrize("block", [1, 16, 64, 128])
@pytest.mark.parametrize("D", [128, 256])
def test_on_band_stage_alone(fa, block, D):
    print(f"generic on-band block={block} D={D}", flush=True)
    B, H, G, Tq, kv_ctx, W = 3, 8, 2, 256, 700, 600
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=block)
    tds = [256, 1500, 400]
    run_and_check(fa, q, k, v, o, tds, [1, 1, 2], W, 1, stage=ix.STAGE_ON_BAND, on_band_block=block, scale=D**-0.5)
    # what the stage means, independently of the oracle: block 1 = every query sees its own key only, so o is that V row
    if block == 1:
        got = o.float().cpu().numpy()
        vv = v.float().cpu().numpy()
        for b in (0, 1):
            win = min(tds[b], W)
            rows = [ix.ring_row(tds[b], W, kv_ctx, win - Tq + i) for i in range(Tq)]
            for h in range(H):
                np.testing.assert_allclose(got[b, h], vv[b, h // (H // G)][rows], atol=1e-3)


def test_on_band_decode_and_missing_block(fa):
    B, H, G, D, kv_ctx = 2, 8, 2, 256, 128
    q, k, v, o = make_case(B, H, G, 1, D, kv_ctx, seed=3)
    run_and_check(fa, q, k, v, o, [100, 300], [2, 2], kv_ctx, 2, stage=ix.STAGE_ON_BAND, on_band_block=32)
    with pytest.raises(ValueError, match="on_band_block"):
        fa.flash_attention(q, k, v, o, i32([100, 300]), u8([2, 2]), kv_ctx, 2, stage=ix.STAGE_ON_BAND)


def test_generic_path_bf16_per_slot_windows_and_query_window(fa):
    B, H, G, Tq, D, kv_ctx = 3, 9, 3, 50, 192, 260
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=11, dtype=torch.bfloat16, q_dtype=torch.float32)
    win = i32([260, 64, 100])
    run_and_check(fa, q, k, v, o, [500, 120, 50], [1, 1, 1], kv_ctx, 1, scale=0.07, window_sizes=win, query_window=17,
                  tol=dict(atol=2e-5, rtol=2e-5))
    o16 = torch.full_like(o, 777.0, dtype=torch.bfloat16)
    run_and_check(fa, q, k, v, o16, [500, 120, 50], [1, 1, 1], kv_ctx, 1, scale=0.07, stage=ix.STAGE_FULL,
                  tol=dict(atol=ATOL_BF16, rtol=RTOL_BF16))


def test_generic_path_through_the_static_scratch_entry_and_plans(fa):
    """Shapes of the plain kernel need no scratch: the allocation-free entry point and a bound plan serve them too."""
    B, H, G, Tq, D, kv_ctx = 2, 4, 2, 33, 72, 90
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=13)
    tds, ph = i32([80, 33]), u8([1, 1])
    plan = fa.plan_flash_attention(q, k, v, o, tds, ph, kv_ctx, 1, scale=0.1, workspace="static")
    plan.launch()
    torch.cuda.synchronize()
    ref = oracle(q, k, v, [80, 33], [1, 1], kv_ctx, 1, scale=0.1)
    assert_close(o.float().cpu().numpy(), ref)


def test_fp32_cache_engine_step(fa):
    """G4B_DTKV_FP32 end to end for one prefill chunk and one decode step: K append, V append with the fused weightless
    RMSNorm (g4b/kernels/add_kv_to_cache.py:146-159) into fp32 rings, attention on them."""
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache

    B, H, G, D, t, W = 2, 8, 2, 256, 24, 40
    T = W + t - 1
    eps = 1e-6
    gen = torch.Generator(device="cpu").manual_seed(5)
    k_cache = torch.zeros(B, G, T, D, device="cuda")
    v_cache = torch.zeros(B, G, T, D, device="cuda")
    ctx = [0, 0]
    streams = [[np.zeros((G, 0, D)), np.zeros((G, 0, D))] for _ in range(B)]
    for t_now, phase_id in ((t, 1), (t, 1), (1, 2), (1, 2)):
        q = torch.randn(B, t_now, H, D, generator=gen).cuda().permute(0, 2, 1, 3) * 0.25
        kx = torch.randn(B, t_now, G, D, generator=gen).cuda().permute(0, 2, 1, 3)
        vx = torch.randn(B, t_now, G, D, generator=gen).cuda().permute(0, 2, 1, 3)
        rs = (vx * vx).sum(-1)
        o = torch.full((B, t_now, H, D), 777.0, device="cuda").permute(0, 2, 1, 3)
        offs, tds, ph = i32(ctx), i32([c + t_now for c in ctx]), u8([phase_id] * B)
        add_kv_to_cache(kx, k_cache, offs, eps, user_phase=ph, phase=phase_id)
        add_kv_to_cache(vx, v_cache, offs, eps, rs, user_phase=ph, phase=phase_id)
        fa.flash_attention(q, k_cache, v_cache, o, tds, ph, W, phase_id, use_fp32_dot=True, scale=1 / 8)
        torch.cuda.synchronize()
        vn = vx.double() * torch.rsqrt(rs.double() / D + eps)[..., None]
        for b in range(B):
            streams[b][0] = np.concatenate([streams[b][0], kx[b].double().cpu().numpy()], 1)
            streams[b][1] = np.concatenate([streams[b][1], vn[b].cpu().numpy()], 1)
            n = ctx[b] + t_now
            lo = max(n - W, 0)
            ks = np.repeat(streams[b][0][:, lo:n], H // G, 0)
            vs = np.repeat(streams[b][1][:, lo:n], H // G, 0)
            s = np.einsum("htd,hnd->htn", q[b].double().cpu().numpy(), ks) / 8
            s = np.where(np.arange(n - t_now, n)[:, None] < np.arange(lo, n)[None, :], -np.inf, s)
            p = np.exp(s - s.max(-1, keepdims=True))
            ref = np.einsum("htn,hnd->htd", p / p.sum(-1, keepdims=True), vs)
            assert_close(o[b].cpu().numpy(), ref, atol=2e-5, rtol=2e-5, what=f"slot {b} at ctx {ctx[b]}")
        ctx = [c + t_now for c in ctx]
