"""Parity at the full sizes of the five benchmark configurations.

The fp64 oracle is evaluated on sampled slots / query rows so that it finishes in seconds; every element of the
large configurations (3a, 3b, 4, 5) is compared with the fp32 CPU restatement of the reference's attention as well
(the tests at the end of this file); in addition, size-independent properties are checked on the whole output: split and unsplit launches
agree, the anchored and the per-query window coincide where they must, uniform attention (K = 0)
returns the mean of the visible V rows, and a launch is idempotent.
"""

import numpy as np
import pytest
import torch

from helpers import assert_close, i32, ix, u8

pytestmark = pytest.mark.gpu
H, G, D, SCALE = 8, 2, 256, 1 / 16


def randn16(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn(shape, generator=g, device="cuda", dtype=torch.float16)


def oracle_rows(q, k, v, b, rows, tds, W, Tq, stage=ix.STAGE_CAUSAL, qw=None):
    """fp64 attention of selected query rows of slot b (all heads)."""
    kv_ctx = k.shape[2]
    win, start = ix.window_size(tds, W), ix.ring_start(tds, W, kv_ctx)
    idx = (torch.arange(win, device=k.device) + start) % kv_ctx
    kl = k[b][:, idx].double().cpu().numpy()
    vl = v[b][:, idx].double().cpu().numpy()
    out = np.zeros((H, len(rows), q.shape[-1]))
    for n, i in enumerate(rows):
        lo, hi = ix.visible_range(i, tds, W, Tq, stage, qw)
        for h in range(H):
            g = h // (H // G)
            s = (kl[g, lo:hi] @ q[b, h, i].double().cpu().numpy()) * SCALE
            p = np.exp(s - s.max())
            out[h, n] = (p / p.sum()) @ vl[g, lo:hi]
    return out


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


def test_config1_single_decode_2048(fa):
    q, k, v = randn16((1, H, 1, D), 1), randn16((1, G, 2048, D), 2), randn16((1, G, 2048, D), 3)
    o = torch.empty_like(q)
    ws = torch.empty(fa.workspace_bytes(1, H, G, 1, D), dtype=torch.uint8, device="cuda")
    fa.flash_attention(q, k, v, o, i32([2048]), u8([2]), 2048, 2, scale=SCALE, workspace=ws)
    torch.cuda.synchronize()
    assert_close(o[0, :, :1].float().cpu().numpy(), oracle_rows(q, k, v, 0, [0], 2048, 2048, 1), what="config 1")


def test_config4_batched_decode_64_sequences(fa):
    B, kv_ctx = 64, 32768
    rng = np.random.default_rng(0)
    tds = rng.integers(128, 32768 + 1, B).tolist()
    win = [512 if b % 2 == 0 else kv_ctx for b in range(B)]
    q, k, v = randn16((B, H, 1, D), 1), randn16((B, G, kv_ctx, D), 2), randn16((B, G, kv_ctx, D), 3)
    phase = u8([2] * B)
    ws = torch.empty(fa.workspace_bytes(B, H, G, 1, D), dtype=torch.uint8, device="cuda")
    o = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o, i32(tds), phase, kv_ctx, 2, scale=SCALE, window_sizes=i32(win), workspace=ws)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    assert np.isfinite(got).all() and not (got == 777.0).any()
    for b in [0, 1, 2, 7, 31, 32, 62, 63, int(np.argmax(tds)), int(np.argmin(tds))]:
        assert_close(got[b], oracle_rows(q, k, v, b, [0], tds[b], win[b], 1), what=f"config 4 slot {b}")
    # property: the unsplit launch (one wave per pair) and a launch dealt to 3000 waves agree with the default
    o1 = torch.empty_like(q)
    fa.flash_attention(q, k, v, o1, i32(tds), phase, kv_ctx, 2, scale=SCALE, window_sizes=i32(win))
    ws2 = torch.empty(fa.workspace_bytes(B, H, G, 1, D, 3000), dtype=torch.uint8, device="cuda")
    o2 = torch.empty_like(q)
    fa.flash_attention(q, k, v, o2, i32(tds), phase, kv_ctx, 2, scale=SCALE, window_sizes=i32(win), workspace=ws2, num_workers=3000)
    torch.cuda.synchronize()
    for other in (o1, o2):
        d = (other.float() - o.float()).abs()
        assert bool((d <= 5e-4 + 2e-3 * o.float().abs()).all()), d.max().item()
    # the same batch as two reference-style launches: sliding-window slots on a ring of 1023 rows
    # (gemma4e.py:703-705 with t = 512), full-context slots on their own cache
    swa = [b for b in range(B) if b % 2 == 0]
    T_swa = 1023
    k_s, v_s = torch.zeros(len(swa), G, T_swa, D, device="cuda", dtype=torch.float16), torch.zeros(len(swa), G, T_swa, D, device="cuda", dtype=torch.float16)
    for n, b in enumerate(swa):  # move the last min(tds, 512) keys of slot b into the small ring at their ring rows
        n_vis = min(tds[b], 512)
        pos = torch.arange(tds[b] - n_vis, tds[b], device="cuda")
        k_s[n][:, pos % T_swa] = k[b][:, pos % kv_ctx]
        v_s[n][:, pos % T_swa] = v[b][:, pos % kv_ctx]
    o_s = torch.empty(len(swa), H, 1, D, device="cuda", dtype=torch.float16)
    fa.flash_attention(q[swa].contiguous(), k_s, v_s, o_s, i32([tds[b] for b in swa]), u8([2] * len(swa)), 512, 2, scale=SCALE)
    torch.cuda.synchronize()
    d = (o_s.float() - o[swa].float()).abs()
    assert bool((d <= 5e-4 + 2e-3 * o[swa].float().abs()).all()), d.max().item()


@pytest.mark.parametrize("qw", [None, 512], ids=["config3b_causal", "config3a_swa512"])
def test_config3_prefill_8192(fa, qw):
    S = 8192
    q, k, v = randn16((1, H, S, D), 1), randn16((1, G, S, D), 2), randn16((1, G, S, D), 3)
    o = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=SCALE, query_window=qw)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    assert np.isfinite(got).all()
    rows = [0, 1, 31, 32, 63, 64, 511, 512, 513, 1000, 4095, 4096, 8190, 8191] + np.random.default_rng(1).integers(0, S, 18).tolist()
    assert_close(got[0][:, rows], oracle_rows(q, k, v, 0, rows, S, S, S, qw=qw), what=f"config 3 qw={qw}")
    if qw is None:
        # property: a per-query window at least as long as the sequence is the plain causal mask
        o2 = torch.empty_like(q)
        fa.flash_attention(q, k, v, o2, i32([S]), u8([1]), S, 1, scale=SCALE, query_window=S)
        torch.cuda.synchronize()
        assert torch.equal(o2, o)
    # property: idempotent
    o3 = torch.empty_like(q)
    fa.flash_attention(q, k, v, o3, i32([S]), u8([1]), S, 1, scale=SCALE, query_window=qw)
    torch.cuda.synchronize()
    assert torch.equal(o3, o)


def test_config3_prefill_8192_bf16(fa):
    """Configuration 3b with bf16 q / caches / output (the other operand type of the same kernels)."""
    from helpers import ATOL_BF16, RTOL_BF16

    S = 8192
    q, k, v = (randn16(shape, seed).bfloat16() for shape, seed in (((1, H, S, D), 1), ((1, G, S, D), 2), ((1, G, S, D), 3)))
    o = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=SCALE)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    assert np.isfinite(got).all()
    rows = [0, 1, 31, 32, 511, 512, 4095, 4096, 8190, 8191] + np.random.default_rng(5).integers(0, S, 10).tolist()
    assert_close(got[0][:, rows], oracle_rows(q, k, v, 0, rows, S, S, S), atol=ATOL_BF16, rtol=RTOL_BF16, what="config 3b bf16")


def test_config3_uniform_attention_is_the_running_mean(fa):
    """K = 0: every visible key has the same weight, so row i of a causal prefill is mean(V[0..i])."""
    S = 8192
    q = randn16((1, H, S, D), 1)
    k = torch.zeros(1, G, S, D, device="cuda", dtype=torch.float16)
    v = randn16((1, G, S, D), 3)
    o = torch.empty(1, H, S, D, device="cuda", dtype=torch.float32)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=SCALE)
    torch.cuda.synchronize()
    mean = (v[0].double().cumsum(1) / torch.arange(1, S + 1, device="cuda").double()[None, :, None])
    exp = mean.repeat_interleave(H // G, 0)
    assert_close(o[0].cpu().numpy(), exp.cpu().numpy(), atol=1e-3, rtol=1e-3, what="running mean")
    # sliding window 512: windowed mean
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=SCALE, query_window=512)
    torch.cuda.synchronize()
    cs = torch.cat([torch.zeros(G, 1, D, device="cuda", dtype=torch.float64), v[0].double().cumsum(1)], 1)
    idx = torch.arange(S, device="cuda")
    lo = (idx - 511).clamp(min=0)
    wmean = (cs[:, idx + 1] - cs[:, lo]) / (idx + 1 - lo).double()[None, :, None]
    assert_close(o[0].cpu().numpy(), wmean.repeat_interleave(H // G, 0).cpu().numpy(), atol=1e-3, rtol=1e-3, what="windowed mean")


def test_head_dim_512_prefill_8192_and_decode_batch(fa):
    """Head dimension 512 (the global-attention layers) at the sizes of configurations 3 and 4: sampled rows against the
    oracle, uniform attention as the running mean, split against unsplit decode."""
    S, D5 = 8192, 512
    q, k, v = randn16((1, H, S, D5), 1), randn16((1, G, S, D5), 2), randn16((1, G, S, D5), 3)
    o = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=SCALE)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    assert np.isfinite(got).all()
    rows = [0, 1, 31, 32, 127, 128, 4095, 4096, 8190, 8191] + np.random.default_rng(2).integers(0, S, 10).tolist()
    assert_close(got[0][:, rows], oracle_rows(q, k, v, 0, rows, S, S, S), what="D=512 prefill 8192")
    o32 = torch.empty(1, H, S, D5, device="cuda", dtype=torch.float32)
    fa.flash_attention(q, torch.zeros_like(k), v, o32, i32([S]), u8([1]), S, 1, scale=SCALE)
    torch.cuda.synchronize()
    mean = v[0].double().cumsum(1) / torch.arange(1, S + 1, device="cuda").double()[None, :, None]
    assert_close(o32[0].cpu().numpy(), mean.repeat_interleave(H // G, 0).cpu().numpy(), atol=1e-3, rtol=1e-3, what="running mean")
    del q, k, v, o, o32
    B, kv_ctx = 32, 32768
    tds = np.random.default_rng(3).integers(128, kv_ctx + 1, B).tolist()
    q, k, v = randn16((B, H, 1, D5), 1), randn16((B, G, kv_ctx, D5), 2), randn16((B, G, kv_ctx, D5), 3)
    o = torch.full_like(q, 777.0)
    ws = torch.empty(fa.workspace_bytes(B, H, G, 1, D5), dtype=torch.uint8, device="cuda")
    fa.flash_attention(q, k, v, o, i32(tds), u8([2] * B), kv_ctx, 2, scale=SCALE, workspace=ws)
    o1 = torch.empty_like(q)
    fa.flash_attention(q, k, v, o1, i32(tds), u8([2] * B), kv_ctx, 2, scale=SCALE)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    for b in [0, 5, 31, int(np.argmax(tds)), int(np.argmin(tds))]:
        assert_close(got[b], oracle_rows(q, k, v, b, [0], tds[b], kv_ctx, 1), what=f"D=512 decode slot {b}")
    d = (o1.float() - o.float()).abs()
    assert bool((d <= 5e-4 + 2e-3 * o.float().abs()).all()), d.max().item()


def test_config2_causal_prefill_2048_all_rows(fa):
    S = 2048
    q, k, v = randn16((1, H, S, D), 1), randn16((1, G, S, D), 2), randn16((1, G, S, D), 3)
    o = torch.empty_like(q)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=SCALE)
    torch.cuda.synchronize()
    from helpers import oracle

    assert_close(o.float().cpu().numpy(), oracle(q, k, v, [S], [1], S, 1, scale=SCALE), what="config 2")


def test_config5_mixed_step_two_launches_per_layer(fa):
    """32 decode slots + one 512-token chunk on a 16384-token context; a sliding-window and a global layer."""
    B, t, ctx = 33, 512, 16384
    rng = np.random.default_rng(0)
    tds = rng.integers(1024, 16384 + 1, 32).tolist() + [ctx + t]
    phase = [2] * 32 + [1]
    qp, qd = randn16((B, H, t, D), 1), randn16((B, H, 1, D), 2)
    ws = torch.empty(fa.workspace_bytes(B, H, G, 1, D), dtype=torch.uint8, device="cuda")
    for name, W, T in (("swa", 512, 512 + t - 1), ("global", 32768, 32768 + t - 1)):
        k, v = randn16((B, G, T, D), 3), randn16((B, G, T, D), 4)
        op, od = torch.full_like(qp, 777.0), torch.full_like(qd, 777.0)
        fa.flash_attention(qp, k, v, op, i32(tds), u8(phase), W, 1, scale=SCALE)
        fa.flash_attention(qd, k, v, od, i32(tds), u8(phase), W, 2, scale=SCALE, workspace=ws)
        torch.cuda.synchronize()
        assert (op[:32] == 777.0).all() and (od[32] == 777.0).all()  # each launch touches its own phase only
        rows = [0, 1, 63, 64, 255, 256, 510, 511]
        assert_close(op[32].float().cpu().numpy()[:, rows], oracle_rows(qp, k, v, 32, rows, tds[32], W, t), what=f"{name} chunk")
        for b in (0, 5, 17, 31):
            assert_close(od[b].float().cpu().numpy(), oracle_rows(qd, k, v, b, [0], tds[b], W, 1), what=f"{name} decode slot {b}")


# ---- every output element of the large configurations against the CPU restatement of the reference ----------------
# The fp64 oracle above is affordable on sampled rows only.  The fp32 torch-CPU restatement of the reference's own
# attention (scripts/reference_impl.py:434-443, oracle.attention_ref.attention_cpu_baseline, query rows in blocks of
# 512 so that the score tensor stays small) finishes the full configurations in seconds to tens of seconds, so every
# element is compared with it as well, at the north-star tolerance widened by 2e-5 for the fp32 sums of the CPU path
# itself (up to 32768 terms of magnitude <= 1 per row).
CPU_FP32_SLACK = 2e-5


def _cpu_reference(q, k, v, tds, phase, W, phase_id, **kw):
    from oracle import attention_ref as ar

    torch.set_num_threads(min(torch.get_num_threads(), 16))
    return ar.attention_cpu_baseline(q.cpu(), k.cpu(), v.cpu(), tds, phase, W, phase_id, scale=SCALE, row_block=512, **kw).numpy()


@pytest.mark.parametrize("qw", [None, 512], ids=["config3b_causal", "config3a_swa512"])
def test_config3_prefill_8192_every_element(fa, qw):
    S = 8192
    q, k, v = randn16((1, H, S, D), 1), randn16((1, G, S, D), 2), randn16((1, G, S, D), 3)
    o = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=SCALE, query_window=qw)
    torch.cuda.synchronize()
    ref = _cpu_reference(q, k, v, [S], [1], S, 1, query_window=qw)
    assert_close(o.float().cpu().numpy(), ref, atol=2e-3 + CPU_FP32_SLACK, what=f"config 3 qw={qw}, all {H * S} rows")


def test_config4_batched_decode_every_element(fa):
    B, kv_ctx = 64, 32768
    rng = np.random.default_rng(0)
    tds = rng.integers(128, 32768 + 1, B).tolist()
    win = [512 if b % 2 == 0 else kv_ctx for b in range(B)]
    q, k, v = randn16((B, H, 1, D), 1), randn16((B, G, kv_ctx, D), 2), randn16((B, G, kv_ctx, D), 3)
    ws = torch.empty(fa.workspace_bytes(B, H, G, 1, D), dtype=torch.uint8, device="cuda")
    o = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o, i32(tds), u8([2] * B), kv_ctx, 2, scale=SCALE, window_sizes=i32(win), workspace=ws)
    torch.cuda.synchronize()
    ref = _cpu_reference(q, k, v, tds, [2] * B, kv_ctx, 2, window_sizes=win)
    assert_close(o.float().cpu().numpy(), ref, atol=2e-3 + CPU_FP32_SLACK, what="config 4, all 64 slots")


def test_config5_mixed_step_one_launch_every_element(fa):
    """Configuration 5 at full size through the one-launch mixed mode, both layer kinds, every element of both halves."""
    B, t, ctx = 33, 512, 16384
    rng = np.random.default_rng(0)
    tds = rng.integers(1024, 16384 + 1, 32).tolist() + [ctx + t]
    phase = [2] * 32 + [1]
    qp, qd = randn16((B, H, t, D), 1), randn16((B, H, 1, D), 2)
    for W, T in ((32768, 32768 + t - 1), (512, 512 + t - 1)):
        k, v = randn16((B, G, T, D), 3), randn16((B, G, T, D), 4)
        ws = torch.empty(fa.mixed_workspace_bytes(B, H, G, t, 1, D, T, W), dtype=torch.uint8, device="cuda")
        op, od = torch.full_like(qp, 777.0), torch.full_like(qd, 777.0)
        fa.flash_attention(qp, k, v, op, i32(tds), u8(phase), W, 1, scale=SCALE, workspace=ws, decode_q=qd, decode_o=od)
        torch.cuda.synchronize()
        ref_p = _cpu_reference(qp[32:], k[32:], v[32:], tds[32:], [1], W, 1)
        assert_close(op[32:].float().cpu().numpy(), ref_p, atol=2e-3 + CPU_FP32_SLACK, what=f"config 5 chunk, W={W}")
        assert (op[:32] == 777.0).all()
        ref_d = _cpu_reference(qd, k, v, tds, phase, W, 2)
        assert_close(od[:32].float().cpu().numpy(), ref_d[:32], atol=2e-3 + CPU_FP32_SLACK, what=f"config 5 decode, W={W}")
        assert (od[32:] == 777.0).all()
        del k, v
