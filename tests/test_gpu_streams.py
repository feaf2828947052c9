"""Launches on explicit streams.  The engine enqueues everything on one stream of its own (g4b/device.py:99,117-124);
here every wrapper is driven through ``utils.set_stream`` and through ``stream=`` on a ``torch.cuda.Stream`` that is
not the current one, ordered against the default stream with events, and checked against the oracle.  The static
scratch belongs to one stream at a time: a launch on a second stream while the first still has work in flight is
refused (``workspace="static"``) or runs without a key split (the default ``workspace=None``).
"""

import warnings

import numpy as np
import pytest
import torch

from helpers import assert_close, i32, ix, make_case, oracle, partials, u8

pytestmark = pytest.mark.gpu
H, G, D = 8, 2, 256


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


def test_engine_step_on_a_stream_pinned_with_set_stream(fa):
    """K append, V append, attention and advance on a side stream pinned once, as the engine does with its own
    stream; the default stream stays idle and is only joined through an event."""
    from g4b_amd.kernels import utils
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache
    from g4b_amd.kernels.advance_decode_state import advance_decode_state

    B, W, n0 = 3, 700, 650
    T = W + 1 - 1
    side = torch.cuda.Stream()
    gen = torch.Generator(device="cpu").manual_seed(5)
    k_all = torch.randn(B, G, n0 + 2, D, generator=gen).half().cuda()
    v_all = torch.randn(B, G, n0 + 2, D, generator=gen).half().cuda()
    q_all = torch.randn(2, B, H, 1, D, generator=gen).half().cuda()
    kc = torch.zeros(B, G, T, D, dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    kc[:, :, :n0] = k_all[:, :, :n0]
    vc[:, :, :n0] = v_all[:, :, :n0]
    offsets, tds = i32([n0] * B), i32([n0 + 1] * B)
    phase = u8([2, 2, 2])
    inp = torch.zeros(1, B, dtype=torch.int32, device="cuda")
    out_tok = torch.arange(B, dtype=torch.int32, device="cuda").view(B, 1).contiguous()
    outs = [torch.full((B, H, 1, D), 777.0, dtype=torch.float16, device="cuda") for _ in range(2)]
    torch.cuda.synchronize()
    utils.set_stream(side)
    try:
        for step in range(2):
            n = n0 + step
            add_kv_to_cache(k_all[:, :, n : n + 1], kc, offsets, 1e-6, user_phase=phase, phase=2)
            add_kv_to_cache(v_all[:, :, n : n + 1], vc, offsets, 1e-6, user_phase=phase, phase=2)
            fa.flash_attention(q_all[step], kc, vc, outs[step], tds, phase, W, 2, *partials(8, B, H, 1, D), scale=0.0625)
            advance_decode_state(inp, out_tok, offsets, tds, phase)
    finally:
        utils.set_stream(None)
    done = torch.cuda.Event()
    done.record(side)
    torch.cuda.current_stream().wait_event(done)
    got = [o.clone() for o in outs]  # on the default stream, after the event
    torch.cuda.synchronize()
    assert tds.tolist() == [n0 + 3] * B and offsets.tolist() == [n0 + 2] * B
    for step in range(2):
        n = n0 + step + 1
        lo = max(n - W, 0)
        ref = oracle(q_all[step], k_all[:, :, lo:n], v_all[:, :, lo:n], [n - lo] * B, [2] * B, n - lo, 2, scale=0.0625)
        assert_close(got[step].float().cpu().numpy(), ref, what=f"step {step} on the pinned stream")


def test_stream_argument_on_every_wrapper(fa):
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache

    side = torch.cuda.Stream()
    B, Tq, ctx = 2, 96, 900
    kv_ctx = ctx + Tq
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=9)
    tds, phase = [kv_ctx, Tq + 100], [1, 1]
    ws = torch.empty(fa.workspace_bytes(B, H, G, Tq, D), dtype=torch.uint8, device="cuda")
    x = torch.randn(B, G, 4, D, device="cuda").half()
    cache = torch.zeros(B, G, 16, D, dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    add_kv_to_cache(x, cache, i32([14, 3]), 1e-6, stream=side)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), kv_ctx, 1, scale=0.0625, workspace=ws, stream=side)
    fa.plan_flash_attention(q, k, v, o, i32(tds), u8(phase), kv_ctx, 1, scale=0.0625, workspace=ws).launch(stream=side.cuda_stream)
    side.synchronize()
    assert_close(o.float().cpu().numpy(), oracle(q, k, v, tds, phase, kv_ctx, 1, scale=0.0625), what="stream= launch")
    for b, off in enumerate((14, 3)):
        rows = (torch.arange(4) + off) % 16
        assert torch.equal(cache[b][:, rows], x[b])


def test_static_scratch_belongs_to_one_stream_at_a_time(fa):
    from g4b_amd import _native

    side = torch.cuda.Stream()
    B, W = 48, 16000
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=3)
    tds, phase = i32([W - 7 * b for b in range(B)]), u8([2] * B)
    parts = partials(8, B, H, 1, D)
    ref = oracle(q, k, v, [W - 7 * b for b in range(B)], [2] * B, W, 2, scale=0.0625)
    plan = fa.plan_flash_attention(q, k, v, o, tds, phase, W, 2, *parts, scale=0.0625, workspace="static")
    plan.launch()
    o2, o3 = torch.full_like(q, 777.0), torch.full_like(q, 777.0)  # filled before the queue below builds up
    torch.cuda.synchronize()
    # a few hundred launches on the default stream: milliseconds of queued work that use the array
    for _ in range(300):
        plan.launch()
    with pytest.raises(_native.ScratchBusyError, match="another stream"):
        fa.flash_attention(q, k, v, o2, tds, phase, W, 2, *parts, scale=0.0625, workspace="static", stream=side)
    # the default path does not fail: it runs without a key split on the second stream and says so once
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        fa._warned.discard("busy")
        fa.flash_attention(q, k, v, o2, tds, phase, W, 2, *parts, scale=0.0625, stream=side)
    assert any("static scratch is in use" in str(w.message) for w in caught)
    side.synchronize()
    torch.cuda.synchronize()
    assert_close(o2.float().cpu().numpy(), ref, what="fallback without a key split")
    assert_close(o.float().cpu().numpy(), ref, what="the queued launches on the first stream")
    # with the first stream idle the array changes hands
    fa.flash_attention(q, k, v, o3, tds, phase, W, 2, *parts, scale=0.0625, workspace="static", stream=side)
    side.synchronize()
    assert_close(o3.float().cpu().numpy(), ref, what="static scratch on the second stream")
    plan.launch()  # and back
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what="static scratch back on the first stream")
