"""Pins ``oracle.attention_ref`` without retyping its formulas.

* library opinion: ``torch.nn.functional.scaled_dot_product_attention`` on CPU with an explicit
  boolean mask built from absolute positions of a token stream appended to the ring;
* exact special cases: all-zero K returns the mean of the visible V rows (with one-hot V rows
  that reads back the visible set itself); one dominant key returns that V row;
* two independent codings of ``scripts/reference_impl.py:421-443`` agree
  (``attention_ref`` masks, ``retrieve_ref_torch`` slices like the reference);
* the tile-by-tile Triton restatement (additive -1e6 masks, exp2, splits + merge) equals the
  dense form;
* KV append against the reference test's one-liner at its shapes.
"""

import numpy as np
import pytest
import torch

from oracle import attention_ref as ar
from oracle import index_spec as ix


def stream_case(rng, B, H, G, Tq, D, kv_ctx, W, tds_list, dtype=np.float64):
    """Build ring caches by appending a per-slot token stream; also return the streams."""
    q = rng.standard_normal((B, H, Tq, D)).astype(dtype)
    k_cache = rng.standard_normal((B, G, kv_ctx, D)).astype(dtype)  # stale garbage first
    v_cache = rng.standard_normal((B, G, kv_ctx, D)).astype(dtype)
    streams = []
    for b in range(B):
        tds = tds_list[b]
        ks = rng.standard_normal((G, tds, D)).astype(dtype)
        vs = rng.standard_normal((G, tds, D)).astype(dtype)
        for p in range(tds):
            k_cache[b, :, p % kv_ctx] = ks[:, p]
            v_cache[b, :, p % kv_ctx] = vs[:, p]
        streams.append((ks, vs))
    return q, k_cache, v_cache, streams


def sdpa_positions(q_b, ks, vs, tds, W, stage, scale, query_window=None):
    """Expected output of one slot from absolute positions, via torch SDPA (fp64, CPU)."""
    H, Tq, D = q_b.shape
    G = ks.shape[0]
    lo = max(tds - W, 0)
    k_pos = torch.arange(lo, tds)[None, :]
    q_pos = torch.arange(tds - Tq, tds)[:, None]
    allow = torch.ones((Tq, tds - lo), dtype=torch.bool) if stage == ix.STAGE_FULL else ~(q_pos < k_pos)
    if query_window is not None:
        allow = allow & ~(q_pos - k_pos >= query_window)
    k = torch.from_numpy(ks[:, lo:tds]).repeat_interleave(H // G, 0)
    v = torch.from_numpy(vs[:, lo:tds]).repeat_interleave(H // G, 0)
    out = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q_b)[None], k[None], v[None], attn_mask=allow[None, None], scale=scale
    )
    return out[0].numpy()


CASES = [
    # B, H, G, Tq, D, kv_ctx, W, tds list
    (2, 8, 2, 1, 16, 17, 17, [17, 34]),  # wrap case tds = W + 17 (test_fa2.py:286-290)
    (3, 8, 2, 1, 32, 23, 9, [1, 9, 40]),  # sliding window decode, ring wrap
    (2, 4, 4, 5, 8, 21, 16, [5, 37]),  # chunk on context, R = 1
    (2, 8, 2, 7, 16, 17, 11, [7, 30]),  # chunk, anchored window, ring = W + t - 1
    (1, 16, 4, 12, 8, 12, 12, [12]),  # one-shot causal prefill
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("stage", [ix.STAGE_CAUSAL, ix.STAGE_FULL])
@pytest.mark.parametrize("scale", [1.0, 0.25])
def test_dense_oracle_matches_sdpa_on_positions(case, stage, scale):
    B, H, G, Tq, D, kv_ctx, W, tds_list = case
    rng = np.random.default_rng(hash((case[:7], stage)) % 2**32)
    q, kc, vc, streams = stream_case(rng, B, H, G, Tq, D, kv_ctx, W, tds_list)
    phase = np.full(B, ix.PHASE_PREFILL)
    got = ar.attention_ref(q, kc, vc, tds_list, phase, W, ix.PHASE_PREFILL, stage=stage, scale=scale)
    for b in range(B):
        exp = sdpa_positions(q[b], *streams[b], tds_list[b], W, stage, scale)
        np.testing.assert_allclose(got[b], exp, rtol=1e-10, atol=1e-12)


def test_per_query_window_matches_sdpa_on_positions():
    rng = np.random.default_rng(7)
    B, H, G, Tq, D, kv_ctx, W = 2, 8, 2, 24, 8, 24, 24
    tds_list = [24, 24]
    q, kc, vc, streams = stream_case(rng, B, H, G, Tq, D, kv_ctx, W, tds_list)
    phase = np.full(B, 1)
    for qw in (1, 5, 24, 100):
        got = ar.attention_ref(q, kc, vc, tds_list, phase, W, 1, scale=0.5, query_window=qw)
        for b in range(B):
            exp = sdpa_positions(q[b], *streams[b], 24, W, ix.STAGE_CAUSAL, 0.5, qw)
            np.testing.assert_allclose(got[b], exp, rtol=1e-10, atol=1e-12)


def test_zero_keys_read_back_the_visible_set_exactly():
    """K = 0 gives uniform weights; one-hot V rows turn the output into indicator / count."""
    B, H, G, Tq, kv_ctx, W = 1, 4, 2, 3, 13, 8
    D = kv_ctx
    for tds in (3, 8, 11, 20, 27):
        q = np.ones((B, H, Tq, D))
        kc = np.zeros((B, G, kv_ctx, D))
        vc = np.zeros((B, G, kv_ctx, D))
        for r in range(kv_ctx):
            vc[0, :, r, r] = 1.0  # V row r = e_r: output[d] = [row d visible] / count
        got = ar.attention_ref(q, kc, vc, [tds], [1], W, 1)
        ring = [None] * kv_ctx
        for p in range(tds):
            ring[p % kv_ctx] = p
        for i in range(Tq):
            q_pos = tds - Tq + i
            vis_rows = [r for r in range(kv_ctx) if ring[r] is not None and max(tds - W, 0) <= ring[r] <= q_pos]
            exp = np.zeros(D)
            exp[vis_rows] = 1.0 / len(vis_rows)
            for h in range(H):
                np.testing.assert_allclose(got[0, h, i], exp, rtol=0, atol=1e-15)


def test_dominant_key_returns_its_value_row():
    rng = np.random.default_rng(3)
    B, H, G, Tq, D, kv_ctx, W, tds = 1, 4, 2, 1, 8, 16, 16, 10
    q = np.zeros((B, H, Tq, D))
    q[..., 0] = 1.0
    kc = np.zeros((B, G, kv_ctx, D))
    vc = rng.standard_normal((B, G, kv_ctx, D))
    kc[0, :, 6, 0] = 800.0  # position 6 dominates
    got = ar.attention_ref(q, kc, vc, [tds], [2], W, 2)
    for h in range(H):
        np.testing.assert_allclose(got[0, h, 0], vc[0, h // 2, 6], rtol=0, atol=1e-12)


def test_off_phase_slots_untouched_and_empty_rows_reported():
    rng = np.random.default_rng(4)
    B, H, G, Tq, D, kv_ctx, W = 4, 4, 2, 2, 8, 9, 9
    q = rng.standard_normal((B, H, Tq, D))
    kc = rng.standard_normal((B, G, kv_ctx, D))
    vc = rng.standard_normal((B, G, kv_ctx, D))
    out = np.full((B, H, Tq, D), 123.0)
    o, empty = ar.attention_ref(q, kc, vc, [5, 5, 0, 1], [1, 2, 1, 1], W, 1, out=out, return_empty_rows=True)
    assert np.all(o[1] == 123.0)  # decode-phase slot skipped by a prefill launch
    assert not empty[0].any()
    assert empty[2].all() and np.all(o[2] == 0)  # tds = 0: no keys
    assert empty[3].tolist() == [True, False]  # tds < Tq: first query has no key


@pytest.mark.parametrize("case", CASES)
def test_reference_style_slicing_equals_masked_dense(case):
    B, H, G, Tq, D, kv_ctx, W, tds_list = case
    rng = np.random.default_rng(11)
    q, kc, vc, _ = stream_case(rng, B, H, G, Tq, D, kv_ctx, W, tds_list, dtype=np.float32)
    phase = [1] * B
    dense = ar.attention_ref(q, kc, vc, tds_list, phase, W, 1, scale=0.3)
    sliced = ar.attention_cpu_baseline(
        torch.from_numpy(q), torch.from_numpy(kc), torch.from_numpy(vc), tds_list, phase, W, 1, scale=0.3
    ).numpy()
    np.testing.assert_allclose(sliced, dense, rtol=2e-5, atol=2e-6)
    blocked = ar.attention_cpu_baseline(
        torch.from_numpy(q), torch.from_numpy(kc), torch.from_numpy(vc), tds_list, phase, W, 1, scale=0.3, row_block=3
    ).numpy()
    np.testing.assert_allclose(blocked, dense, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("stage", [ix.STAGE_CAUSAL, ix.STAGE_FULL, ix.STAGE_ON_BAND])
def test_triton_tile_restatement_equals_dense(stage):
    rng = np.random.default_rng(5)
    n = 0
    for (B, H, G, Tq, D, kv_ctx, W, tds_list) in [
        (2, 4, 2, 4, 8, 11, 8, [8, 19]),
        (2, 4, 2, 1, 8, 11, 11, [11, 28]),
        (1, 2, 1, 2, 4, 7, 5, [6]),
    ]:
        q, kc, vc, _ = stream_case(rng, B, H, G, Tq, D, kv_ctx, W, tds_list, dtype=np.float32)
        q *= 0.5
        phase = [1] * B
        for BM in (1, 2, 4):
            if Tq % BM:
                continue
            # only the on-band stage alone depends on the tile size
            dense = ar.attention_ref(q, kc, vc, tds_list, phase, W, 1, stage=stage, scale=1.0, on_band_block=BM)
            for BN in (1, 2, 4):
                for S in (1, 2, 3):
                    tiles = ar.flash_tiles_ref(q, kc, vc, tds_list, phase, W, 1, stage=stage, BM=BM, BN=BN, num_splits=S)
                    np.testing.assert_allclose(tiles, dense, rtol=3e-5, atol=3e-6)
                    n += 1
    assert n >= 40


def test_split_merge_is_invariant():
    rng = np.random.default_rng(6)
    S, B, H, T, D = 5, 2, 3, 2, 4
    # build partials from a known dense problem: scores in log2 units
    n = 40
    s = rng.standard_normal((B, H, T, n)).astype(np.float32) * 3
    v = rng.standard_normal((B, H, n, D)).astype(np.float32)
    p = np.exp2(s - s.max(-1, keepdims=True))
    dense = (p @ v) / p.sum(-1, keepdims=True)
    bounds = [0, 3, 3, 17, 30, 40]  # includes an empty split
    po = np.zeros((S, B, H, T, D), np.float32)
    pl = np.zeros((S, B, H, T), np.float32)
    pm = np.full((S, B, H, T), -np.inf, np.float32)
    for i in range(S):
        a, b = bounds[i], bounds[i + 1]
        if a == b:
            continue
        m = s[..., a:b].max(-1)
        pp = np.exp2(s[..., a:b] - m[..., None])
        po[i], pl[i], pm[i] = pp @ v[..., a:b, :], pp.sum(-1), m
    # an empty split placed first gives exp2(-inf - -inf) = nan in the reference formula as well
    # (fa2.py:618-624); the reference never produces one first, so order them non-empty first.
    order = [0, 2, 1, 3, 4]
    merged = ar.reduce_split_kv_ref(po[order], pl[order], pm[order])
    np.testing.assert_allclose(merged, dense, rtol=2e-5, atol=2e-6)


def test_kv_append_reference_test_shapes():
    """tests/compare_scripts/test_add_kv.py:19-59."""
    rng = np.random.default_rng(8)
    B, G, t, T, D = 2, 4, 7, 17, 256
    x = rng.standard_normal((B, G, t, D)).astype(np.float32)
    cache0 = rng.standard_normal((B, G, T, D)).astype(np.float32)
    offs = np.array([15, 3])
    eps = 1e-6
    # plain
    exp = cache0.copy()
    for b in range(B):
        exp[b][:, (np.arange(t) + offs[b]) % T, :] = x[b]
    got = ar.kv_append_ref(x, cache0.copy(), offs, eps)
    assert np.array_equal(got, exp)
    # fused weightless RMSNorm
    rsos = (x * x).sum(-1)
    xn = x / np.sqrt(rsos[..., None] / D + eps)
    exp = cache0.copy()
    for b in range(B):
        exp[b][:, (np.arange(t) + offs[b]) % T, :] = xn[b]
    got = ar.kv_append_ref(x, cache0.copy(), offs, eps, x_rsos=rsos)
    np.testing.assert_allclose(got, exp, rtol=3e-7, atol=0)
    # phase skip + fp16 cache dtype
    c16 = cache0.astype(np.float16)
    got = ar.kv_append_ref(x, c16.copy(), offs, eps, user_phase=[1, 2], phase=2)
    assert np.array_equal(got[0], c16[0])
    assert np.array_equal(got[1][:, (np.arange(t) + 3) % T], x[1].astype(np.float16))


def test_advance_decode_state_arrays():
    inp = np.zeros((3, 4), np.int32)
    out = np.array([[5], [6], [7], [8]], np.int32)
    off = np.array([10, 20, 30, 40], np.int32)
    tds = off + 1
    ar.advance_decode_state_ref(inp, out, off, tds, np.array([2, 1, 0, 2], np.uint8))
    assert inp[0].tolist() == [5, 0, 0, 8] and not inp[1:].any()
    assert off.tolist() == [11, 20, 30, 41] and tds.tolist() == [12, 21, 31, 42]
