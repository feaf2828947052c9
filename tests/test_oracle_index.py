"""Pins the integer contracts of ``oracle.index_spec`` by brute force against a position model.

The position model is independent of the window formulas: a stream of tokens with absolute
positions 0..tds-1 is appended to a ring one row at a time (row = position % KV_CTX, as the
KV append does), and a query at absolute position p attends absolute positions according to
the CPU reference's rule (``scripts/reference_impl.py:437-441``).  The formulas of
``g4b/kernels/fa2.py:52-96`` must select exactly the same physical rows.
"""

import itertools

import numpy as np
import pytest

from oracle import index_spec as ix


def ring_after_appends(tds, kv_ctx):
    """Physical row -> absolute position held there after appending positions 0..tds-1."""
    ring = [None] * kv_ctx
    for p in range(tds):
        ring[p % kv_ctx] = p
    return ring


def small_cases():
    for kv_ctx in range(1, 10):
        for W in range(1, kv_ctx + 1):  # fa2.py:298 ctx_window_size <= KV_CTX
            for tds in range(0, 2 * kv_ctx + 3):
                for Tq in range(1, 6):
                    # live keys must not have been overwritten: the engine sizes rings as
                    # W + t - 1 (gemma4e.py:703-705) so the window never outruns the ring.
                    yield kv_ctx, W, tds, Tq


def test_window_selects_the_last_W_positions_of_the_stream():
    n = 0
    for kv_ctx, W, tds, Tq in small_cases():
        ring = ring_after_appends(tds, kv_ctx)
        win = ix.window_size(tds, W)
        base = ix.window_base(tds, W)
        assert win == len(range(max(tds - W, 0), tds))
        for j in range(win):
            row = ix.ring_row(tds, W, kv_ctx, j)
            assert 0 <= row < kv_ctx
            assert ring[row] == base + j, (kv_ctx, W, tds, j)
            n += 1
    assert n > 1000


def test_causal_visibility_equals_position_rule():
    for kv_ctx, W, tds, Tq in small_cases():
        if tds < Tq:
            continue  # caller never does this (scheduler.py:167-172)
        win = ix.window_size(tds, W)
        if win < Tq:
            continue
        base = ix.window_base(tds, W)
        for i in range(Tq):
            q_pos = tds - Tq + i  # reference_impl.py:437 with t_end = tds
            for j in range(-1, win + 2):
                k_pos = base + j
                expect = 0 <= j < win and not (q_pos < k_pos)  # reference_impl.py:439
                assert ix.visible(i, j, tds, W, Tq, ix.STAGE_CAUSAL) == expect
                assert ix.visible(i, j, tds, W, Tq, ix.STAGE_FULL) == (0 <= j < win)
                for qw in (1, 2, 3, 5):
                    expect_w = expect and not (q_pos - k_pos >= qw)  # reference_impl.py:441
                    assert ix.visible(i, j, tds, W, Tq, ix.STAGE_CAUSAL, qw) == expect_w
            lo, hi = ix.visible_range(i, tds, W, Tq, ix.STAGE_CAUSAL)
            assert [j for j in range(win) if ix.visible(i, j, tds, W, Tq, ix.STAGE_CAUSAL)] == list(range(lo, hi))
            for qw in (1, 3):
                lo, hi = ix.visible_range(i, tds, W, Tq, ix.STAGE_CAUSAL, qw)
                got = [j for j in range(win) if ix.visible(i, j, tds, W, Tq, ix.STAGE_CAUSAL, qw)]
                assert got == list(range(lo, hi))


@pytest.mark.parametrize("stage", [ix.STAGE_CAUSAL, ix.STAGE_FULL, ix.STAGE_ON_BAND])
def test_triton_program_grid_covers_exactly_the_visible_set(stage):
    """Union over (q tile, split) programs == visible(); programs of one q tile are disjoint.  STAGE_ON_BAND alone is
    the one stage whose result depends on the tile size, which visible() therefore takes as on_band_block."""
    checked = 0
    for kv_ctx, W, tds, Tq in itertools.product([5, 8], [3, 5], [0, 1, 4, 5, 6, 9, 13], [1, 2, 4]):
        if W > kv_ctx or tds < Tq or ix.window_size(tds, W) < Tq:
            continue
        for BM, BN, S in itertools.product([1, 2, 4], [1, 2, 4], [1, 2, 3]):
            if Tq % BM:
                continue
            sets = ix.program_key_sets(tds, W, Tq, stage, BM, BN, S)
            union = set()
            for (start_m, s), pairs in sets.items():
                assert not (union & pairs)
                union |= pairs
            expect = {
                (i, j)
                for i in range(Tq)
                for j in range(ix.window_size(tds, W))
                if ix.visible(i, j, tds, W, Tq, stage, on_band_block=BM)
            }
            for i in range(Tq):
                lo, hi = ix.visible_range(i, tds, W, Tq, stage, on_band_block=BM)
                assert {j for (ii, j) in expect if ii == i} == set(range(lo, hi))
            assert union == expect, (kv_ctx, W, tds, Tq, BM, BN, S)
            checked += 1
    assert checked > 200


def test_kv_split_ranges_partition_the_range():
    for lo in range(0, 4):
        for hi in range(lo, lo + 40):
            for S in (1, 2, 3, 4, 8, 16):
                parts = [ix.kv_split_range(lo, hi, S, s) for s in range(S)]
                covered = []
                for a, b in parts:
                    covered += list(range(a, max(a, b)))
                assert covered == list(range(lo, hi))


def test_ring_unroll_matches_the_reference_test_one_liner():
    """tests/compare_scripts/test_fa2.py:128-132: roll(x, -ring_start)[:, :window]."""
    rng = np.random.default_rng(0)
    for kv_ctx, W, tds in [(17, 17, 17), (17, 17, 34), (17, 12, 29), (64, 64, 64 + 17), (64, 32, 7)]:
        x = rng.standard_normal((3, kv_ctx, 4))
        win = min(tds, W)
        start = max(tds - W, 0) % kv_ctx
        expect = np.roll(x, -start, axis=1)[:, :win]
        rows = [ix.ring_row(tds, W, kv_ctx, j) for j in range(win)]
        assert np.array_equal(x[:, rows], expect)


def test_kv_append_rows_reference_test_case():
    """tests/compare_scripts/test_add_kv.py:19,29: t=7, T=17, offsets [15, 3]."""
    assert [ix.kv_append_row(t, 15, 17) for t in range(7)] == [15, 16, 0, 1, 2, 3, 4]
    assert [ix.kv_append_row(t, 3, 17) for t in range(7)] == [3, 4, 5, 6, 7, 8, 9]


def test_append_then_window_roundtrip():
    """Rows written by the append path are the rows the attention window reads back."""
    for T, W, t in [(17, 11, 7), (9, 9, 1), (23, 16, 8)]:
        ring = [None] * T
        ctx = 0
        for step in range(9):
            off, tds = ix.prefill_step_integers(ctx, t)
            for tt in range(t):
                ring[ix.kv_append_row(tt, off, T)] = off + tt
            ctx += t
            assert T >= W + t - 1  # gemma4e.py:703-705
            win, base = ix.window_size(tds, W), ix.window_base(tds, W)
            assert [ring[ix.ring_row(tds, W, T, j)] for j in range(win)] == list(range(base, base + win))


def test_split_heuristic_table():
    """g4b/kernels/fa2.py:201-212."""
    D, P = ix.PHASE_DECODE, ix.PHASE_PREFILL
    assert ix.select_num_kv_splits(P, 1, 65536, 16) == 1
    assert ix.select_num_kv_splits(D, 4, 65536, 16) == 1
    assert ix.select_num_kv_splits(D, 1, 4096, 16) == 1
    assert ix.select_num_kv_splits(D, 1, 4097, 16) == 4
    assert ix.select_num_kv_splits(D, 1, 8191, 16) == 4
    assert ix.select_num_kv_splits(D, 1, 8192, 16) == 8
    assert ix.select_num_kv_splits(D, 1, 32767, 16) == 8
    assert ix.select_num_kv_splits(D, 1, 32768, 16) == 16
    assert ix.select_num_kv_splits(D, 1, 32768, 4) == 4
    assert ix.select_num_kv_splits(D, 1, 32768, 1) == 1
    assert ix.select_num_kv_splits(D, 1, 32768, 3) == 1  # 3 -> 3 // 2 = 1 (fa2.py:214-218)


def test_scheduler_integers_and_geometry():
    assert ix.prefill_step_integers(0, 512) == (0, 512)
    assert ix.prefill_step_integers(700, 512) == (700, 1212)  # padded width, scheduler.py:172
    assert ix.decode_step_integers(1212) == (1212, 1213)
    g = ix.cache_geometry(32768, 512, 512)
    assert g == {"T_global": 33279, "T_swa": 1023, "W_global": 32768, "W_swa": 512}
    # q_t_base is never negative for what the scheduler uploads
    for ctx in (0, 3, 511, 512, 40000):
        off, tds = ix.prefill_step_integers(ctx, 512)
        for W in (512, 32768):
            assert ix.q_t_base(tds, W, 512) >= 0


def test_program_slot_decoding():
    G, tiles = 2, 3
    seen = set()
    for pid in range(4 * G * tiles):
        b, g, ht = ix.program_slot(pid, G, tiles)
        assert pid == (b * G + g) * tiles + ht
        seen.add((b, g, ht))
    assert len(seen) == 4 * G * tiles


def test_advance_decode_state_lists():
    inp, off, tds = ix.advance_decode_state([9, 9, 9], [5, 6, 7], [10, 20, 30], [11, 21, 31], [2, 1, 0])
    assert (inp, off, tds) == ([5, 9, 9], [11, 20, 30], [12, 21, 31])
