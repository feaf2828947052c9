"""Integer contracts of the attention hot path (test infrastructure, CPU only).

Pure-Python integer restatements of the index arithmetic the reference performs
on the device and in its scheduler.  All functions are total on Python ints and
are cheap enough for exhaustive brute force on small sizes.

Reference lines followed (paths relative to the reference checkout):

* ``g4b/kernels/fa2.py:14-34``    stage / phase constants
* ``g4b/kernels/fa2.py:52-67``    window, ring start, query base, stage ranges,
                                  split ranges
* ``g4b/kernels/fa2.py:73-96``    logical->physical key row, tail mask, causal mask
* ``g4b/kernels/fa2.py:186-225``  decode split-count heuristic
* ``g4b/kernels/fa2.py:322-335``  program -> (slot, kv head, head tile), phase skip
* ``g4b/kernels/add_kv_to_cache.py:146-159``  ring write row
* ``g4b/kernels/advance_decode_state.py:52-63`` decode state advance
* ``g4b/scheduler.py:133-212``    per-slot offsets / lengths the scheduler uploads
* ``g4b/models/gemma4e.py:702-717,856-866`` cache geometry
"""

from __future__ import annotations

# g4b/kernels/fa2.py:14-19
STAGE_FULL = 1
STAGE_ON_BAND = 2
STAGE_CAUSAL = STAGE_FULL | STAGE_ON_BAND
INNER_STAGE_OFF_BAND = 1
INNER_STAGE_ON_BAND = 2
INNER_STAGE_FULL = 3
# g4b/kernels/fa2.py:29-31
PHASE_UNALLOCATED = 0
PHASE_PREFILL = 1
PHASE_DECODE = 2


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


# --------------------------------------------------------------------------- ring / window
def window_size(tds: int, W: int) -> int:
    """Number of keys of a slot that an attention launch may look at (fa2.py:53)."""
    return min(tds, W)


def window_base(tds: int, W: int) -> int:
    """Absolute position of logical key 0 (fa2.py:54 before the modulo)."""
    return max(tds - W, 0)


def ring_start(tds: int, W: int, kv_ctx: int) -> int:
    """Physical ring row of logical key 0 (fa2.py:54)."""
    return max(tds - W, 0) % kv_ctx


def ring_row(tds: int, W: int, kv_ctx: int, j: int) -> int:
    """Physical ring row of logical key ``j`` (fa2.py:75)."""
    return (ring_start(tds, W, kv_ctx) + j) % kv_ctx


def q_t_base(tds: int, W: int, Tq: int) -> int:
    """Logical key index aligned with query 0 (fa2.py:55); bottom-right aligned."""
    return window_size(tds, W) - Tq


def visible(i: int, j: int, tds: int, W: int, Tq: int, stage: int, query_window: int | None = None,
            on_band_block: int | None = None) -> bool:
    """Does query ``i`` (0-based inside the launch) attend logical key ``j``?

    ``STAGE_FULL``: every key of the window (fa2.py:62-64, tail mask :74,:90).
    ``STAGE_CAUSAL``: keys ``j <= q_t_base + i`` (off-band range ``[0, q_tile_start)``
    plus the causally masked diagonal block, fa2.py:58-61,93-96); the union over
    tiles does not depend on the tile size.
    ``STAGE_ON_BAND`` alone: only the diagonal block of the query's tile (fa2.py:56,61,93-96),
    keys ``q_tile_start <= j <= q_t_base + i`` with ``q_tile_start = q_t_base +
    (i // Q_BLOCKSIZE_T) * Q_BLOCKSIZE_T``; the tile size (``on_band_block``) is the
    reference's autotuned constant and has to be named.
    ``query_window`` (extension; ``scripts/reference_impl.py:440-441``): additionally
    ``q_pos - k_pos < query_window``, the per-query sliding window of a one-shot
    prefill longer than the window.
    """
    win = window_size(tds, W)
    if j < 0 or j >= win:
        return False
    if stage == STAGE_FULL:
        ok = True
    elif stage == STAGE_CAUSAL:
        ok = j <= q_t_base(tds, W, Tq) + i
    elif stage == STAGE_ON_BAND:
        if on_band_block is None or on_band_block < 1:
            raise ValueError("STAGE_ON_BAND alone depends on the tile size: pass on_band_block")
        qb = q_t_base(tds, W, Tq)
        ok = qb + (i // on_band_block) * on_band_block <= j <= qb + i
    else:
        raise ValueError("unknown stage")
    if ok and query_window is not None:
        ok = (q_t_base(tds, W, Tq) + i) - j < query_window
    return ok


def visible_range(i: int, tds: int, W: int, Tq: int, stage: int, query_window: int | None = None,
                  on_band_block: int | None = None) -> tuple[int, int]:
    """Half-open logical key range ``[lo, hi)`` of query ``i`` (empty if ``hi <= lo``)."""
    win = window_size(tds, W)
    qp = q_t_base(tds, W, Tq) + i
    hi = win if stage == STAGE_FULL else min(win, qp + 1)
    lo = 0
    if stage == STAGE_ON_BAND:
        lo = max(0, q_t_base(tds, W, Tq) + (i // on_band_block) * on_band_block)
    if query_window is not None:
        lo = max(0, qp - query_window + 1)
    return lo, max(hi, lo)


# --------------------------------------------------------------------------- stage / split ranges of one Triton program
def stage_range(inner_stage: int, tds: int, W: int, Tq: int, start_m: int, BM: int) -> tuple[int, int]:
    """Key range a program walks in one inner stage before split partitioning (fa2.py:56-64)."""
    win = window_size(tds, W)
    q_tile_start = q_t_base(tds, W, Tq) + start_m * BM
    if inner_stage == INNER_STAGE_OFF_BAND:
        return 0, q_tile_start
    if inner_stage == INNER_STAGE_ON_BAND:
        return q_tile_start, q_tile_start + BM
    return 0, win


def kv_split_range(lo: int, hi: int, num_splits: int, split: int) -> tuple[int, int]:
    """Sub-range of ``[lo, hi)`` owned by ``split`` (fa2.py:65-67).  May be empty."""
    size = cdiv(hi - lo, num_splits)
    lo2 = lo + split * size
    hi2 = min(hi, lo2 + size)
    return lo2, hi2


def program_slot(off_bgh: int, G: int, q_head_tiles_per_kv: int) -> tuple[int, int, int]:
    """Decode ``program_id(2)`` into (slot, kv head, query-head tile) (fa2.py:325-330)."""
    off_b = off_bgh // (G * q_head_tiles_per_kv)
    off_gqh = off_bgh % (G * q_head_tiles_per_kv)
    return off_b, off_gqh // q_head_tiles_per_kv, off_gqh % q_head_tiles_per_kv


def program_key_sets(tds: int, W: int, Tq: int, stage: int, BM: int, BN: int, num_splits: int):
    """Enumerate, program by program, the (query, key) pairs the Triton grid touches unmasked.

    Returns ``{(start_m, split): set((i, j))}`` following fa2.py:58-96 literally: stage
    ranges, split partition, KV tiles of ``BN`` with the tail mask ``j < hi`` and, on the
    diagonal block, the causal mask ``q_t_base + i >= j``.
    """
    out = {}
    qb = q_t_base(tds, W, Tq)
    for start_m in range(cdiv(Tq, BM)):
        rows = [i for i in range(start_m * BM, start_m * BM + BM) if i < Tq]
        for s in range(num_splits):
            pairs = set()
            stages = []
            if stage & STAGE_FULL:
                stages.append(INNER_STAGE_FULL if stage == STAGE_FULL else INNER_STAGE_OFF_BAND)
            if stage & STAGE_ON_BAND:
                stages.append(INNER_STAGE_ON_BAND)
            for inner in stages:
                lo, hi = stage_range(inner, tds, W, Tq, start_m, BM)
                lo, hi = kv_split_range(lo, hi, num_splits, s)
                for start_n in range(lo, hi, BN):
                    for j in range(start_n, start_n + BN):
                        if not j < hi:
                            continue
                        for i in rows:
                            if inner == INNER_STAGE_ON_BAND and not (qb + i >= j):
                                continue
                            pairs.add((i, j))
            out[(start_m, s)] = pairs
    return out


def select_num_kv_splits(phase: int, Tq: int, W: int, max_kv_splits: int) -> int:
    """The reference's decode split count with its default (untuned) config list (fa2.py:151-158,186-225)."""
    available = [1, 2, 4, 8, 16]
    if phase != PHASE_DECODE or Tq != 1:
        return 1
    if max_kv_splits <= 1 or W <= 4096:
        target = 1
    elif W < 8192:
        target = 4
    elif W < 32768:
        target = 8
    else:
        target = 16
    target = min(target, max_kv_splits)
    while target > 1 and not (target in available and target <= max_kv_splits):
        target //= 2
    return max(target, 1)


# --------------------------------------------------------------------------- KV append / decode advance
def kv_append_row(t: int, cache_offset: int, T: int) -> int:
    """Ring row that new token ``t`` of a slot is written to (add_kv_to_cache.py:153-158)."""
    return (t + cache_offset) % T


def slot_in_phase(user_phase, b: int, phase: int) -> bool:
    """Per-slot skip predicate (g4b/kernels/utils.py:32-48 at one slot per program; fa2.py:332-335).

    ``user_phase is None`` disables skipping (add_kv_to_cache default).
    """
    if user_phase is None:
        return True
    return int(user_phase[b]) == phase


def advance_decode_state(input_tok_row0, out_tok_col0, cache_offsets, time_dim_sizes, user_phase):
    """List-in / list-out restatement of advance_decode_state.py:52-63."""
    inp, off, tds = list(input_tok_row0), list(cache_offsets), list(time_dim_sizes)
    for b in range(len(user_phase)):
        if int(user_phase[b]) == PHASE_DECODE:
            inp[b] = out_tok_col0[b]
            off[b] += 1
            tds[b] += 1
    return inp, off, tds


# --------------------------------------------------------------------------- scheduler integers / cache geometry
def prefill_step_integers(ctx_len_before: int, t: int) -> tuple[int, int]:
    """(cache_offset, time_dim_size) the scheduler uploads for a prefilling slot (scheduler.py:160-172).

    The length is ``offset + t`` (the padded chunk width), never the real token count.
    Inactive slots get ``(0, 0)`` (scheduler.py:142-148).
    """
    return ctx_len_before, ctx_len_before + t


def decode_step_integers(ctx_len: int) -> tuple[int, int]:
    """(cache_offset, time_dim_size) for a decoding slot (scheduler.py:195-201)."""
    return ctx_len, ctx_len + 1


def cache_geometry(context_len: int, sliding_window: int, t: int) -> dict:
    """Ring lengths and window sizes of the engine (gemma4e.py:702-705,856-858)."""
    return {
        "T_global": context_len + t - 1,
        "T_swa": sliding_window + t - 1,
        "W_global": context_len,
        "W_swa": min(sliding_window, context_len),
    }
