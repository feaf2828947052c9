"""Floating-point restatements of the attention hot path (test infrastructure, CPU only).

* :func:`attention_ref` -- dense masked softmax attention over the un-rolled ring,
  any float dtype (fp64 by default).  This is the parity oracle.  Semantics follow
  ``g4b/kernels/fa2.py:52-136,322-480`` (window, ring, stages, per-slot phase skip)
  and ``scripts/reference_impl.py:434-443`` (GQA by head replication, ``q_pos < k_pos``
  mask, optional per-query window mask, ``softmax(q k^T + mask) v``).
* :func:`retrieve_ref_torch` -- torch-CPU fp32 restatement of
  ``scripts/reference_impl.py:421-443`` written the way the reference writes it
  (slice the visible keys, ``repeat_interleave``, dense additive mask, two matmuls).
  This is what ``bench.py`` times as the CPU baseline.
* :func:`flash_tiles_ref` -- tile-by-tile restatement of the Triton program
  (``fa2.py:37-136``: additive ``-1e6`` masks, ``exp2`` with ``log2(e)`` folded in,
  online softmax, optional split partials) and :func:`reduce_split_kv_ref`
  (``fa2.py:585-631``).
* :func:`kv_append_ref` (``g4b/kernels/add_kv_to_cache.py:146-159``) and
  :func:`advance_decode_state_ref` (``g4b/kernels/advance_decode_state.py:52-63``).

Rows whose visible key set is empty (``tds == 0`` on an in-phase slot, or
``tds < Tq``) are ``0/0`` in the reference and are ignored by its caller
(``g4b/scheduler.py:142-148,167-172``); this oracle returns 0 for them and reports
them through ``empty_rows`` so that tests can treat them as unspecified.
"""

from __future__ import annotations

import numpy as np

from . import index_spec as ix

LOG2E = 1.44269504  # the constant the reference multiplies by (fa2.py:89)


# --------------------------------------------------------------------------- ring helpers
def unroll_ring(cache_b: np.ndarray, tds: int, W: int) -> np.ndarray:
    """``[G, KV_CTX, D]`` ring -> ``[G, window, D]`` in logical key order.

    Built row by row from :func:`index_spec.ring_row`; the reference test's one-liner
    (``torch.roll(x, -ring_start, 1)[:, :window]``, test_fa2.py:128-132) is checked
    against this in the tests rather than used here.
    """
    kv_ctx = cache_b.shape[1]
    win = ix.window_size(tds, W)
    rows = [ix.ring_row(tds, W, kv_ctx, j) for j in range(win)]
    return cache_b[:, rows, :]


def visibility_mask(tds: int, W: int, Tq: int, stage: int, query_window: int | None = None,
                    on_band_block: int | None = None) -> np.ndarray:
    """Boolean ``[Tq, window]`` mask, vectorised form of :func:`index_spec.visible`."""
    win = ix.window_size(tds, W)
    i = np.arange(Tq)[:, None]
    j = np.arange(win)[None, :]
    qp = ix.q_t_base(tds, W, Tq) + i
    if stage == ix.STAGE_FULL:
        m = np.ones((Tq, win), dtype=bool)
    elif stage == ix.STAGE_CAUSAL:
        m = j <= qp
    elif stage == ix.STAGE_ON_BAND:
        if on_band_block is None or on_band_block < 1:
            raise ValueError("STAGE_ON_BAND alone depends on the tile size: pass on_band_block")
        tile_start = ix.q_t_base(tds, W, Tq) + (i // on_band_block) * on_band_block  # fa2.py:56,61
        m = (j >= tile_start) & (j <= qp)
    else:
        raise ValueError("unknown stage")
    if query_window is not None:
        m = m & (qp - j < query_window)
    return m


# --------------------------------------------------------------------------- the parity oracle
def attention_ref(
    q,
    k_cache,
    v_cache,
    time_dim_sizes,
    user_phase,
    ctx_window_size: int,
    phase: int,
    *,
    stage: int = ix.STAGE_CAUSAL,
    scale: float = 1.0,
    query_window: int | None = None,
    window_sizes=None,
    out=None,
    dtype=np.float64,
    return_empty_rows: bool = False,
    on_band_block: int | None = None,
):
    """Dense reference attention.

    ``q``: ``[B,H,Tq,D]``; ``k_cache, v_cache``: ``[B,G,KV_CTX,D]``;
    ``time_dim_sizes``: ``[B]`` ints; ``user_phase``: ``[B]`` ints.  Slots whose phase
    differs from ``phase`` are left as they are in ``out`` (fa2.py:332-335).
    ``window_sizes`` (extension): per-slot override of ``ctx_window_size``.
    """
    q = np.asarray(q, dtype=dtype)
    k_cache = np.asarray(k_cache, dtype=dtype)
    v_cache = np.asarray(v_cache, dtype=dtype)
    B, H, Tq, D = q.shape
    G = k_cache.shape[1]
    R = H // G
    o = np.zeros((B, H, Tq, D), dtype=dtype) if out is None else out
    empty = np.zeros((B, Tq), dtype=bool)
    for b in range(B):
        if int(user_phase[b]) != phase:
            continue
        tds = int(time_dim_sizes[b])
        W = int(ctx_window_size if window_sizes is None else window_sizes[b])
        k = unroll_ring(k_cache[b], tds, W)
        v = unroll_ring(v_cache[b], tds, W)
        mask = visibility_mask(tds, W, Tq, stage, query_window, on_band_block)
        empty[b] = ~mask.any(axis=1)
        for h in range(H):
            g = h // R  # repeat_interleave(k, H // G, 1): head h reads kv head h // R (reference_impl.py:434-435)
            s = (q[b, h] @ k[g].T) * scale
            s = np.where(mask, s, -np.inf)
            smax = np.max(s, axis=1, keepdims=True, initial=-np.inf)
            smax = np.where(np.isfinite(smax), smax, 0.0)
            p = np.exp(s - smax)
            denom = p.sum(axis=1, keepdims=True)
            res = (p @ v[g]) / np.where(denom == 0, 1.0, denom)
            o[b, h] = np.where(denom == 0, 0.0, res)
    if return_empty_rows:
        return o, empty
    return o


# --------------------------------------------------------------------------- the timed CPU baseline
def retrieve_ref_torch(q, k_lin, v_lin, *, scale: float = 1.0, query_window: int | None = None, causal: bool = True):
    """One slot of ``LayerKVCache.retrieve`` (scripts/reference_impl.py:434-443), torch CPU fp32.

    ``q``: ``[1,H,Tq,D]``; ``k_lin, v_lin``: ``[1,G,Tk,D]`` already sliced to the visible
    physical range ``[t_start, t_end)`` (reference_impl.py:427-431).  The query block is
    the last ``Tq`` positions.  ``scale`` multiplies ``q`` (the reference has none).
    """
    import torch

    q = q.float()
    k = torch.repeat_interleave(k_lin.float(), q.shape[1] // k_lin.shape[1], 1)
    v = torch.repeat_interleave(v_lin.float(), q.shape[1] // v_lin.shape[1], 1)
    t_end = k.shape[-2]
    q_pos = torch.arange(t_end - q.shape[-2], t_end)[:, None]
    k_pos = torch.arange(0, t_end)[None, :]
    if causal:
        mask = q_pos < k_pos
    else:
        mask = torch.zeros((q.shape[-2], t_end), dtype=torch.bool)
    if query_window is not None:
        mask = torch.logical_or(mask, q_pos - k_pos >= query_window)
    mask = torch.where(mask, float("-inf"), 0.0)
    if scale != 1.0:
        q = q * scale
    return (q @ k.transpose(-1, -2) + mask).softmax(-1) @ v


def attention_cpu_baseline(
    q,
    k_cache,
    v_cache,
    time_dim_sizes,
    user_phase,
    ctx_window_size: int,
    phase: int,
    *,
    stage: int = ix.STAGE_CAUSAL,
    scale: float = 1.0,
    query_window: int | None = None,
    window_sizes=None,
    slots=None,
    row_block: int | None = None,
):
    """Whole-batch CPU attention the way the reference's CPU path would run it.

    torch tensors in, torch fp32 ``[B,H,Tq,D]`` out.  Per in-phase slot: un-roll the ring
    to the visible keys (the reference keeps a linear buffer instead, reference_impl.py:
    427-431), then :func:`retrieve_ref_torch`.  ``slots`` restricts the work to a subset
    (bounded timing samples); ``row_block`` processes query rows in blocks to bound the
    score tensor.
    """
    import torch

    B, H, Tq, D = q.shape
    o = torch.zeros((B, H, Tq, D), dtype=torch.float32)
    for b in range(B) if slots is None else slots:
        if int(user_phase[b]) != phase:
            continue
        tds = int(time_dim_sizes[b])
        W = int(ctx_window_size if window_sizes is None else window_sizes[b])
        kv_ctx = k_cache.shape[2]
        win = ix.window_size(tds, W)
        if win == 0:
            continue
        start = ix.ring_start(tds, W, kv_ctx)
        rows = (torch.arange(win) + start) % kv_ctx
        k_lin = k_cache[b : b + 1, :, rows]
        v_lin = v_cache[b : b + 1, :, rows]
        if row_block is None or Tq <= row_block:
            o[b] = retrieve_ref_torch(
                q[b : b + 1], k_lin, v_lin, scale=scale, query_window=query_window, causal=stage != ix.STAGE_FULL
            )[0]
        else:
            for r0 in range(0, Tq, row_block):
                r1 = min(Tq, r0 + row_block)
                # queries r0..r1 are the last rows of a problem truncated at key (win - Tq + r1)
                hi = win - Tq + r1 if stage != ix.STAGE_FULL else win
                o[b, :, r0:r1] = retrieve_ref_torch(
                    q[b : b + 1, :, r0:r1],
                    k_lin[:, :, :hi],
                    v_lin[:, :, :hi],
                    scale=scale,
                    query_window=query_window,
                    causal=stage != ix.STAGE_FULL,
                )[0]
    return o


# --------------------------------------------------------------------------- Triton program restatement
def flash_tiles_ref(
    q,
    k_cache,
    v_cache,
    time_dim_sizes,
    user_phase,
    ctx_window_size: int,
    phase: int,
    *,
    stage: int = ix.STAGE_CAUSAL,
    BM: int = 4,
    BN: int = 4,
    num_splits: int = 1,
    out=None,
):
    """Tile-by-tile fp32 restatement of ``_attn_kernel`` + ``_reduce_split_kv_kernel``.

    Follows fa2.py literally: scale 1.0 with ``log2(e)`` folded into the scores (:89),
    additive ``-1e6`` masks (:90,:96), ``exp2`` online softmax (:99-134), un-normalised
    split partials merged by :func:`reduce_split_kv_ref`.  Small sizes only.
    """
    f32 = np.float32
    q = np.asarray(q, dtype=f32)
    k_cache = np.asarray(k_cache, dtype=f32)
    v_cache = np.asarray(v_cache, dtype=f32)
    B, H, Tq, D = q.shape
    G, kv_ctx = k_cache.shape[1], k_cache.shape[2]
    R = H // G
    o = np.zeros((B, H, Tq, D), dtype=f32) if out is None else out
    W = ctx_window_size
    part_o = np.zeros((num_splits, B, H, Tq, D), dtype=f32)
    part_l = np.zeros((num_splits, B, H, Tq), dtype=f32)
    part_m = np.full((num_splits, B, H, Tq), -np.inf, dtype=f32)
    for b in range(B):
        if int(user_phase[b]) != phase:
            continue
        tds = int(time_dim_sizes[b])
        qb = ix.q_t_base(tds, W, Tq)
        rs = ix.ring_start(tds, W, kv_ctx)
        for h in range(H):
            g = h // R
            for start_m in range(ix.cdiv(Tq, BM)):
                rows = np.arange(start_m * BM, min(Tq, start_m * BM + BM))
                for s in range(num_splits):
                    m_i = np.full(len(rows), -np.inf, dtype=f32)
                    l_i = np.zeros(len(rows), dtype=f32)
                    acc = np.zeros((len(rows), D), dtype=f32)
                    inner_stages = []
                    if stage & ix.STAGE_FULL:
                        inner_stages.append(ix.INNER_STAGE_FULL if stage == ix.STAGE_FULL else ix.INNER_STAGE_OFF_BAND)
                    if stage & ix.STAGE_ON_BAND:
                        inner_stages.append(ix.INNER_STAGE_ON_BAND)
                    for inner in inner_stages:
                        lo, hi = ix.stage_range(inner, tds, W, Tq, start_m, BM)
                        lo, hi = ix.kv_split_range(lo, hi, num_splits, s)
                        for start_n in range(lo, hi, BN):
                            jl = start_n + np.arange(BN)
                            kv_mask = jl < hi
                            phys = (rs + jl) % kv_ctx
                            kt = np.where(kv_mask[:, None], k_cache[b, g, phys], f32(0))
                            vt = np.where(kv_mask[:, None], v_cache[b, g, phys], f32(0))
                            with np.errstate(invalid="ignore", over="ignore"):
                                qk = (q[b, h, rows] @ kt.T) * f32(LOG2E)
                                qk = qk + np.where(kv_mask[None, :], f32(0), f32(-1.0e6))
                                if inner == ix.INNER_STAGE_ON_BAND:
                                    cm = (qb + rows)[:, None] >= jl[None, :]
                                    qk = qk + np.where(cm, f32(0), f32(-1.0e6))
                                m_ij = np.maximum(m_i, qk.max(axis=1))
                                p = np.exp2(qk - m_ij[:, None])
                                alpha = np.exp2(m_i - m_ij)
                                acc = acc * alpha[:, None] + p @ vt
                                l_i = l_i * alpha + p.sum(axis=1)
                                m_i = m_ij
                    if num_splits > 1:
                        part_o[s, b, h, rows] = acc
                        part_l[s, b, h, rows] = l_i
                        part_m[s, b, h, rows] = m_i
                    else:
                        with np.errstate(invalid="ignore", divide="ignore"):
                            o[b, h, rows] = acc / l_i[:, None]
    if num_splits > 1:
        merged = reduce_split_kv_ref(part_o, part_l, part_m)
        for b in range(B):
            if int(user_phase[b]) == phase:
                o[b] = merged[b]
    return o


def reduce_split_kv_ref(part_o, part_l, part_m):
    """Merge ``S`` split partials (fa2.py:585-631).  ``part_m`` is in log2 units."""
    f32 = np.float32
    S = part_o.shape[0]
    m = np.full(part_m.shape[1:], -np.inf, dtype=f32)
    l = np.zeros(part_l.shape[1:], dtype=f32)
    acc = np.zeros(part_o.shape[1:], dtype=f32)
    with np.errstate(invalid="ignore", divide="ignore"):
        for s in range(S):
            m_new = np.maximum(part_m[s], m)
            a_new = np.exp2(part_m[s] - m_new)
            a_cur = np.exp2(m - m_new)
            acc = acc * a_cur[..., None] + part_o[s].astype(f32) * a_new[..., None]
            l = l * a_cur + part_l[s] * a_new
            m = m_new
        return acc / l[..., None]


# --------------------------------------------------------------------------- KV append / advance
def kv_append_ref(x, cache, cache_offsets, rmsnorm_eps: float, x_rsos=None, user_phase=None, phase: int = 0):
    """In-place ring write (add_kv_to_cache.py:124-159).

    ``x``: ``[B,G,t,D]``; ``cache``: ``[B,G,T,D]`` (written in the cache's dtype);
    ``x_rsos``: ``[B,G,t]`` row sums of squares, enabling the weightless RMSNorm
    ``x * rsqrt(x_rsos / D + eps)`` evaluated in fp32 (add_kv_to_cache.py:148-151).
    """
    B, G, t, D = x.shape
    T = cache.shape[2]
    assert t <= T  # add_kv_to_cache.py:119
    for b in range(B):
        if not ix.slot_in_phase(user_phase, b, phase):
            continue
        off = int(cache_offsets[b])
        for tt in range(t):
            row = ix.kv_append_row(tt, off, T)
            val = np.asarray(x[b, :, tt, :], dtype=np.float32)
            if x_rsos is not None:
                r = np.asarray(x_rsos[b, :, tt], dtype=np.float32)
                inv = (np.float32(1.0) / np.sqrt(r / np.float32(D) + np.float32(rmsnorm_eps))).astype(np.float32)
                val = val * inv[:, None]
            cache[b, :, row, :] = val.astype(cache.dtype)
    return cache


def advance_decode_state_ref(input_token_ids, out_token_ids, cache_offsets, time_dim_sizes, user_phase):
    """In-place restatement of advance_decode_state.py:52-63 on numpy arrays.

    ``input_token_ids``: ``[t, B]`` (row 0 is written), ``out_token_ids``: ``[B, >=1]``.
    """
    B = input_token_ids.shape[1]
    for b in range(B):
        if int(user_phase[b]) == ix.PHASE_DECODE:
            input_token_ids[0, b] = out_token_ids[b, 0]
            cache_offsets[b] += 1
            time_dim_sizes[b] += 1
    return input_token_ids, cache_offsets, time_dim_sizes
