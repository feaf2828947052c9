"""CPU restatement of the step right before the attention path: q/k RMSNorm + rotary embedding
(test infrastructure only; nothing under ``g4b_amd/`` imports this).

* :func:`apply_rope_ref` follows ``g4b/kernels/rope.py:9-40`` (one tile: load the two halves of a head,
  scale by ``rsqrt(rsos / D + eps) * w``, rotate) and ``:177-186`` (``theta = (time_dim_offsets[b] + t) *
  rope_freqs[k]`` in fp32, ``sin``/``cos`` of that fp32 angle, shared by q and k).
* :func:`populate_rope_frequencies_ref` follows ``g4b/kernels/rope.py:262-288``
  (``1 / freq_base ** (k / n)``, optionally divided by per-frequency scalars).
* :func:`rope_append_ref` is the engine's sequence ``apply_rope`` -> ``add_kv_to_cache(k)`` ->
  ``add_kv_to_cache(v, v_rsos)`` (``g4b/models/gemma4e.py:564-590``) composed from the restatements.

Pinned without the reference (tests/test_oracle_rope.py): the rotation is complex multiplication by
``exp(i*theta)`` (checked against numpy complex arithmetic), it preserves the norm of every (x[k], x[k + D/2])
pair, angle 0 is the identity; the normalisation equals ``x / sqrt(mean(x^2) + eps) * w`` when ``rsos`` is the row's
sum of squares; the whole equals the CPU reference model's formulation ``x*cos + rotate_half(x)*sin`` with
``theta`` concatenated to full width (``scripts/reference_impl.py:249-263``), restated there with torch ops.
"""

from __future__ import annotations

import numpy as np

from .attention_ref import kv_append_ref


def rope_angles(time_dim_offsets, t: int, rope_freqs) -> np.ndarray:
    """``[B, t, D/2]`` fp32 angles: integer position times fp32 frequency, rounded to fp32 (rope.py:177-183)."""
    pos = np.asarray(time_dim_offsets, dtype=np.int64)[:, None] + np.arange(t, dtype=np.int64)[None, :]
    return (pos.astype(np.float32)[:, :, None] * np.asarray(rope_freqs, dtype=np.float32)[None, None, :]).astype(np.float32)


def _rope_tile(x, rsos, w, sin, cos, eps: float) -> np.ndarray:
    """rope.py:22-40 on a ``[B, heads, t, D]`` array; fp32 arithmetic in the kernel's order."""
    x = np.asarray(x, dtype=np.float32)
    D = x.shape[-1]
    half = D // 2
    inv_rms = (np.float32(1.0) / np.sqrt(np.asarray(rsos, dtype=np.float32) / np.float32(D) + np.float32(eps))).astype(np.float32)
    w = np.asarray(w, dtype=np.float32)
    x1 = x[..., :half] * (inv_rms[..., None] * w[:half])
    x2 = x[..., half:] * (inv_rms[..., None] * w[half:])
    s, c = sin[:, None, :, :], cos[:, None, :, :]
    y1 = c * x1 - s * x2
    y2 = c * x2 + s * x1
    return np.concatenate([y1, y2], axis=-1).astype(np.float32)


def apply_rope_ref(q, k, rope_freqs, time_dim_offsets, q_rsos, k_rsos, q_rmsnorm_w, k_rmsnorm_w, rmsnorm_eps: float):
    """Returns the rotated (q, k) as fp32 arrays; the kernel writes them back in place (rope.py:39-40)."""
    assert q.shape[0] == k.shape[0] and q.shape[2] == k.shape[2] and q.shape[3] == k.shape[3]  # rope.py:150-153
    assert len(rope_freqs) == k.shape[3] // 2  # rope.py:149
    theta = rope_angles(time_dim_offsets, k.shape[2], rope_freqs)
    # the angle is fp32; its sine and cosine are evaluated exactly and rounded once
    sin = np.sin(theta.astype(np.float64)).astype(np.float32)
    cos = np.cos(theta.astype(np.float64)).astype(np.float32)
    return (
        _rope_tile(q, q_rsos, q_rmsnorm_w, sin, cos, rmsnorm_eps),
        _rope_tile(k, k_rsos, k_rmsnorm_w, sin, cos, rmsnorm_eps),
    )


def populate_rope_frequencies_ref(n: int, freq_base: float, freq_scalars=None) -> np.ndarray:
    """rope.py:275-286: ``1 / 2 ** (log2(freq_base) * k / n)`` [``/ freq_scalars[k]``], fp64 here."""
    k = np.arange(n, dtype=np.float64)
    out = 1.0 / np.exp2(np.log2(freq_base) * (k / n))
    if freq_scalars is not None:
        out = out / np.asarray(freq_scalars, dtype=np.float64)
    return out


def rope_append_ref(q, k, v, rope_freqs, cache_offsets, q_rsos, k_rsos, v_rsos, q_rmsnorm_w, k_rmsnorm_w,
                    rmsnorm_eps: float, k_cache, v_cache, user_phase=None, phase: int = 0):
    """gemma4e.py:564-590: rotate q and k, append rotated k and (weightlessly normalised) v to the rings.

    Returns (q_rot, k_rot); the caches are updated in place in their own dtype.
    """
    q_rot, k_rot = apply_rope_ref(q, k, rope_freqs, cache_offsets, q_rsos, k_rsos, q_rmsnorm_w, k_rmsnorm_w, rmsnorm_eps)
    kv_append_ref(k_rot, k_cache, cache_offsets, rmsnorm_eps, None, user_phase, phase)
    kv_append_ref(np.asarray(v, dtype=np.float32), v_cache, cache_offsets, rmsnorm_eps, v_rsos, user_phase, phase)
    return q_rot, k_rot
