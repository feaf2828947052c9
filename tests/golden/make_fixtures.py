"""Writes the committed golden fixtures of the attention path.

    python tests/golden/make_fixtures.py

The reference ships no stored vectors for this path (its compare scripts draw unseeded random
inputs), so these fixtures are produced by this repository's own fp64 oracle
(``oracle.attention_ref``, ``oracle.rope_ref``), which ``tests/test_oracle_*.py`` pin against closed forms.  Each
``.npz`` holds the inputs exactly as the kernels see them (fp16 / int) and the fp64 result rounded
to fp32.  Nothing of the reference is read or executed.
"""

from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import attention_ref as ar  # noqa: E402
from oracle import index_spec as ix  # noqa: E402
from oracle import rope_ref as rr  # noqa: E402

CASES = {
    # name: B, H, G, Tq, D, kv_ctx, W, tds, user_phase, launch phase, stage, scale, query_window
    "decode_wrap": (4, 8, 2, 1, 128, 96, 96, [96, 113, 1, 40], [2, 2, 2, 1], 2, ix.STAGE_CAUSAL, 1.0, None),
    "decode_swa_scaled": (3, 8, 2, 1, 256, 80, 48, [48, 200, 7], [2, 2, 2], 2, ix.STAGE_CAUSAL, 1 / 16, None),
    "chunk_on_context": (2, 8, 2, 40, 128, 103, 64, [40, 167], [1, 1], 1, ix.STAGE_CAUSAL, 1 / 16, None),
    "full_stage": (2, 4, 4, 24, 128, 24, 24, [24, 41], [1, 1], 1, ix.STAGE_FULL, 1.0, None),
    "per_query_window": (1, 8, 2, 72, 128, 72, 72, [72], [1], 1, ix.STAGE_CAUSAL, 1 / 16, 17),
    # the diagonal block alone, for a tile size (Q_BLOCKSIZE_T, fa2.py:56,61) of 16 query positions
    "on_band_block16": (2, 8, 2, 48, 128, 120, 96, [48, 200], [1, 1], 1, ix.STAGE_ON_BAND, 1 / 16, None, 16),
}


def build(name):
    B, H, G, Tq, D, kv_ctx, W, tds, phase_arr, phase, stage, scale, qw, *rest = CASES[name]
    band = rest[0] if rest else None
    rng = np.random.default_rng(sum(map(ord, name)))
    q = rng.standard_normal((B, H, Tq, D)).astype(np.float16)
    k = rng.standard_normal((B, G, kv_ctx, D)).astype(np.float16)
    v = rng.standard_normal((B, G, kv_ctx, D)).astype(np.float16)
    out0 = np.full((B, H, Tq, D), 777.0)
    o = ar.attention_ref(q, k, v, tds, phase_arr, W, phase, stage=stage, scale=scale, query_window=qw, out=out0.copy(),
                         on_band_block=band)
    extra = {} if band is None else {"on_band_block": np.int32(band)}
    return dict(
        **extra,
        q=q, k_cache=k, v_cache=v, time_dim_sizes=np.array(tds, np.int32), user_phase=np.array(phase_arr, np.uint8),
        ctx_window_size=np.int32(W), phase=np.int32(phase), stage=np.int32(stage), scale=np.float32(scale),
        query_window=np.int32(0 if qw is None else qw), expected=o.astype(np.float32),
    )


def kv_append_fixture():
    """Shapes of tests/compare_scripts/test_add_kv.py:19,29 (B,G,t,T,D = 2,4,7,17,256; offsets [15, 3])."""
    rng = np.random.default_rng(17)
    B, G, t, T, D = 2, 4, 7, 17, 256
    x = rng.standard_normal((B, G, t, D)).astype(np.float32)
    cache = rng.standard_normal((B, G, T, D)).astype(np.float16)
    offs = np.array([15, 3], np.int32)
    rsos = (x * x).sum(-1).astype(np.float32)
    plain = ar.kv_append_ref(x, cache.copy(), offs, 1e-6)
    normed = ar.kv_append_ref(x, cache.copy(), offs, 1e-6, x_rsos=rsos)
    return dict(x=x, cache=cache, cache_offsets=offs, x_rsos=rsos, eps=np.float32(1e-6), expected_plain=plain, expected_rmsnorm=normed)


def rope_fixture():
    """Head dim 256, GQA 8:2, a 5-token chunk per slot at positions up to 30000, ring of 11 rows (wraps), one slot off phase."""
    rng = np.random.default_rng(23)
    B, H, G, t, D, T = 3, 8, 2, 5, 256, 11
    q = rng.standard_normal((B, H, t, D)).astype(np.float32)
    k = rng.standard_normal((B, G, t, D)).astype(np.float32)
    v = rng.standard_normal((B, G, t, D)).astype(np.float32)
    freqs = rr.populate_rope_frequencies_ref(D // 2, 1e6).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    offs = np.array([0, 29998, 8], np.int32)
    phase = np.array([1, 1, 2], np.uint8)
    kc = rng.standard_normal((B, G, T, D)).astype(np.float16)
    vc = rng.standard_normal((B, G, T, D)).astype(np.float16)
    q_rsos, k_rsos, v_rsos = ((x * x).sum(-1).astype(np.float32) for x in (q, k, v))
    kc_out, vc_out = kc.copy(), vc.copy()
    q_rot, k_rot = rr.rope_append_ref(q, k, v, freqs, offs, q_rsos, k_rsos, v_rsos, qw, kw, 1e-6, kc_out, vc_out, phase, 1)
    return dict(q=q, k=k, v=v, rope_freqs=freqs, cache_offsets=offs, user_phase=phase, q_rsos=q_rsos, k_rsos=k_rsos, v_rsos=v_rsos,
                q_rmsnorm_w=qw, k_rmsnorm_w=kw, eps=np.float32(1e-6), k_cache=kc, v_cache=vc, phase=np.int32(1),
                expected_q=q_rot, expected_k=k_rot, expected_k_cache=kc_out, expected_v_cache=vc_out)


def main():
    for name in CASES:
        np.savez_compressed(os.path.join(HERE, f"attn_{name}.npz"), **build(name))
    np.savez_compressed(os.path.join(HERE, "kv_append_ref_case.npz"), **kv_append_fixture())
    np.savez_compressed(os.path.join(HERE, "rope_append_case.npz"), **rope_fixture())
    print("wrote", len(CASES) + 2, "fixtures to", HERE)


if __name__ == "__main__":
    main()
