"""fp32 queries as the engine hands them over, compared with the oracle on the UNROUNDED values.

The engine keeps q in fp32 scratchpads (DTA = float32, g4b/models/gemma4e.py:30), RMS-normalises q and k to
norm sqrt(D) times a learned weight, rotates both (g4b/kernels/rope.py:22-40) and calls flash_attention with
scale 1.0 and use_fp32_dot=True (gemma4e.py:593-607); the CPU reference computes softmax(q k^T + mask) v in fp32
(scripts/reference_impl.py:443).  Scores reach +-D at scale 1.0, so a query rounded to the cache's 16-bit type
moves every score by several 1e-3 (fp16) or 1e-2 (bf16) -- enough to leave the tolerance on rows whose weight is
shared by keys with close scores.  With use_fp32_dot=True the kernels feed K Q^T with the query as a hi + lo pair
of 16-bit operands; these tests hold that path to the fp16 tolerance against the oracle on the fp32 query, and
show that the rounded path (use_fp32_dot=False, the reference's q.to(fp16)) equals the oracle on the rounded query.
"""

import numpy as np
import pytest
import torch

from helpers import ATOL_BF16, ATOL_F16, RTOL_BF16, RTOL_F16, ar, assert_close, i32, ix, partials, u8
from oracle import rope_ref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


def engine_inputs(B, H, G, Tq, D, n_ctx, *, seed, clustered, freq_base=1e6, eps=1e-6):
    """fp32 q [B,H,Tq,D] and fp32 k, v streams [B,G,n_ctx,D] the way the engine produces them: RMS-normalised with
    weights near 1, rotated at their absolute positions; v normalised without weights.  ``clustered``: keys are noisy
    copies of a few directions, so that many keys have nearly the same score and the weights are shared."""
    rng = np.random.default_rng(seed)
    if clustered:
        centres = rng.standard_normal((B, G, 6, D))
        pick = rng.integers(0, 6, (B, G, n_ctx))
        k_raw = np.take_along_axis(centres, pick[..., None], 2) + 0.02 * rng.standard_normal((B, G, n_ctx, D))
        q_raw = centres[:, :, :1].repeat(H // G, 1).repeat(Tq, 2) + 0.3 * rng.standard_normal((B, H, Tq, D))
    else:
        k_raw = rng.standard_normal((B, G, n_ctx, D))
        q_raw = rng.standard_normal((B, H, Tq, D))
    v_raw = rng.standard_normal((B, G, n_ctx, D))
    wq = (1.0 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    wk = (1.0 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    freqs = rope_ref.populate_rope_frequencies_ref(D // 2, freq_base).astype(np.float32)
    # keys sit at positions 0..n_ctx-1, queries at the last Tq of them; one rope call per tensor (it rotates a pair)
    zeros = [0] * B
    _, k_rot = rope_ref.apply_rope_ref(np.zeros((B, 1, n_ctx, D), np.float32), k_raw.astype(np.float32), freqs, zeros,
                                       np.ones((B, 1, n_ctx), np.float32), (k_raw**2).sum(-1), wq, wk, eps)
    q_rot, _ = rope_ref.apply_rope_ref(q_raw.astype(np.float32), np.zeros((B, 1, Tq, D), np.float32), freqs, [n_ctx - Tq] * B,
                                       (q_raw**2).sum(-1), np.ones((B, 1, Tq), np.float32), wq, wk, eps)
    v_n = (v_raw / np.sqrt((v_raw**2).mean(-1, keepdims=True) + eps)).astype(np.float32)
    return q_rot.astype(np.float32), k_rot.astype(np.float32), v_n


def place_in_ring(stream, kv_ctx, dtype, dev):
    """[B,G,n,D] token stream -> ring cache [B,G,kv_ctx,D]: position p lives in row p % kv_ctx (fa2.py:54,75)."""
    B, G, n, D = stream.shape
    cache = torch.zeros(B, G, kv_ctx, D, dtype=dtype, device=dev)
    lo = max(0, n - kv_ctx)
    rows = torch.arange(lo, n) % kv_ctx
    cache[:, :, rows] = torch.from_numpy(stream[:, :, lo:n]).to(dev).to(dtype)
    return cache


def excess(got, ref, atol, rtol):
    err = np.abs(np.asarray(got, np.float64) - ref)
    return float((err - (atol + rtol * np.abs(ref))).max()), float(err.max())


CASES = [
    # name, D, Tq, n_ctx, W, kv_ctx, split
    ("decode_unsplit_d256", 256, 1, 3000, 4096, 4096, False),
    ("decode_split_d256", 256, 1, 3000, 4096, 4096, True),
    ("decode_swa_wrapped_d256", 256, 1, 3000, 512, 1023, False),
    ("decode_split_d512", 512, 1, 3000, 4096, 4096, True),
    ("decode_unsplit_d512", 512, 1, 2000, 4096, 4096, False),
    ("chunk512_on_context_d256", 256, 512, 2048 + 512, 4096, 4096 + 511, False),
    ("chunk512_on_context_d512", 512, 512, 1024 + 512, 4096, 4096 + 511, False),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("clustered", [False, True], ids=["random_keys", "clustered_keys"])
@pytest.mark.parametrize("kv_dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_engine_fp32_query_scale_one(fa, case, clustered, kv_dtype):
    name, D, Tq, n_ctx, W, kv_ctx, split = case
    print(f"case {name} clustered={clustered} kv={kv_dtype}", flush=True)
    dev = "cuda"
    B, H, G = 2, 8, 2
    q32, k32, v32 = engine_inputs(B, H, G, Tq, D, n_ctx, seed=11 + D + Tq, clustered=clustered)
    k_cache = place_in_ring(k32, kv_ctx, kv_dtype, dev)
    v_cache = place_in_ring(v32, kv_ctx, kv_dtype, dev)
    # the engine's layout: q and o are [B, t, H, D] fp32 scratchpads viewed as [B, H, t, D]
    q = torch.from_numpy(q32).to(dev).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    phase_id = ix.PHASE_DECODE if Tq == 1 else ix.PHASE_PREFILL
    tds, phase = [n_ctx] * B, [phase_id] * B
    parts = partials(16, B, H, Tq, D) if split else ()
    kc, vc = k_cache.float().cpu().numpy(), v_cache.float().cpu().numpy()
    ref = ar.attention_ref(q32, kc, vc, tds, phase, W, phase_id, scale=1.0)
    atol, rtol = (ATOL_F16, RTOL_F16) if kv_dtype == torch.float16 else (ATOL_BF16, RTOL_BF16)

    # use_fp32_dot=True: parity with the oracle on the fp32 query
    o = torch.full((B, Tq, H, D), 777.0, device=dev).permute(0, 2, 1, 3)
    fa.flash_attention(q, k_cache, v_cache, o, i32(tds), u8(phase), W, phase_id, *parts, use_grouped_query_tile=True,
                       use_fp32_dot=True)
    torch.cuda.synchronize()
    got = o.cpu().numpy()
    ex, worst = excess(got, ref, atol, rtol)
    print(f"  use_fp32_dot=True : max abs err {worst:.3e}, worst excess over tolerance {ex:.3e}", flush=True)
    assert_close(got, ref, atol=atol, rtol=rtol, what=f"{name} fp32 q, use_fp32_dot=True")

    # use_fp32_dot=False: the query is rounded to the cache type first (fa2.py:88); equal to the oracle on that query
    o2 = torch.full((B, Tq, H, D), 777.0, device=dev).permute(0, 2, 1, 3)
    fa.flash_attention(q, k_cache, v_cache, o2, i32(tds), u8(phase), W, phase_id, *parts, use_grouped_query_tile=True,
                       use_fp32_dot=False)
    torch.cuda.synchronize()
    got2 = o2.cpu().numpy()
    q_rounded = torch.from_numpy(q32).to(kv_dtype).float().numpy()
    ref2 = ar.attention_ref(q_rounded, kc, vc, tds, phase, W, phase_id, scale=1.0)
    assert_close(got2, ref2, atol=atol, rtol=rtol, what=f"{name} fp32 q rounded, use_fp32_dot=False")
    ex2, worst2 = excess(got2, ref, atol, rtol)
    print(f"  use_fp32_dot=False: against the unrounded oracle max abs err {worst2:.3e}, worst excess {ex2:.3e}", flush=True)


def test_fp16_query_over_bf16_cache_is_split_too(fa):
    """A query type wider than the cache type is any of f32/f16 over bf16: with use_fp32_dot the fp16 query keeps its
    11 bits against a bf16 cache."""
    B, H, G, D, Tq, n_ctx, W = 2, 8, 2, 256, 1, 1500, 2048
    q32, k32, v32 = engine_inputs(B, H, G, Tq, D, n_ctx, seed=5, clustered=True)
    k_cache = place_in_ring(k32, W, torch.bfloat16, "cuda")
    v_cache = place_in_ring(v32, W, torch.bfloat16, "cuda")
    q = torch.from_numpy(q32).cuda().half()
    o = torch.empty_like(q)
    tds, phase = [n_ctx] * B, [2] * B
    fa.flash_attention(q, k_cache, v_cache, o, i32(tds), u8(phase), W, 2, use_fp32_dot=True)
    torch.cuda.synchronize()
    ref = ar.attention_ref(q.float().cpu().numpy(), k_cache.float().cpu().numpy(), v_cache.float().cpu().numpy(), tds, phase, W, 2)
    assert_close(o.float().cpu().numpy(), ref, atol=ATOL_BF16, rtol=RTOL_BF16, what="fp16 q over bf16 cache")
    ex, worst = excess(o.float().cpu().numpy(), ref, ATOL_F16, RTOL_F16)
    print(f"fp16 q over bf16 cache: max abs err {worst:.3e}, excess over the fp16 tolerance {ex:.3e}", flush=True)
