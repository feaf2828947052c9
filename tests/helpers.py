"""Shared helpers of the GPU parity tests: seeded inputs, oracle calls, tolerances."""

from __future__ import annotations

import numpy as np
import torch

from oracle import attention_ref as ar
from oracle import index_spec as ix

# north-star tolerance for fp16 I/O with fp32 accumulation: |got - ref| <= 2e-3 + 1e-2 * |ref|
ATOL_F16, RTOL_F16 = 2e-3, 1e-2
# bf16 caches: 8-bit mantissas on K, V and P; same form, looser constants
ATOL_BF16, RTOL_BF16 = 1.6e-2, 2e-2


def assert_close(got, ref, atol=ATOL_F16, rtol=RTOL_F16, what=""):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - ref)
    bound = atol + rtol * np.abs(ref)
    worst = float((err - bound).max())
    assert worst <= 0, f"{what}: max abs err {err.max():.3e}, worst excess over tolerance {worst:.3e}"


def make_case(B, H, G, Tq, D, kv_ctx, *, seed=0, dtype=torch.float16, device="cuda", q_dtype=None, engine_layout=False):
    """Seeded N(0,1) q / caches.  ``engine_layout``: q and o are permuted views of [B,Tq,H,D] buffers."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    q_dtype = q_dtype or dtype
    if engine_layout:
        q = torch.randn(B, Tq, H, D, generator=gen).to(q_dtype).to(device).permute(0, 2, 1, 3)
        o = torch.full((B, Tq, H, D), 777.0, dtype=q_dtype, device=device).permute(0, 2, 1, 3)
    else:
        q = torch.randn(B, H, Tq, D, generator=gen).to(q_dtype).to(device)
        o = torch.full((B, H, Tq, D), 777.0, dtype=q_dtype, device=device)
    k = torch.randn(B, G, kv_ctx, D, generator=gen).to(dtype).to(device)
    v = torch.randn(B, G, kv_ctx, D, generator=gen).to(dtype).to(device)
    return q, k, v, o


def oracle(q, k, v, tds, phase_arr, W, phase, **kw):
    """fp64 oracle on exactly the values the GPU sees (inputs already rounded to their dtypes)."""
    return ar.attention_ref(
        q.detach().float().cpu().numpy(),
        k.detach().float().cpu().numpy(),
        v.detach().float().cpu().numpy(),
        [int(x) for x in tds],
        [int(x) for x in phase_arr],
        W,
        phase,
        **kw,
    )


def i32(vals, device="cuda"):
    return torch.tensor(list(vals), dtype=torch.int32, device=device)


def u8(vals, device="cuda"):
    return torch.tensor(list(vals), dtype=torch.uint8, device=device)


def partials(S, B, H, Tq, D, device="cuda"):
    """The reference's split buffers (tests/compare_scripts/test_fa2.py:257-284)."""
    return (
        torch.empty(S, B, H, Tq, D, dtype=torch.float16, device=device),
        torch.empty(S, B, H, Tq, dtype=torch.float32, device=device),
        torch.empty(S, B, H, Tq, dtype=torch.float32, device=device),
    )


__all__ = ["ar", "ix", "assert_close", "make_case", "oracle", "i32", "u8", "partials"]
