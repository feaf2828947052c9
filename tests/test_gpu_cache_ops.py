"""GPU parity of add_kv_to_cache and advance_decode_state: slot mapping must be bit-exact."""

import numpy as np
import pytest
import torch

from helpers import ar, i32, ix, u8

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(gpu_device):
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache
    from g4b_amd.kernels.advance_decode_state import advance_decode_state

    return add_kv_to_cache, advance_decode_state


@pytest.mark.parametrize("x_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("off_dtype", [torch.int64, torch.int32])
def test_kv_append_reference_test_case(ops, x_dtype, cache_dtype, off_dtype):
    """tests/compare_scripts/test_add_kv.py:19-59: B,G,t,T,D = 2,4,7,17,256, offsets [15, 3] (wraps)."""
    add_kv, _ = ops
    B, G, t, T, D = 2, 4, 7, 17, 256
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(B, G, t, D, generator=gen).to(x_dtype)
    cache0 = torch.randn(B, G, T, D, generator=gen).to(cache_dtype)
    offs = torch.tensor([15, 3], dtype=off_dtype)
    eps = 1e-6
    # plain: bit-exact (one rounding into the cache dtype)
    cache = cache0.clone().cuda()
    add_kv(x.cuda(), cache, offs.cuda(), eps)
    torch.cuda.synchronize()
    exp = cache0.clone()
    for b in range(B):
        exp[b][:, (torch.arange(t) + offs[b]) % T, :] = x[b].to(cache_dtype)
    assert torch.equal(cache.cpu(), exp)
    # fused weightless RMSNorm, fp32 math then one rounding
    rsos = (x.float() * x.float()).sum(-1)
    cache = cache0.clone().cuda()
    add_kv(x.cuda(), cache, offs.cuda(), eps, rsos.cuda())
    torch.cuda.synchronize()
    exp_np = ar.kv_append_ref(
        x.float().numpy(), cache0.float().numpy().copy(), offs.numpy(), eps, x_rsos=rsos.numpy()
    )
    exp_t = torch.from_numpy(exp_np).to(cache_dtype)
    got = cache.cpu()
    untouched = torch.ones(T, dtype=torch.bool)
    assert torch.equal(got[0][:, [5, 6, 7, 8, 9, 10, 11, 12, 13, 14]], cache0[0][:, [5, 6, 7, 8, 9, 10, 11, 12, 13, 14]])
    ulp = {torch.float32: 2e-7, torch.float16: 1e-3, torch.bfloat16: 8e-3}[cache_dtype]
    torch.testing.assert_close(got.float(), exp_t.float(), rtol=ulp, atol=ulp * 1e-2)


def test_kv_append_engine_views_and_phase_skip(ops):
    """x as a permuted view of a [B, t, G, D] fp32 scratchpad, rsos as a view of [B, t, G] (gemma4e.py:557-592)."""
    add_kv, _ = ops
    B, G, t, T, D = 5, 2, 512, 1023, 256
    gen = torch.Generator().manual_seed(1)
    xbuf = torch.randn(B, t, G, D, generator=gen)
    x = xbuf.cuda().permute(0, 2, 1, 3)
    rs = (xbuf * xbuf).sum(-1).cuda().permute(0, 2, 1)
    cache0 = torch.randn(B, G, T, D, generator=gen).half()
    offs = [0, 700, 1023 * 3 + 5, 17, 999]
    phase = [1, 1, 1, 2, 0]
    cache = cache0.clone().cuda()
    add_kv(x, cache, i32(offs), 1e-6, rs, user_phase=u8(phase), phase=1)
    torch.cuda.synchronize()
    exp = ar.kv_append_ref(
        xbuf.permute(0, 2, 1, 3).numpy(),
        cache0.numpy().copy(),
        offs,
        1e-6,
        x_rsos=(xbuf * xbuf).sum(-1).permute(0, 2, 1).numpy(),
        user_phase=phase,
        phase=1,
    )
    got = cache.cpu().numpy()
    assert np.array_equal(got[3], cache0[3].numpy()) and np.array_equal(got[4], cache0[4].numpy())
    # rows written: exactly the oracle's rows; values within one fp16 ulp of the fp32 formula
    changed_got = (got != cache0.numpy()).any(-1)
    changed_exp = (exp != cache0.numpy()).any(-1)
    assert np.array_equal(changed_got, changed_exp)
    np.testing.assert_allclose(got.astype(np.float32), exp.astype(np.float32), rtol=1e-3, atol=1e-5)
    # without user_phase nothing is skipped (add_kv_to_cache.py:162-170 default)
    cache = cache0.clone().cuda()
    add_kv(x, cache, i32(offs), 1e-6)
    torch.cuda.synchronize()
    exp = ar.kv_append_ref(xbuf.permute(0, 2, 1, 3).numpy(), cache0.numpy().copy(), offs, 1e-6)
    assert np.array_equal(cache.cpu().numpy(), exp)


def test_kv_append_rejects_more_tokens_than_ring_rows(ops):
    add_kv, _ = ops
    x = torch.zeros(1, 2, 9, 256, device="cuda")
    cache = torch.zeros(1, 2, 8, 256, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError):  # add_kv_to_cache.py:119
        add_kv(x, cache, i32([0]), 1e-6)


def test_advance_decode_state(ops):
    _, advance = ops
    B, t = 300, 4
    rng = np.random.default_rng(0)
    inp = rng.integers(0, 1000, (t, B)).astype(np.int32)
    out = rng.integers(0, 1000, (B, 1)).astype(np.int32)
    off = rng.integers(0, 30000, B).astype(np.int32)
    tds = off + 1
    ph = rng.integers(0, 3, B).astype(np.uint8)
    d = [torch.from_numpy(a.copy()).cuda() for a in (inp, out, off, tds, ph)]
    advance(*d)
    torch.cuda.synchronize()
    ar.advance_decode_state_ref(inp, out, off, tds, ph)
    assert np.array_equal(d[0].cpu().numpy(), inp)
    assert np.array_equal(d[2].cpu().numpy(), off)
    assert np.array_equal(d[3].cpu().numpy(), tds)
    assert np.array_equal(d[1].cpu().numpy(), out)
