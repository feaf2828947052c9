"""GPU parity of apply_rope (and of the launch that also appends K and V to the rings) against oracle/rope_ref.py.

Shapes follow the reference's compare script (tests/compare_scripts/test_rope.py: head dim 256 and 512, GQA groups,
decode t = 1 and prefill chunks) scaled to seconds of CPU time; positions reach tens of thousands so that the fp32
angle and the range reduction of sin / cos matter.
"""

import numpy as np
import pytest
import torch

from helpers import i32, u8
from oracle import rope_ref as rr

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rope(gpu_device):
    from g4b_amd.kernels import rope

    return rope


def _case(B, H, G, t, D, seed, dtype=torch.float32, engine_layout=False):
    gen = torch.Generator().manual_seed(seed)
    if engine_layout:  # [B, t, heads, D] scratchpads viewed as [B, heads, t, D] (gemma4e.py:557-560)
        q = torch.randn(B, t, H, D, generator=gen).to(dtype).cuda().permute(0, 2, 1, 3)
        k = torch.randn(B, t, G, D, generator=gen).to(dtype).cuda().permute(0, 2, 1, 3)
    else:
        q = torch.randn(B, H, t, D, generator=gen).to(dtype).cuda()
        k = torch.randn(B, G, t, D, generator=gen).to(dtype).cuda()
    freqs = torch.from_numpy(rr.populate_rope_frequencies_ref(D // 2, 1e6).astype(np.float32)).cuda()
    qw = (1 + 0.1 * torch.randn(D, generator=gen)).cuda()
    kw = (1 + 0.1 * torch.randn(D, generator=gen)).cuda()
    q_rsos = (q.float() ** 2).sum(-1)
    k_rsos = (k.float() ** 2).sum(-1)
    return q, k, freqs, q_rsos, k_rsos, qw, kw


def _np(x):
    return x.float().cpu().numpy()


CASES = [
    # name, B, H, G, t, D, offsets
    ("decode_d256", 4, 8, 2, 1, 256, [0, 1, 4095, 32767]),
    ("decode_d512", 2, 8, 2, 1, 512, [17, 100000]),
    ("chunk_d256", 2, 8, 2, 96, 256, [0, 16384]),
    ("chunk_ragged_d128", 3, 4, 4, 37, 128, [5, 999, 20000]),
    ("chunk_d64", 1, 2, 1, 300, 64, [123]),
    # D / 16 does not divide the 256 threads of a workgroup: the spare threads must stay out of the next block's token
    ("chunk_d96", 2, 4, 2, 130, 96, [7, 3000]),
    ("chunk_d160", 1, 4, 1, 77, 160, [41]),
    # 138 token blocks of 8 tokens, the last one ragged: enough blocks for the launch to deal them unevenly to the
    # workgroups of even and odd XCDs
    ("prompt_d256", 1, 8, 2, 1100, 256, [3]),
    ("prompt_two_slots_d128", 2, 4, 2, 2100, 128, [0, 50000]),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("layout", ["plain", "engine"])
def test_apply_rope_matches_oracle(rope, case, layout):
    name, B, H, G, t, D, offs = case
    q, k, freqs, q_rsos, k_rsos, qw, kw = _case(B, H, G, t, D, seed=21, engine_layout=(layout == "engine"))
    q_ref, k_ref = rr.apply_rope_ref(_np(q), _np(k), _np(freqs), np.array(offs), _np(q_rsos), _np(k_rsos), _np(qw), _np(kw), 1e-6)
    rope.apply_rope(q, k, freqs, i32(offs), q_rsos, k_rsos, qw, kw, 1e-6)
    torch.cuda.synchronize()
    # fp32 in, fp32 out: a few ulps of the products (sin / cos of the same fp32 angle, fused multiply-adds may differ)
    np.testing.assert_allclose(_np(q), q_ref, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(_np(k), k_ref, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)])
def test_apply_rope_on_16_bit_scratchpads(rope, dtype, tol):
    B, H, G, t, D = 2, 8, 2, 33, 256
    q, k, freqs, q_rsos, k_rsos, qw, kw = _case(B, H, G, t, D, seed=22, dtype=dtype)
    offs = [7, 9000]
    q_ref, k_ref = rr.apply_rope_ref(_np(q), _np(k), _np(freqs), np.array(offs), _np(q_rsos), _np(k_rsos), _np(qw), _np(kw), 1e-6)
    rope.apply_rope(q, k, freqs, i32(offs), q_rsos, k_rsos, qw, kw, 1e-6)
    torch.cuda.synchronize()
    np.testing.assert_allclose(_np(q), q_ref, rtol=tol, atol=tol)
    np.testing.assert_allclose(_np(k), k_ref, rtol=tol, atol=tol)


@pytest.mark.parametrize("Dv", [256, 128, 512])
@pytest.mark.parametrize("cache_dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("t,T", [(40, 97), (1030, 1200)], ids=["chunk", "prompt"])
def test_fused_append_equals_rope_then_two_appends(rope, Dv, cache_dtype, t, T):
    """One launch == apply_rope + add_kv_to_cache(k) + add_kv_to_cache(v, v_rsos) with phase skip and ring wrap (the
    prompt-sized case has enough token blocks for the uneven deal between even and odd XCDs)."""
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache

    B, H, G, D = 4, 8, 2, 256
    q, k, freqs, q_rsos, k_rsos, qw, kw = _case(B, H, G, t, D, seed=23, engine_layout=True)
    gen = torch.Generator().manual_seed(24)
    v = torch.randn(B, t, G, Dv, generator=gen).cuda().permute(0, 2, 1, 3)
    v_rsos = (v ** 2).sum(-1)
    offs = i32([0, 80, T * 5 + T - 7, 3])
    phase = u8([1, 1, 1, 2])
    kc0 = torch.randn(B, G, T, D, generator=gen).to(cache_dtype).cuda()
    vc0 = torch.randn(B, G, T, Dv, generator=gen).to(cache_dtype).cuda()

    # three launches
    q3, k3 = q.clone(), k.clone()
    kc3, vc3 = kc0.clone(), vc0.clone()
    rope.apply_rope(q3, k3, freqs, offs, q_rsos, k_rsos, qw, kw, 1e-6)
    add_kv_to_cache(k3, kc3, offs, 1e-6, user_phase=phase, phase=1)
    add_kv_to_cache(v, vc3, offs, 1e-6, v_rsos, user_phase=phase, phase=1)
    # one launch
    q1, k1 = q.clone(), k.clone()
    kc1, vc1 = kc0.clone(), vc0.clone()
    rope.apply_rope_and_append(q1, k1, v, freqs, offs, q_rsos, k_rsos, v_rsos, qw, kw, 1e-6, kc1, vc1, phase, 1)
    torch.cuda.synchronize()
    assert torch.equal(q1, q3)
    assert torch.equal(kc1, kc3) and torch.equal(vc1, vc3)  # same arithmetic, same single rounding
    assert torch.equal(k1, k)  # the K scratchpad is left alone ...
    k1b, kc1b, vc1b = k.clone(), kc0.clone(), vc0.clone()
    rope.apply_rope_and_append(q.clone(), k1b, v, freqs, offs, q_rsos, k_rsos, v_rsos, qw, kw, 1e-6, kc1b, vc1b, phase, 1, k_writeback=True)
    torch.cuda.synchronize()
    assert torch.equal(k1b, k3) and torch.equal(kc1b, kc3)  # ... unless asked for
    # and against the oracle's composition
    kc_ref, vc_ref = kc0.float().cpu().numpy().copy(), vc0.float().cpu().numpy().copy()
    rr.rope_append_ref(_np(q), _np(k), _np(v), _np(freqs), offs.cpu().numpy(), _np(q_rsos), _np(k_rsos), _np(v_rsos), _np(qw), _np(kw),
                       1e-6, kc_ref, vc_ref, phase.cpu().numpy(), 1)
    tol = 2e-3 if cache_dtype == torch.float16 else 1.6e-2
    np.testing.assert_allclose(_np(kc1), kc_ref, rtol=tol, atol=tol)
    np.testing.assert_allclose(_np(vc1), vc_ref, rtol=tol, atol=tol)
    assert torch.equal(kc1[3], kc0[3]) and torch.equal(vc1[3], vc0[3])  # off-phase slot


def test_rope_frequencies(rope):
    for n, base, scal in ((128, 1e6, False), (256, 1e4, True), (32, 5e5, False)):
        out = torch.empty(n, device="cuda")
        s = torch.linspace(1, 8, n).cuda() if scal else None
        rope.populate_rope_frequencies(out, s, base)
        torch.cuda.synchronize()
        ref = rr.populate_rope_frequencies_ref(n, base, None if s is None else s.cpu().numpy())
        np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=3e-6)


def test_partial_rotary_through_infinite_frequency_scalars(rope):
    """tests/compare_scripts/test_rope.py:24-25: scalars of -inf on the upper half of the frequencies turn them into
    -0.0, i.e. those column pairs are normalised but not rotated."""
    B, H, G, t, D = 1, 48, 48, 1, 512
    q, k, _, q_rsos, k_rsos, qw, kw = _case(B, H, G, t, D, seed=26)
    scal = torch.cat([torch.ones(D // 4), torch.full((D // 4,), float("-inf"))]).cuda()
    freqs = torch.empty(D // 2, device="cuda")
    rope.populate_rope_frequencies(freqs, scal, 100000.0)
    torch.cuda.synchronize()
    assert bool((freqs[D // 4 :] == 0).all())
    offs = [31337]
    q_ref, k_ref = rr.apply_rope_ref(_np(q), _np(k), _np(freqs), np.array(offs), _np(q_rsos), _np(k_rsos), _np(qw), _np(kw), 1e-6)
    q_in = q.clone()
    rope.apply_rope(q, k, freqs, i32(offs), q_rsos, k_rsos, qw, kw, 1e-6)
    torch.cuda.synchronize()
    np.testing.assert_allclose(_np(q), q_ref, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(_np(k), k_ref, rtol=2e-5, atol=2e-5)
    # unrotated columns: x * inv_rms * w exactly
    inv = 1.0 / torch.sqrt(q_rsos / D + 1e-6)
    want = q_in[..., D // 4 : D // 2] * (inv[..., None] * qw[D // 4 : D // 2])
    assert torch.allclose(q[..., D // 4 : D // 2], want, rtol=1e-6, atol=1e-7)


def test_rope_argument_errors(rope):
    q, k, freqs, q_rsos, k_rsos, qw, kw = _case(2, 4, 2, 3, 64, seed=25)
    offs = i32([0, 1])
    with pytest.raises(ValueError):  # rope.py:149
        rope.apply_rope(q, k, freqs[:-1], offs, q_rsos, k_rsos, qw, kw, 1e-6)
    with pytest.raises(ValueError):  # rope.py:152-153
        rope.apply_rope(q, k[:, :, :2], freqs, offs, q_rsos, k_rsos[:, :, :2], qw, kw, 1e-6)
    with pytest.raises(ValueError):  # rope.py:157-159
        rope.apply_rope(q, k, freqs, offs, q_rsos[:, :1], k_rsos, qw, kw, 1e-6)
    with pytest.raises(ValueError):
        rope.apply_rope(q, k, freqs, offs.long(), q_rsos, k_rsos, qw, kw, 1e-6)
    q40 = torch.zeros(2, 4, 3, 40, device="cuda")
    with pytest.raises(NotImplementedError):  # head dim not a multiple of 16
        rope.apply_rope(q40, q40[:, :2].clone(), torch.zeros(20, device="cuda"), offs, q_rsos, k_rsos, torch.ones(40, device="cuda"),
                        torch.ones(40, device="cuda"), 1e-6)
