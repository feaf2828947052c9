"""Pins of the rope / q-k RMSNorm restatement (oracle/rope_ref.py) that do not need the reference."""

import numpy as np
import torch

from oracle import rope_ref as rr


def _case(B=3, H=4, G=2, t=5, D=16, seed=0):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, H, t, D)).astype(np.float32)
    k = rng.standard_normal((B, G, t, D)).astype(np.float32)
    freqs = rr.populate_rope_frequencies_ref(D // 2, 10000.0).astype(np.float32)
    offs = rng.integers(0, 5000, B).astype(np.int32)
    qw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    return q, k, freqs, offs, (q * q).sum(-1), (k * k).sum(-1), qw, kw


def test_rotation_is_complex_multiplication_and_norm_is_the_textbook_rmsnorm():
    q, k, freqs, offs, q_rsos, k_rsos, qw, kw = _case()
    eps = 1e-6
    q_rot, k_rot = rr.apply_rope_ref(q, k, freqs, offs, q_rsos, k_rsos, qw, kw, eps)
    for x, w, y in ((q, qw, q_rot), (k, kw, k_rot)):
        D = x.shape[-1]
        xn = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + eps) * w
        z = xn[..., : D // 2] + 1j * xn[..., D // 2 :]
        pos = offs.astype(np.int64)[:, None] + np.arange(x.shape[2])[None, :]
        theta = (pos.astype(np.float32)[:, :, None] * freqs[None, None, :]).astype(np.float64)  # the fp32 angle
        zr = z * np.exp(1j * theta)[:, None, :, :]
        want = np.concatenate([zr.real, zr.imag], -1)
        assert np.abs(y - want).max() < 2e-6


def test_pairs_keep_their_norm_and_angle_zero_is_the_identity():
    q, k, freqs, offs, q_rsos, k_rsos, qw, kw = _case(seed=1)
    ones = np.ones_like(qw)
    # rsos = D and eps = 0 switch the normalisation off
    D = q.shape[-1]
    q_rot, k_rot = rr.apply_rope_ref(q, k, freqs, offs, np.full(q.shape[:3], D, np.float32), np.full(k.shape[:3], D, np.float32), ones, ones, 0.0)
    for x, y in ((q, q_rot), (k, k_rot)):
        n_in = x[..., : D // 2] ** 2 + x[..., D // 2 :] ** 2
        n_out = y[..., : D // 2] ** 2 + y[..., D // 2 :] ** 2
        assert np.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)
    q0, k0 = rr.apply_rope_ref(q[:, :, :1], k[:, :, :1], freqs, np.zeros(3, np.int32), np.full(q.shape[:2] + (1,), D, np.float32),
                               np.full(k.shape[:2] + (1,), D, np.float32), ones, ones, 0.0)
    assert np.array_equal(q0, q[:, :, :1]) and np.array_equal(k0, k[:, :, :1])


def test_matches_the_cpu_reference_models_formulation():
    """scripts/reference_impl.py:249-263 restated with torch: x*cos + rotate_half(x)*sin, theta duplicated to full width."""
    q, k, freqs, offs, q_rsos, k_rsos, qw, kw = _case(B=1, t=7, seed=2)
    D = q.shape[-1]
    ones = np.ones(D, np.float32)
    q_rot, k_rot = rr.apply_rope_ref(q, k, freqs, offs, np.full(q.shape[:3], D, np.float32), np.full(k.shape[:3], D, np.float32), ones, ones, 0.0)
    T = q.shape[2]
    theta = torch.arange(int(offs[0]), int(offs[0]) + T).reshape(T, 1) * torch.from_numpy(freqs)
    theta = torch.cat([theta, theta], dim=-1)
    sin, cos = theta.sin(), theta.cos()

    def rotate_half(x):
        return torch.cat([-x[..., D // 2 :], x[..., : D // 2]], dim=-1)

    for x, y in ((q, q_rot), (k, k_rot)):
        xt = torch.from_numpy(x)
        want = xt * cos + rotate_half(xt) * sin
        assert np.abs(y - want.numpy()).max() < 2e-6


def test_frequencies_follow_the_power_law():
    f = rr.populate_rope_frequencies_ref(64, 1e6)
    assert f[0] == 1.0 and np.allclose(f[1:] / f[:-1], 1e6 ** (-1 / 64))
    s = np.linspace(1, 2, 64)
    assert np.allclose(rr.populate_rope_frequencies_ref(64, 1e6, s), f / s)
    # the reference model's expression (reference_impl.py:243): 1 / base ** (arange(0, dim, 2) / dim), dim = 2n
    want = 1.0 / (1e6 ** (torch.arange(0, 128, 2) / 128))
    assert np.allclose(f, want.numpy(), rtol=1e-6)


def test_append_composition_writes_rotated_k_and_normalised_v_to_the_ring():
    rng = np.random.default_rng(3)
    B, H, G, t, D, T = 2, 4, 2, 3, 8, 7
    q, k, freqs, offs, q_rsos, k_rsos, qw, kw = _case(B, H, G, t, D, seed=3)
    v = rng.standard_normal((B, G, t, D)).astype(np.float32)
    v_rsos = (v * v).sum(-1)
    offs = np.array([5, 12], np.int32)
    kc = np.full((B, G, T, D), 9.0, np.float16)
    vc = np.full((B, G, T, D), 9.0, np.float16)
    q_rot, k_rot = rr.rope_append_ref(q, k, v, freqs, offs, q_rsos, k_rsos, v_rsos, qw, kw, 1e-6, kc, vc, np.array([1, 2], np.uint8), 1)
    for tt in range(t):
        row = (tt + 5) % T
        assert np.array_equal(kc[0, :, row], k_rot[0, :, tt].astype(np.float16))
        vn = v[0, :, tt] / np.sqrt((v[0, :, tt] ** 2).mean(-1, keepdims=True) + 1e-6)
        assert np.abs(vc[0, :, row].astype(np.float32) - vn).max() < 2e-3
    assert (kc[1] == 9.0).all() and (vc[1] == 9.0).all()  # off-phase slot untouched
