"""The committed fixtures under tests/golden/: the oracle must reproduce them (CPU), the kernels must match them (GPU)."""

import glob
import os

import numpy as np
import pytest

from oracle import attention_ref as ar
from oracle import rope_ref as rr

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ATTN = sorted(glob.glob(os.path.join(GOLDEN, "attn_*.npz")))


def test_fixtures_present():
    assert len(ATTN) >= 5 and os.path.exists(os.path.join(GOLDEN, "kv_append_ref_case.npz"))
    assert os.path.exists(os.path.join(GOLDEN, "rope_append_case.npz"))


@pytest.mark.parametrize("path", ATTN, ids=[os.path.basename(p)[5:-4] for p in ATTN])
def test_oracle_reproduces_fixture(path):
    f = np.load(path)
    qw = int(f["query_window"]) or None
    band = int(f["on_band_block"]) if "on_band_block" in f else None
    out = np.full(f["expected"].shape, 777.0)
    got = ar.attention_ref(
        f["q"], f["k_cache"], f["v_cache"], f["time_dim_sizes"], f["user_phase"], int(f["ctx_window_size"]),
        int(f["phase"]), stage=int(f["stage"]), scale=float(f["scale"]), query_window=qw, out=out, on_band_block=band,
    )
    assert np.array_equal(got.astype(np.float32), f["expected"])
    # skipped slots keep the sentinel, everything else is finite
    assert np.isfinite(f["expected"]).all()


def test_oracle_reproduces_kv_append_fixture():
    f = np.load(os.path.join(GOLDEN, "kv_append_ref_case.npz"))
    plain = ar.kv_append_ref(f["x"], f["cache"].copy(), f["cache_offsets"], float(f["eps"]))
    assert np.array_equal(plain, f["expected_plain"])
    normed = ar.kv_append_ref(f["x"], f["cache"].copy(), f["cache_offsets"], float(f["eps"]), x_rsos=f["x_rsos"])
    assert np.array_equal(normed, f["expected_rmsnorm"])


@pytest.mark.gpu
@pytest.mark.parametrize("path", ATTN, ids=[os.path.basename(p)[5:-4] for p in ATTN])
@pytest.mark.parametrize("split", [False, True])
def test_kernels_match_fixture(gpu_device, path, split):
    import torch

    from g4b_amd.kernels.fa2 import flash_attention
    from helpers import assert_close, partials

    f = np.load(path)
    t = lambda name: torch.from_numpy(f[name]).to(gpu_device)
    q, k, v = t("q"), t("k_cache"), t("v_cache")
    B, H, Tq, D = q.shape
    o = torch.full((B, H, Tq, D), 777.0, dtype=torch.float16, device=gpu_device)
    decode_shaped = (H // k.shape[1]) * Tq <= 16
    # decode-shaped launches split their keys when the partial buffers are passed; prefill-shaped ones split by
    # themselves when the shape would underfill the chip unless workspace=False forbids it
    parts = partials(4, B, H, Tq, D) if split and decode_shaped else ()
    extra = {} if split or decode_shaped else {"workspace": False}
    flash_attention(
        q, k, v, o, t("time_dim_sizes"), t("user_phase"), int(f["ctx_window_size"]), int(f["phase"]), *parts,
        stage=int(f["stage"]), scale=float(f["scale"]), query_window=int(f["query_window"]) or None,
        on_band_block=int(f["on_band_block"]) if "on_band_block" in f else None, **extra,
    )
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), f["expected"], what=os.path.basename(path))


@pytest.mark.gpu
def test_kv_append_matches_fixture(gpu_device):
    import torch

    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache

    f = np.load(os.path.join(GOLDEN, "kv_append_ref_case.npz"))
    t = lambda name: torch.from_numpy(f[name]).to(gpu_device)
    cache = t("cache")
    add_kv_to_cache(t("x"), cache, t("cache_offsets"), float(f["eps"]))
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), f["expected_plain"])
    cache = t("cache")
    add_kv_to_cache(t("x"), cache, t("cache_offsets"), float(f["eps"]), t("x_rsos"))
    torch.cuda.synchronize()
    got, exp = cache.cpu().numpy().astype(np.float32), f["expected_rmsnorm"].astype(np.float32)
    np.testing.assert_allclose(got, exp, rtol=1e-3, atol=1e-6)
    assert np.array_equal(got == f["cache"].astype(np.float32), exp == f["cache"].astype(np.float32))


def _rope_fixture():
    return np.load(os.path.join(GOLDEN, "rope_append_case.npz"))


def test_oracle_reproduces_rope_fixture():
    f = _rope_fixture()
    kc, vc = f["k_cache"].copy(), f["v_cache"].copy()
    q_rot, k_rot = rr.rope_append_ref(f["q"], f["k"], f["v"], f["rope_freqs"], f["cache_offsets"], f["q_rsos"], f["k_rsos"], f["v_rsos"],
                                      f["q_rmsnorm_w"], f["k_rmsnorm_w"], float(f["eps"]), kc, vc, f["user_phase"], int(f["phase"]))
    assert np.array_equal(q_rot, f["expected_q"]) and np.array_equal(k_rot, f["expected_k"])
    assert np.array_equal(kc, f["expected_k_cache"]) and np.array_equal(vc, f["expected_v_cache"])


@pytest.mark.gpu
def test_rope_kernels_match_fixture(gpu_device):
    import torch

    from g4b_amd.kernels.rope import apply_rope, apply_rope_and_append

    f = _rope_fixture()
    t = lambda name: torch.from_numpy(f[name]).to(gpu_device)
    q, k = t("q"), t("k")
    apply_rope(q, k, t("rope_freqs"), t("cache_offsets"), t("q_rsos"), t("k_rsos"), t("q_rmsnorm_w"), t("k_rmsnorm_w"), float(f["eps"]))
    torch.cuda.synchronize()
    np.testing.assert_allclose(q.cpu().numpy(), f["expected_q"], rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(k.cpu().numpy(), f["expected_k"], rtol=2e-5, atol=2e-5)
    q, k, kc, vc = t("q"), t("k"), t("k_cache"), t("v_cache")
    apply_rope_and_append(q, k, t("v"), t("rope_freqs"), t("cache_offsets"), t("q_rsos"), t("k_rsos"), t("v_rsos"), t("q_rmsnorm_w"),
                          t("k_rmsnorm_w"), float(f["eps"]), kc, vc, t("user_phase"), int(f["phase"]))
    torch.cuda.synchronize()
    np.testing.assert_allclose(kc.float().cpu().numpy(), f["expected_k_cache"].astype(np.float32), rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(vc.float().cpu().numpy(), f["expected_v_cache"].astype(np.float32), rtol=2e-3, atol=2e-3)
    assert np.array_equal(kc[2].cpu().numpy(), f["k_cache"][2])  # off-phase slot
