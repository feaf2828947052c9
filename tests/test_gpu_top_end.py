"""The largest shapes of the reference's own compare script (tests/compare_scripts/test_fa2.py:57,63-76): a ring of
65 536 rows read by one decode token (unwrapped and with the reference's ``tds = W + 17`` wrap, :286-290), a 256-token
chunk on a 65 536-token context, and a one-shot causal prefill of 65 536 tokens, at H = 16, G = 4, D = 256 as listed
there, plus the decode shapes at head dimension 512.  These are the sizes where a 32-bit offset or a corner of the
grid map would show (the reference flags its own int32 risk, g4b/kernels/fa2.py:1-4).

The fp64 oracle runs on sampled rows; the whole output is covered by a closed form (K = 0 makes every row the mean of
its visible V rows, computed on the device in fp64) and by split-against-unsplit agreement.
"""

import numpy as np
import pytest
import torch

from helpers import assert_close, i32, ix, partials, u8

pytestmark = pytest.mark.gpu
H, G = 16, 4
N = 65536


def randn16(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn(shape, generator=g, device="cuda", dtype=torch.float16)


def oracle_rows(q, k, v, b, rows, tds, W, Tq, scale, stage=ix.STAGE_CAUSAL):
    """fp64 attention of the selected query rows of slot b, all heads."""
    kv_ctx = k.shape[2]
    win, start = ix.window_size(tds, W), ix.ring_start(tds, W, kv_ctx)
    idx = (torch.arange(win, device=k.device) + start) % kv_ctx
    kl = k[b][:, idx].double()
    vl = v[b][:, idx].double()
    out = np.zeros((H, len(rows), q.shape[-1]))
    for n, i in enumerate(rows):
        lo, hi = ix.visible_range(i, tds, W, Tq, stage, None)
        for h in range(H):
            g = h // (H // G)
            s = (kl[g, lo:hi] @ q[b, h, i].double()) * scale
            p = torch.exp(s - s.max())
            out[h, n] = ((p / p.sum()) @ vl[g, lo:hi]).cpu().numpy()
    return out


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


@pytest.mark.parametrize("D", [256, 512])
@pytest.mark.parametrize("tds", [N, N + 17], ids=["unwrapped", "wrapped_by_17"])
def test_decode_on_a_ring_of_65536_rows(fa, D, tds):
    print(f"decode ring {N} D={D} tds={tds}", flush=True)
    scale = 1 / 16
    q, k, v = randn16((1, H, 1, D), 1), randn16((1, G, N, D), 2), randn16((1, G, N, D), 3)
    ref = oracle_rows(q, k, v, 0, [0], tds, N, 1, scale)
    outs = {}
    for how in ("unsplit", "workspace", "static", "many_workers"):
        o = torch.full_like(q, 777.0)
        if how == "unsplit":
            fa.flash_attention(q, k, v, o, i32([tds]), u8([2]), N, 2, scale=scale, workspace=False)
        elif how == "workspace":
            ws = torch.empty(fa.workspace_bytes(1, H, G, 1, D), dtype=torch.uint8, device="cuda")
            fa.flash_attention(q, k, v, o, i32([tds]), u8([2]), N, 2, scale=scale, workspace=ws)
        elif how == "static":  # the reference's call: split buffers for 64 splits (test_fa2.py:57), no workspace
            fa.flash_attention(q, k, v, o, i32([tds]), u8([2]), N, 2, *partials(64, 1, H, 1, D), scale=scale)
        else:
            ws = torch.empty(fa.workspace_bytes(1, H, G, 1, D, 5000), dtype=torch.uint8, device="cuda")
            fa.flash_attention(q, k, v, o, i32([tds]), u8([2]), N, 2, scale=scale, workspace=ws, num_workers=5000)
        torch.cuda.synchronize()
        outs[how] = o.float().cpu().numpy()
        assert_close(outs[how][0], ref, what=f"decode ring {N} D={D} tds={tds} {how}")
    for how, got in outs.items():
        assert np.abs(got - outs["unsplit"]).max() <= 5e-4, how


def test_chunk_of_256_tokens_on_a_65536_token_context(fa):
    D, Tq, scale = 256, 256, 1 / 16
    print(f"chunk {Tq} on ring {N}", flush=True)
    q, k, v = randn16((1, H, Tq, D), 4), randn16((1, G, N, D), 5), randn16((1, G, N, D), 6)
    rows = [0, 1, 7, 8, 31, 32, 127, 128, 254, 255]
    for tds in (N, N + 17):
        ref = oracle_rows(q, k, v, 0, rows, tds, N, Tq, scale)
        got = {}
        for how in ("static", "workspace", "unsplit"):
            o = torch.full_like(q, 777.0)
            if how == "static":
                fa.flash_attention(q, k, v, o, i32([tds]), u8([1]), N, 1, scale=scale)
            elif how == "workspace":
                ws = torch.empty(fa.workspace_bytes(1, H, G, Tq, D), dtype=torch.uint8, device="cuda")
                fa.flash_attention(q, k, v, o, i32([tds]), u8([1]), N, 1, scale=scale, workspace=ws)
            else:
                fa.flash_attention(q, k, v, o, i32([tds]), u8([1]), N, 1, scale=scale, workspace=False)
            torch.cuda.synchronize()
            got[how] = o.float()
            assert bool(torch.isfinite(got[how]).all()) and not bool((got[how] == 777.0).any())
            assert_close(got[how][0][:, rows].cpu().numpy(), ref, what=f"chunk on {N} tds={tds} {how}")
        for how in ("static", "workspace"):
            d = (got[how] - got["unsplit"]).abs()
            assert bool((d <= 1e-3 + 4e-3 * got["unsplit"].abs()).all()), (how, d.max().item())


def test_one_shot_causal_prefill_of_65536_tokens(fa):
    D, S, scale = 256, N, 1 / 16
    print(f"one-shot prefill {S}", flush=True)
    q, k, v = randn16((1, H, S, D), 7), randn16((1, G, S, D), 8), randn16((1, G, S, D), 9)
    o = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=scale)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o).all())
    rng = np.random.default_rng(3)
    rows = [0, 1, 7, 8, 63, 64, 4095, 4096, 32767, 32768, 65534, 65535] + rng.integers(0, S, 28).tolist()
    got = o[0][:, rows].float().cpu().numpy()
    assert_close(got, oracle_rows(q, k, v, 0, rows, S, S, S, scale), what="one-shot 65536")
    # closed form on every row: K = 0 makes all visible keys equal, so row i is the mean of V[0 .. i]
    k.zero_()
    o.fill_(777.0)
    fa.flash_attention(q, k, v, o, i32([S]), u8([1]), S, 1, scale=scale)
    torch.cuda.synchronize()
    mean = v[0].double().cumsum(1) / torch.arange(1, S + 1, device="cuda", dtype=torch.float64).view(1, S, 1)  # [G, S, D]
    for h in range(H):
        ref = mean[h // (H // G)]
        d = (o[0, h].double() - ref).abs()
        assert bool((d <= 2e-3 + 1e-2 * ref.abs()).all()), (h, d.max().item())
