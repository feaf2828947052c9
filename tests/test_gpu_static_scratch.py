"""Launches through the library's static scratch against the fp64 oracle and against the same launch with a
caller-owned workspace: decode launches short and long (the one-kernel variant for short windows, the flat worker
list with its merge kernel), prefill shapes that split keys, prompts cut into key spans.  Every case is launched
several times in a row and the shapes alternate, so each launch runs over what the previous ones left in the array.
"""

import numpy as np
import pytest
import torch

from helpers import ATOL_BF16, RTOL_BF16, assert_close, i32, ix, make_case, oracle, partials, u8

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


def static_and_workspace(fa, q, k, v, tds, phase, W, phase_id, parts=(), repeats=3, **kw):
    """Outputs of `repeats` launches through the static scratch and of one launch with a workspace."""
    B, H, Tq, D = q.shape
    G = k.shape[1]
    need = fa.workspace_bytes(B, H, G, Tq, D, kw.get("num_workers", 0))
    assert need > 0, "the shape must be one that splits keys"
    outs = []
    for _ in range(repeats):
        o = torch.full_like(q, 777.0)
        fa.flash_attention(q, k, v, o, tds, phase, W, phase_id, *parts, workspace="static", **kw)
        outs.append(o)
    ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    o_ws = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o_ws, tds, phase, W, phase_id, *parts, workspace=ws, **kw)
    torch.cuda.synchronize()
    return outs, o_ws


@pytest.mark.parametrize("D,dtype", [(128, torch.float16), (256, torch.float16), (256, torch.bfloat16), (512, torch.float16)])
@pytest.mark.parametrize("Tq,R", [(1, 4), (2, 4), (1, 1), (3, 5), (4, 4)])
def test_decode_batches_through_the_static_scratch(fa, D, dtype, Tq, R):
    if R * Tq > 16:
        pytest.skip("not decode-shaped")
    G, B, W = 2, 7, 2200
    H = G * R
    print(f"fused decode D={D} {dtype} Tq={Tq} R={R}", flush=True)
    q, k, v, _ = make_case(B, H, G, Tq, D, W, seed=D + Tq + R, dtype=dtype)
    #          full ring, short, one tile, empty but in phase, off phase, wrapped, exactly Tq keys
    tds = [W, 300, max(Tq, 20), 0, 900, W + 17, Tq]
    phase = [2, 2, 2, 2, 1, 2, 2]
    for nw in (0, 37, 300):
        outs, o_ws = static_and_workspace(fa, q, k, v, i32(tds), u8(phase), W, 2, partials(8, B, H, Tq, D), scale=0.0625,
                                          num_workers=nw)
        ref = oracle(q, k, v, tds, phase, W, 2, scale=0.0625)
        tol = dict(atol=ATOL_BF16, rtol=RTOL_BF16) if dtype == torch.bfloat16 else {}
        sentinel = float(torch.tensor(777.0, dtype=dtype))  # what the output tensors were filled with
        for n, o in enumerate(outs):
            got = o.float().cpu().numpy()
            for b in range(B):
                if phase[b] != 2:
                    assert (got[b] == sentinel).all(), f"off-phase slot {b} was written (launch {n})"
                elif tds[b] == 0:
                    assert (got[b] == 0.0).all(), f"empty in-phase slot {b} must read zeros (launch {n})"
                else:
                    assert_close(got[b], ref[b], what=f"slot {b} launch {n} nw={nw}", **tol)
            assert torch.equal(o, outs[0]), f"launch {n} differs from launch 0"
        d = (outs[0].float() - o_ws.float()).abs()
        assert float(d.max()) <= (2e-2 if dtype == torch.bfloat16 else 2e-3), float(d.max())


@pytest.mark.parametrize("B,G,R,Tq,W,D", [
    (1, 2, 4, 1, 2048, 256),    # one sequence of 2048 keys: 128 workers of one tile
    (1, 2, 4, 1, 8192, 256),
    (1, 2, 4, 1, 8200, 256),
    (1, 1, 8, 2, 3000, 128),    # one pair, sixteen rows
    (4, 2, 4, 1, 1024, 128),    # the reference's decode_small_w1024
    (40, 4, 4, 1, 700, 256),    # 160 pairs
    (9, 2, 1, 3, 1500, 256),
    (3, 2, 4, 4, 640, 256),
])
def test_short_decode_launches_through_the_static_scratch(fa, B, G, R, Tq, W, D):
    H = G * R
    print(f"short decode launch B={B} G={G} R={R} Tq={Tq} W={W} D={D}", flush=True)
    q, k, v, _ = make_case(B, H, G, Tq, D, W, seed=B + W + D)
    rng = np.random.default_rng(B * W)
    tds = [W] + [int(x) for x in rng.integers(Tq, W + 40, B - 1)]
    phase = [2] * B
    if B > 2:
        phase[1], tds[2] = 1, 0  # an off-phase slot and an empty in-phase one
    ref = oracle(q, k, v, tds, phase, W, 2, scale=0.0625)
    for win in (None, [max(Tq, W // (b + 1)) for b in range(B)]):
        kw = {} if win is None else {"window_sizes": i32(win)}
        ref_w = ref if win is None else oracle(q, k, v, tds, phase, W, 2, scale=0.0625, window_sizes=win)
        outs, o_ws = static_and_workspace(fa, q, k, v, i32(tds), u8(phase), W, 2, partials(8, B, H, Tq, D), scale=0.0625, **kw)
        for n, o in enumerate(outs):
            got = o.float().cpu().numpy()
            for b in range(B):
                if phase[b] != 2:
                    assert (got[b] == 777.0).all()
                elif tds[b] == 0:
                    assert (got[b] == 0.0).all()
                else:
                    assert_close(got[b], ref_w[b], what=f"slot {b} launch {n} win={win is not None}")
            assert torch.equal(o, outs[0]), f"launch {n} differs from launch 0"
        assert float((outs[0].float() - o_ws.float()).abs().max()) <= 2e-3


@pytest.mark.parametrize("D", [128, 256, 512])
def test_prefill_key_splits_through_the_static_scratch(fa, D):
    H, G = 8, 2
    for Tq, ctx, B, seed in ((256, 3000, 3, 1), (96, 700, 2, 2), (512, 5000, 1, 3), (40, 64, 4, 4)):
        print(f"fused chunk D={D} Tq={Tq} ctx={ctx} B={B}", flush=True)
        kv_ctx = ctx + Tq + 64
        q, k, v, _ = make_case(B, H, G, Tq, D, kv_ctx, seed=seed)
        tds = [ctx + Tq] + [Tq, 0, ctx // 2 + Tq][: B - 1]
        phase = [1] + [1, 2, 1][: B - 1]
        outs, o_ws = static_and_workspace(fa, q, k, v, i32(tds), u8(phase), kv_ctx, 1, scale=0.0625)
        ref = oracle(q, k, v, tds, phase, kv_ctx, 1, scale=0.0625)
        for n, o in enumerate(outs):
            got = o.float().cpu().numpy()
            for b in range(B):
                if phase[b] != 1:
                    assert (got[b] == 777.0).all()
                else:
                    assert_close(got[b], ref[b], what=f"chunk D={D} Tq={Tq} slot {b} launch {n}")
            assert torch.equal(o, outs[0]), f"launch {n} differs from launch 0"
        assert torch.equal(outs[0], o_ws), "same kernels, same partition: the scratch's address must not matter"


@pytest.mark.parametrize("S", [1408, 2048, 3072, 4096])
def test_one_shot_prompts_cut_into_key_spans(fa, S):
    """Prompts of 1.4K to 4K tokens: pairs of query tiles cut into spans of equal cost."""
    H, G, D = 8, 2, 256
    print(f"fused spans S={S}", flush=True)
    q, k, v, _ = make_case(1, H, G, S, D, S, seed=S)
    outs, o_ws = static_and_workspace(fa, q, k, v, i32([S]), u8([1]), S, 1, scale=0.0625)
    ref = oracle(q, k, v, [S], [1], S, 1, scale=0.0625)
    for n, o in enumerate(outs):
        assert_close(o.float().cpu().numpy(), ref, what=f"S={S} launch {n}")
        assert torch.equal(o, outs[0])
    assert torch.equal(outs[0], o_ws)


def test_static_launches_of_different_shapes_back_to_back(fa):
    """Decode and prefill launches share the array; none may read what another left."""
    H, G, D = 8, 2, 256
    qd, kd, vd, _ = make_case(5, H, G, 1, D, 4000, seed=11)
    qp, kp, vp, _ = make_case(1, H, G, 2048, D, 2048, seed=12)
    qc, kc, vc, _ = make_case(2, H, G, 128, D, 2500, seed=13)
    tds_d, tds_c = [4000, 17, 2000, 4017, 900], [2500, 1300]
    ref_d = oracle(qd, kd, vd, tds_d, [2] * 5, 4000, 2, scale=0.0625)
    ref_p = oracle(qp, kp, vp, [2048], [1], 2048, 1, scale=0.0625)
    ref_c = oracle(qc, kc, vc, tds_c, [1, 1], 2500, 1, scale=0.0625)
    for rnd in range(3):
        od, op, oc = torch.full_like(qd, 777.0), torch.full_like(qp, 777.0), torch.full_like(qc, 777.0)
        fa.flash_attention(qd, kd, vd, od, i32(tds_d), u8([2] * 5), 4000, 2, *partials(8, 5, H, 1, D), scale=0.0625)
        fa.flash_attention(qp, kp, vp, op, i32([2048]), u8([1]), 2048, 1, scale=0.0625)
        fa.flash_attention(qc, kc, vc, oc, i32(tds_c), u8([1, 1]), 2500, 1, scale=0.0625)
        torch.cuda.synchronize()
        assert_close(od.float().cpu().numpy(), ref_d, what=f"decode, round {rnd}")
        assert_close(op.float().cpu().numpy(), ref_p, what=f"prompt, round {rnd}")
        assert_close(oc.float().cpu().numpy(), ref_c, what=f"chunk, round {rnd}")
