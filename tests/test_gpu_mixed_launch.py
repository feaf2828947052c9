"""A step that holds prefill-phase and decode-phase slots, served by ONE launch (flash_attention(..., decode_q=,
decode_o=)) instead of the reference's two calls over the same batch tensors (its kernel skips per slot on
user_phase[b] != PHASE, g4b/kernels/fa2.py:332-335; its scheduler avoids such steps, g4b/scheduler.py:66,96-98).

Both halves are compared with the fp64 oracle, slot by slot; slots of neither phase must stay untouched.  Both layer
kinds of the mixed benchmark configuration run: a global layer (window = context) whose decode half streams through
split-KV workers, and a sliding-window layer (window 512 on a ring of 512 + t - 1 rows) whose decode half takes the
one-workgroup-per-pair path.
"""

import numpy as np
import pytest
import torch

from helpers import ATOL_BF16, RTOL_BF16, assert_close, i32, ix, oracle, u8

pytestmark = pytest.mark.gpu

H, G, D = 8, 2, 256


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


def make_batch(B, t, kv_ctx, seed, dtype=torch.float16, q_dtype=None, D=D):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    q_dtype = q_dtype or dtype
    qp = torch.randn(B, H, t, D, generator=gen).to(q_dtype).cuda()
    qd = torch.randn(B, H, 1, D, generator=gen).to(q_dtype).cuda()
    k = torch.randn(B, G, kv_ctx, D, generator=gen).to(dtype).cuda()
    v = torch.randn(B, G, kv_ctx, D, generator=gen).to(dtype).cuda()
    return qp, qd, k, v


def check_both_halves(fa, qp, qd, k, v, tds, phase, W, scale, ws, tol=None, **kw):
    B = qp.shape[0]
    op = torch.full_like(qp, 777.0)
    od = torch.full_like(qd, 777.0)
    fa.flash_attention(qp, k, v, op, i32(tds), u8(phase), W, ix.PHASE_PREFILL, scale=scale, workspace=ws,
                       decode_q=qd, decode_o=od, **kw)
    torch.cuda.synchronize()
    okw = {k_: v_ for k_, v_ in kw.items() if k_ in ("stage", "query_window")}
    ref_p = oracle(qp, k, v, tds, phase, W, ix.PHASE_PREFILL, scale=scale, **okw)
    ref_d = oracle(qd, k, v, tds, phase, W, ix.PHASE_DECODE, scale=scale, **okw)
    gp, gd = op.float().cpu().numpy(), od.float().cpu().numpy()
    tol = tol or {}
    for b in range(B):
        if phase[b] == ix.PHASE_PREFILL:
            assert_close(gp[b], ref_p[b], what=f"chunk of slot {b}", **tol)
            assert (gd[b] == 777.0).all(), f"decode output of prefill slot {b} was written"
        elif phase[b] == ix.PHASE_DECODE:
            if tds[b] == 0:
                assert (gd[b] == 0).all()
            else:
                assert_close(gd[b], ref_d[b], what=f"decode slot {b}", **tol)
            assert (gp[b] == 777.0).all(), f"chunk output of decode slot {b} was written"
        else:
            assert (gp[b] == 777.0).all() and (gd[b] == 777.0).all(), f"unallocated slot {b} was written"
    return op, od


@pytest.mark.parametrize("layer", ["global", "sliding_window"])
@pytest.mark.parametrize("with_workspace", [True, False], ids=["split", "unsplit"])
@pytest.mark.parametrize("D", [256, 512])
def test_mixed_step_matches_the_oracle(fa, layer, with_workspace, D):
    print(f"mixed {layer} workspace={with_workspace} D={D}", flush=True)
    B, t = 9, 128
    if layer == "global":
        W = kv_ctx = 3000 + t - 1
    else:
        W, kv_ctx = 512, 512 + t - 1
    qp, qd, k, v = make_batch(B, t, kv_ctx, seed=31, D=D)
    # slots 0-5 decode (lengths 1 .. beyond the ring, one empty), 6 a chunk on a long context, 7 unallocated, 8 a
    # chunk at the start of its sequence
    tds = [1, 77, 2900, 1500, 0, 2999 if layer == "global" else kv_ctx + 40, 2000 + t, 9, t]
    phase = [2, 2, 2, 2, 2, 2, 1, 0, 1]
    ws = None
    if with_workspace:
        n = fa.mixed_workspace_bytes(B, H, G, t, 1, D, kv_ctx, W)
        assert n > 0
        ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    check_both_halves(fa, qp, qd, k, v, tds, phase, W, 1 / 16, ws)


def test_mixed_step_equals_the_two_separate_launches_closely(fa):
    """Same inputs through the two reference-style calls and through the one launch: both are within the tolerance of
    the oracle; against each other they differ by the rounding of differently split partial sums only."""
    B, t, kv_ctx = 5, 256, 4096
    W = kv_ctx
    qp, qd, k, v = make_batch(B, t, kv_ctx, seed=32)
    tds, phase = [4000, 1200, 1000 + t, 300, t + 5], [2, 2, 1, 2, 1]
    ws = torch.empty(fa.mixed_workspace_bytes(B, H, G, t, 1, D, kv_ctx, W), dtype=torch.uint8, device="cuda")
    op, od = check_both_halves(fa, qp, qd, k, v, tds, phase, W, 1.0, ws)
    op2, od2 = torch.full_like(op, 777.0), torch.full_like(od, 777.0)
    fa.flash_attention(qp, k, v, op2, i32(tds), u8(phase), W, ix.PHASE_PREFILL)
    fa.flash_attention(qd, k, v, od2, i32(tds), u8(phase), W, ix.PHASE_DECODE,
                       *[torch.empty(4, B, H, 1, D, dtype=torch.float16, device="cuda"),
                         torch.empty(4, B, H, 1, device="cuda"), torch.empty(4, B, H, 1, device="cuda")])
    torch.cuda.synchronize()
    assert (op.float() - op2.float()).abs().max().item() <= 4e-3
    assert (od.float() - od2.float()).abs().max().item() <= 4e-3


@pytest.mark.parametrize("D", [256, 512])
def test_mixed_step_fp32_queries_and_per_slot_windows(fa, D):
    """Engine-style fp32 q with use_fp32_dot on a bf16 cache (split-query kernels), and per-slot window sizes (which
    force the streaming workers even for short windows)."""
    B, t, kv_ctx = 4, 96, 1500
    qp, qd, k, v = make_batch(B, t, kv_ctx, seed=33, dtype=torch.bfloat16, q_dtype=torch.float32, D=D)
    tds, phase = [1400, 700 + t, 90, 1500], [2, 1, 2, 2]
    win = [512, kv_ctx, kv_ctx, 64]
    n = fa.mixed_workspace_bytes(B, H, G, t, 1, D, kv_ctx, kv_ctx, True)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    op = torch.full_like(qp, 777.0)
    od = torch.full_like(qd, 777.0)
    fa.flash_attention(qp, k, v, op, i32(tds), u8(phase), kv_ctx, ix.PHASE_PREFILL, scale=1 / 16, workspace=ws, use_fp32_dot=True,
                       window_sizes=i32(win), decode_q=qd, decode_o=od)
    torch.cuda.synchronize()
    ref_p = oracle(qp, k, v, tds, phase, kv_ctx, 1, scale=1 / 16, window_sizes=win)
    ref_d = oracle(qd, k, v, tds, phase, kv_ctx, 2, scale=1 / 16, window_sizes=win)
    for b in range(B):
        got, ref = (op, ref_p) if phase[b] == 1 else (od, ref_d)
        assert_close(got[b].cpu().numpy(), ref[b], atol=ATOL_BF16, rtol=RTOL_BF16, what=f"slot {b}")


def test_mixed_step_argument_errors(fa):
    B, t, kv_ctx = 2, 64, 256
    qp, qd, k, v = make_batch(B, t, kv_ctx, seed=34)
    op, od = torch.empty_like(qp), torch.empty_like(qd)
    tds, ph = i32([100, 100 + t]), u8([2, 1])
    with pytest.raises(ValueError, match="go together"):
        fa.flash_attention(qp, k, v, op, tds, ph, kv_ctx, 1, decode_q=qd)
    with pytest.raises(ValueError, match="different phases"):
        fa.flash_attention(qp, k, v, op, tds, ph, kv_ctx, 2, decode_q=qd, decode_o=od)
    with pytest.raises(ValueError, match="prefill-shaped"):
        fa.flash_attention(qd, k, v, od, tds, ph, kv_ctx, 1, decode_q=qd, decode_o=od)
    small = torch.empty(64, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError, match="workspace"):
        fa.flash_attention(qp, k, v, op, tds, ph, kv_ctx, 1, decode_q=qd, decode_o=od, workspace=small)
    torch.cuda.synchronize()


def test_mixed_step_recorded_into_a_graph(fa):
    """The mixed launch is legal under stream capture (static grid, device-side work split, no allocation): five
    replays against eager runs while the decode lengths advance on the device."""
    from g4b_amd.kernels.advance_decode_state import advance_decode_state

    B, t, kv_ctx = 6, 64, 2048
    W = kv_ctx
    qp, qd, k, v = make_batch(B, t, kv_ctx, seed=35)
    tds0, phase = [5, 900, 1999, 300 + t, 40, 1200], [2, 2, 2, 1, 0, 2]
    ws = torch.empty(fa.mixed_workspace_bytes(B, H, G, t, 1, D, kv_ctx, W), dtype=torch.uint8, device="cuda")

    class State:
        def __init__(self):
            self.tds, self.offs, self.ph = i32(tds0), i32([x - 1 for x in tds0]), u8(phase)
            self.op, self.od = torch.full_like(qp, 777.0), torch.full_like(qd, 777.0)
            self.inp = torch.zeros(1, B, dtype=torch.int32, device="cuda")
            self.tok = torch.arange(B, dtype=torch.int32, device="cuda").view(B, 1).contiguous()
            self.ws = torch.empty_like(ws)

        def step(self):
            fa.flash_attention(qp, k, v, self.op, self.tds, self.ph, W, ix.PHASE_PREFILL, scale=1 / 16, workspace=self.ws,
                               decode_q=qd, decode_o=self.od)
            advance_decode_state(self.inp, self.tok, self.offs, self.tds, self.ph)

    eager, replayed = State(), State()
    eager.step(), replayed.step()  # first call eagerly: the kernels' shared-memory attribute is set here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        replayed.step()
    eager.step()
    for _ in range(5):
        graph.replay()
        eager.step()
        torch.cuda.synchronize()
    # the recording itself does not execute: the replayed state is one step behind
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(eager.tds, replayed.tds) and torch.equal(eager.od, replayed.od) and torch.equal(eager.op, replayed.op)


def test_plan_takes_the_arguments_by_keyword(fa):
    """plan_flash_attention binds like flash_attention: every argument may come by keyword, also for a mixed launch."""
    B, t, kv_ctx = 3, 64, 700
    qp, qd, k, v = make_batch(B, t, kv_ctx, seed=36)
    tds, phase = [600, 300 + t, 50], [2, 1, 2]
    ws = torch.empty(fa.mixed_workspace_bytes(B, H, G, t, 1, D, kv_ctx, kv_ctx), dtype=torch.uint8, device="cuda")
    op, od = torch.full_like(qp, 777.0), torch.full_like(qd, 777.0)
    plan = fa.plan_flash_attention(q=qp, k_cache=k, v_cache=v, o=op, time_dim_sizes=i32(tds), user_phase=u8(phase),
                                   ctx_window_size=kv_ctx, phase=ix.PHASE_PREFILL, scale=1 / 16, workspace=ws, decode_q=qd,
                                   decode_o=od, stream=None)
    plan.launch()
    torch.cuda.synchronize()
    ref_p = oracle(qp, k, v, tds, phase, kv_ctx, 1, scale=1 / 16)
    ref_d = oracle(qd, k, v, tds, phase, kv_ctx, 2, scale=1 / 16)
    assert_close(op[1].float().cpu().numpy(), ref_p[1])
    for b in (0, 2):
        assert_close(od[b].float().cpu().numpy(), ref_d[b])
