"""g4b_attn_forward_static_scratch (split partials in the library's own device array, no allocation) against
g4b_attn_forward with a caller-provided workspace: same kernels and the same partition, so the outputs must agree
(checked an order of magnitude inside the parity tolerance).

Two calls in a row per shape family, the second with a smaller input, so that the second call runs over what the
first left in the scratch array.  pytest collects this file last (its name sorts after every other test file), so a failure here hides no other test.
"""

import ctypes as C

import pytest
import torch

from helpers import i32, ix, make_case, partials, u8

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


def run_both(fa, q, k, v, tds, phase, W, phase_id, parts, **kw):
    """-> (output with an explicit workspace, output through the static scratch), both via the C ABI."""
    B, H, Tq, D = q.shape
    G = k.shape[1]
    need = fa.workspace_bytes(B, H, G, Tq, D)
    assert need > 0, "the shape must be one that splits keys"
    ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    o_ws = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o_ws, tds, phase, W, phase_id, *parts, workspace=ws, **kw)
    o_st = torch.full_like(q, 777.0)
    fa.flash_attention(q, k, v, o_st, tds, phase, W, phase_id, *parts, workspace="static", **kw)
    torch.cuda.synchronize()
    return o_ws, o_st


def assert_same(o_ws, o_st, what):
    d = (o_ws.float() - o_st.float()).abs()
    bound = 1e-3 + 2e-3 * o_ws.float().abs()  # an order of magnitude inside 2e-3 + 1e-2 |ref|
    assert bool((d <= bound).all()), f"{what}: static scratch differs from the workspace path by {float(d.max()):.3e}"


def test_decode_split_two_calls_second_smaller(fa):
    from g4b_amd import _native

    lib = _native.load()
    assert lib.g4b_static_scratch_init() == 0, _native.last_error()
    assert lib.g4b_static_scratch_bytes() == 68 << 20
    for B, D, W, seed in ((24, 256, 6000, 1), (5, 256, 1500, 2), (6, 512, 3000, 3), (2, 512, 700, 4)):
        print(f"static scratch decode B={B} D={D} W={W}", flush=True)
        H, G = 8, 2
        q, k, v, _ = make_case(B, H, G, 1, D, W, seed=seed)
        tds = [W if b % 2 == 0 else max(1, W // (b + 1)) for b in range(B)]
        phase = [ix.PHASE_DECODE if b % 5 != 4 else ix.PHASE_PREFILL for b in range(B)]
        o_ws, o_st = run_both(fa, q, k, v, i32(tds), u8(phase), W, ix.PHASE_DECODE, partials(16, B, H, 1, D), scale=0.0625)
        assert_same(o_ws, o_st, f"B={B} D={D}")
        for b in range(B):
            if phase[b] != ix.PHASE_DECODE:
                assert (o_st[b] == 777.0).all()
            else:
                assert (o_st[b] != 777.0).any()


def test_prefill_chunk_split_two_calls_second_smaller(fa):
    for Tq, D, ctx, seed in ((256, 256, 3000, 5), (96, 256, 700, 6), (128, 512, 1500, 7), (64, 512, 300, 8)):
        print(f"static scratch chunk Tq={Tq} D={D} ctx={ctx}", flush=True)
        B, H, G = 3, 8, 2
        kv_ctx = ctx + Tq + 64
        q, k, v, _ = make_case(B, H, G, Tq, D, kv_ctx, seed=seed)
        tds = [ctx + Tq, 0, Tq]
        phase = [ix.PHASE_PREFILL, ix.PHASE_DECODE, ix.PHASE_PREFILL]
        o_ws, o_st = run_both(fa, q, k, v, i32(tds), u8(phase), kv_ctx, ix.PHASE_PREFILL, (), scale=0.0625)
        assert_same(o_ws, o_st, f"Tq={Tq} D={D}")
        assert (o_st[1] == 777.0).all() and (o_st[0] != 777.0).any()


def test_launches_allocate_nothing_and_can_be_recorded_into_a_graph(fa):
    """Free device memory does not move across static-scratch launches (decode and chunk shapes), and a launch
    recorded into a graph after g4b_static_scratch_init replays to the eager result."""
    from g4b_amd import _native

    assert _native.load().g4b_static_scratch_init() == 0, _native.last_error()
    H, G, D = 8, 2, 256
    qd, kd, vd, od = make_case(6, H, G, 1, D, 3000, seed=21)
    qc, kc, vc, oc = make_case(2, H, G, 192, D, 2500, seed=22)
    tds_d, ph_d = i32([3000, 40, 1500, 3017, 800, 2999]), u8([2] * 6)
    tds_c, ph_c = i32([2500, 1200]), u8([1, 1])
    parts = partials(8, 6, H, 1, D)
    plan_d = fa.plan_flash_attention(qd, kd, vd, od, tds_d, ph_d, 3000, 2, *parts, scale=0.0625, workspace="static")
    plan_c = fa.plan_flash_attention(qc, kc, vc, oc, tds_c, ph_c, 2500, 1, scale=0.0625, workspace="static")
    plan_d.launch(), plan_c.launch()  # warm-up: the first launch of a kernel loads its code
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(50):
        plan_d.launch(), plan_c.launch()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"free device memory moved by {free0 - free1} bytes across 100 static-scratch launches"
    eager_d, eager_c = od.clone(), oc.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan_d.launch(), plan_c.launch()
    for _ in range(3):
        od.fill_(777.0), oc.fill_(777.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(od, eager_d) and torch.equal(oc, eager_c)
        plan_d.launch()  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(od, eager_d)


def test_rejects_what_does_not_fit_and_a_foreign_workspace(fa):
    from g4b_amd import _native

    lib = _native.load()
    B, H, G, D, W = 2, 8, 2, 256, 512
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=9)
    args, keep, entry = fa._bind(q, k, v, o, i32([W, W]), u8([2, 2]), W, 2, *partials(4, B, H, 1, D), workspace="static")
    assert C.cast(entry, C.c_void_p).value == C.cast(lib.g4b_attn_forward_static_scratch, C.c_void_p).value
    # the wrapper runs a launch unsplit when its partials would not fit; the entry point itself refuses it
    _, _, entry_big = fa._bind(q, k, v, o, i32([W, W]), u8([2, 2]), W, 2, *partials(4, B, H, 1, D), num_workers=1 << 20)
    assert C.cast(entry_big, C.c_void_p).value == C.cast(lib.g4b_attn_forward, C.c_void_p).value
    args.num_workers = 1 << 20
    rc = lib.g4b_attn_forward_static_scratch(C.byref(args), None)
    assert rc == _native.G4B_ERR_WORKSPACE, rc
    assert "static scratch holds" in _native.last_error()
    args.num_workers = 0
    args.workspace = q.data_ptr()
    args.workspace_bytes = 1 << 30
    rc = lib.g4b_attn_forward_static_scratch(C.byref(args), None)
    assert rc == _native.G4B_ERR_INVALID_ARGUMENT, rc
    torch.cuda.synchronize()
