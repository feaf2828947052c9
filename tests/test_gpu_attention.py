"""GPU parity of flash_attention (through the C ABI) against the fp64 oracle.

Shapes follow the reference's compare script (tests/compare_scripts/test_fa2.py:51-79), scaled so
the CPU oracle finishes in seconds: 7 decode shapes (window 1024..., head dim 128/256, GQA 4:1 and
8:1), prefill chunks on a long context, one-shot causal prefill, one non-causal; half the slots at
tds = W, half at tds = W + 17 so the ring wraps (:286-290).  Every variant the script compares
(no split buffers / split buffers) is compared here as well, with assertions.
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


DECODE_CASES = [
    # name, B, H, G, D, W
    ("decode_small_w1024", 4, 8, 2, 128, 1024),
    ("decode_gemma_w4096", 8, 16, 4, 256, 4096),
    ("decode_gemma_w8192", 4, 16, 4, 256, 8192),
    ("decode_gemma_w16384", 2, 16, 4, 256, 16384),
    ("decode_biggroup_w4096", 4, 32, 4, 256, 4096),
    ("decode_mha_w512", 3, 4, 4, 128, 512),
    ("decode_group16_w2048", 2, 16, 1, 256, 2048),
    ("decode_d512_w2048", 4, 16, 4, 512, 2048),
    ("decode_d512_group8_w1024", 2, 16, 2, 512, 1024),
    ("decode_d512_group16_w700", 3, 16, 1, 512, 700),
]


@pytest.mark.parametrize("case", DECODE_CASES, ids=[c[0] for c in DECODE_CASES])
@pytest.mark.parametrize("scale", [1.0, 1 / 16])
def test_decode_matches_oracle_split_and_unsplit(fa, case, scale):
    name, B, H, G, D, W = case
    print(f"case {name} scale {scale}", flush=True)
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=1)
    tds = [W if b % 2 == 0 else W + 17 for b in range(B)]
    phase = [ix.PHASE_DECODE] * B
    ref = oracle(q, k, v, tds, phase, W, ix.PHASE_DECODE, scale=scale)
    # no split buffers: one wave per (slot, kv head)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, ix.PHASE_DECODE, scale=scale)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what=f"{name} unsplit")
    # split buffers given: keys dealt to many waves, partials merged
    o2 = torch.full_like(o, 777.0)
    fa.flash_attention(q, k, v, o2, i32(tds), u8(phase), W, ix.PHASE_DECODE, *partials(4, B, H, 1, D), scale=scale)
    torch.cuda.synchronize()
    assert_close(o2.float().cpu().numpy(), ref, what=f"{name} split")
    # split and unsplit agree to an fp16 ulp or two of the output (test_fa2.py:432-433 prints this difference)
    diff = (o2.float() - o.float()).abs()
    assert bool((diff <= 5e-4 + 2e-3 * o.float().abs()).all()), diff.max().item()


@pytest.mark.parametrize("num_workers", [1, 3, 64, 100, 153, 154, 777, 4096])
def test_decode_any_worker_count_gives_the_same_answer(fa, num_workers):
    """306 tiles in all: up to 153 workers the shares are weighted by the parity of the worker's XCD (at least two tiles
    per worker), from 154 on they are equal, from 306 on every worker has one tile."""
    B, H, G, D, W = 5, 8, 2, 256, 2048
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=2)
    tds = [1, 33, 700, 2048, 2048 + 300]
    phase = [2] * B
    ref = oracle(q, k, v, tds, phase, W, 2, scale=0.0625)
    ws = torch.empty(fa.workspace_bytes(B, H, G, 1, D, num_workers), dtype=torch.uint8, device="cuda")
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 2, scale=0.0625, workspace=ws, num_workers=num_workers)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what=f"workers={num_workers}")


@pytest.mark.parametrize("Tq,H,G", [(2, 8, 2), (4, 8, 2), (3, 4, 4), (2, 16, 2), (1, 16, 1)])
def test_small_query_blocks_take_the_streaming_kernel(fa, Tq, H, G):
    """(H/G)*Tq <= 16 rows: causal offsets between the rows of one block, wrap, both stages."""
    B, D, kv_ctx, W = 3, 256, 200, 150
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=3)
    tds = [Tq, 150, 150 + 77]
    phase = [1] * B
    for stage in (ix.STAGE_CAUSAL, ix.STAGE_FULL):
        for parts in ((), partials(4, B, H, Tq, D)):
            o.fill_(777.0)
            ref = oracle(q, k, v, tds, phase, W, 1, stage=stage, scale=0.0625)
            fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 1, *parts, stage=stage, scale=0.0625)
            torch.cuda.synchronize()
            assert_close(o.float().cpu().numpy(), ref, what=f"Tq={Tq} stage={stage} split={bool(parts)}")


@pytest.mark.parametrize("Tq,H,G", [(2, 8, 2), (4, 8, 2), (3, 4, 4), (1, 16, 1)])
@pytest.mark.parametrize("num_workers", [0, 5, 2048])
def test_head_dim_512_query_blocks_and_worker_counts(fa, Tq, H, G, num_workers):
    """Head dimension 512 (the global-attention layers): two waves per worker share the dot product."""
    B, D, kv_ctx, W = 3, 512, 300, 260
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=31)
    tds = [Tq, 260, 260 + 91]
    phase = [1] * B
    ref = oracle(q, k, v, tds, phase, W, 1, scale=0.0442)
    ws = torch.empty(fa.workspace_bytes(B, H, G, Tq, D, num_workers), dtype=torch.uint8, device="cuda")
    o.fill_(777.0)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 1, scale=0.0442, workspace=ws, num_workers=num_workers)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what=f"D=512 Tq={Tq} workers={num_workers}")


PREFILL_CASES = [
    # name, B, H, G, Tq, kv_ctx, D, W, stage
    ("prefill_t128_w4096", 2, 16, 4, 128, 4096, 256, 4096, ix.STAGE_CAUSAL),
    ("prefill_t256_w4096", 1, 16, 4, 256, 4096, 256, 4096, ix.STAGE_CAUSAL),
    ("prefill_t256_w1024_d128", 2, 8, 2, 256, 1024, 128, 1024, ix.STAGE_CAUSAL),
    ("full_t256_w256", 2, 16, 4, 256, 256, 256, 256, ix.STAGE_FULL),
    ("prefill_ragged_t100", 2, 8, 2, 100, 600, 256, 512, ix.STAGE_CAUSAL),
    ("prefill_mha_t70", 1, 2, 2, 70, 300, 128, 300, ix.STAGE_CAUSAL),
    ("prefill_group8_t48", 1, 16, 2, 48, 500, 256, 400, ix.STAGE_CAUSAL),
    # head dimension 512: a pair of waves shares each 32-row block
    ("prefill_d512_t128_w1024", 2, 8, 2, 128, 1024, 512, 1024, ix.STAGE_CAUSAL),
    ("prefill_d512_ragged_t100", 2, 8, 2, 100, 600, 512, 512, ix.STAGE_CAUSAL),
    ("full_d512_t96_w256", 2, 16, 4, 96, 256, 512, 256, ix.STAGE_FULL),
    ("prefill_d512_group8_t48", 1, 16, 2, 48, 500, 512, 400, ix.STAGE_CAUSAL),
    ("prefill_d512_mha_t70", 1, 2, 2, 70, 300, 512, 300, ix.STAGE_CAUSAL),
]
SPLIT_CASES = PREFILL_CASES[:3] + PREFILL_CASES[4:5] + PREFILL_CASES[7:9]


@pytest.mark.parametrize("case", PREFILL_CASES, ids=[c[0] for c in PREFILL_CASES])
@pytest.mark.parametrize("scale", [1.0, 1 / 16])
def test_prefill_matches_oracle(fa, case, scale):
    name, B, H, G, Tq, kv_ctx, D, W, stage = case
    print(f"case {name} scale {scale}", flush=True)
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=4)
    tds = [W if b % 2 == 0 else W + 17 for b in range(B)]
    phase = [1] * B
    ref = oracle(q, k, v, tds, phase, W, 1, stage=stage, scale=scale)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 1, stage=stage, scale=scale)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what=name)


@pytest.mark.parametrize("case", SPLIT_CASES, ids=[c[0] for c in SPLIT_CASES])
def test_prefill_key_split_agrees_with_one_workgroup_per_tile(fa, case):
    """Shapes that bring few workgroups split every item's keys over several and merge the partials; with
    ``workspace=False`` nothing is split.  Both must match the oracle and each other."""
    name, B, H, G, Tq, kv_ctx, D, W, stage = case
    assert fa.workspace_bytes(B, H, G, Tq, D) > 0, "these shapes are meant to take the split path"
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=14)
    tds = [W if b % 2 == 0 else W + 17 for b in range(B)]
    ref = oracle(q, k, v, tds, [1] * B, W, 1, stage=stage, scale=1 / 16)
    fa.flash_attention(q, k, v, o, i32(tds), u8([1] * B), W, 1, stage=stage, scale=1 / 16)
    o1 = torch.full_like(o, 777.0)
    fa.flash_attention(q, k, v, o1, i32(tds), u8([1] * B), W, 1, stage=stage, scale=1 / 16, workspace=False)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what=f"{name} split")
    assert_close(o1.float().cpu().numpy(), ref, what=f"{name} unsplit")
    diff = (o1.float() - o.float()).abs()
    assert bool((diff <= 5e-4 + 2e-3 * o.float().abs()).all()), diff.max().item()


@pytest.mark.parametrize("n_prefill,D", [(1, 256), (2, 256), (5, 256), (9, 256), (1, 512), (3, 512), (9, 512)])
def test_prefill_chunk_inside_a_mixed_batch(fa, n_prefill, D):
    """The engine's mixed step: a few slots prefill a chunk while the others decode or are unallocated.  The number of
    key splits follows the number of in-phase slots, which only the device knows."""
    B, H, G, Tq, W = 9, 8, 2, 96, 3000
    kv_ctx = W + Tq - 1
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=15)
    order = [4, 0, 8, 2, 6, 1, 3, 5, 7]
    phase = [2 if b % 2 else 0 for b in range(B)]
    for b in order[:n_prefill]:
        phase[b] = 1
    tds = [Tq + 37 * b * b * 3 for b in range(B)]  # from a bare chunk to a wrapped ring
    tds[order[0]] = 5000 + Tq
    ref = oracle(q, k, v, tds, phase, W, 1, scale=1 / 16)
    o.fill_(123.0)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 1, scale=1 / 16)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    for b in range(B):
        if phase[b] == 1:
            assert_close(got[b], ref[b], what=f"slot {b} of {n_prefill} prefilling")
        else:
            assert (got[b] == 123.0).all(), f"off-phase slot {b} was written"


@pytest.mark.parametrize("Tq,H,G,D", [(1, 8, 2, 256), (1, 16, 2, 128), (3, 8, 2, 256), (1, 16, 1, 256)])
def test_short_window_one_kernel_path_agrees_with_the_two_kernel_path(fa, Tq, H, G, D):
    """Windows of at most 512 keys (the sliding-window layers) run as one launch that merges a pair's waves through
    LDS; passing the same window per slot through window_sizes takes the worker + merge kernels instead.  Ragged
    lengths from 0 keys to a wrapped ring; both against the oracle and against each other."""
    B, W = 11, 512
    kv_ctx = W + 5
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=51)
    tds = [Tq, Tq + 1, 31 + Tq, 32 + Tq, 33 + Tq, 128, 129, 500, 512, 513, 5000]
    phase = [1 if Tq > 1 else 2] * B
    phase[4] = 0
    ph = phase[0]
    ref = oracle(q, k, v, tds, phase, W, ph, scale=1 / 16)
    o.fill_(321.0)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, ph, *partials(4, B, H, Tq, D), scale=1 / 16)
    o2 = torch.full_like(o, 321.0)
    fa.flash_attention(q, k, v, o2, i32(tds), u8(phase), W, ph, *partials(4, B, H, Tq, D), scale=1 / 16,
                       window_sizes=i32([W] * B))
    torch.cuda.synchronize()
    got, got2 = o.float().cpu().numpy(), o2.float().cpu().numpy()
    for b in range(B):
        if phase[b] == 0:
            assert (got[b] == 321.0).all() and (got2[b] == 321.0).all()
        else:
            assert_close(got[b], ref[b], what=f"one-kernel path slot {b}")
            assert_close(got2[b], ref[b], what=f"two-kernel path slot {b}")
    d = np.abs(got - got2)
    assert (d <= 5e-4 + 2e-3 * np.abs(got2)).all(), d.max()


@pytest.mark.parametrize("D", [256, 512])
def test_more_than_64_slots(fa, D):
    """Batches beyond one wavefront of slots: the device-side work lists walk the slots 64 (decode) or 256 (prefill
    shapes) at a time.  150 slots with ragged lengths; decode over the odd slots, then a 40-token chunk on five slots
    scattered over the batch."""
    B, H, G, W = 150, 8, 2, 96
    rng = np.random.default_rng(41)
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=41)
    tds = rng.integers(0, 2 * W, B).tolist()
    phase = [2 if b % 2 else 0 for b in range(B)]
    ref = oracle(q, k, v, tds, phase, W, 2, scale=1 / 16)
    for parts in ((), partials(4, B, H, 1, D)):
        o.fill_(123.0)
        fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 2, *parts, scale=1 / 16)
        torch.cuda.synchronize()
        got = o.float().cpu().numpy()
        for b in range(B):
            if phase[b] == 2:
                assert_close(got[b], ref[b], what=f"decode slot {b} split={bool(parts)}")
            else:
                assert (got[b] == 123.0).all(), f"off-phase slot {b} was written"
    Tq = 40
    kv_ctx = W + Tq - 1
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=42)
    chunking = [3, 64, 65, 128, 149]
    phase = [1 if b in chunking else 2 for b in range(B)]
    tds = [Tq + int(x) for x in rng.integers(0, 3 * W, B)]
    ref = oracle(q, k, v, tds, phase, W, 1, scale=1 / 16)
    o.fill_(123.0)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, 1, scale=1 / 16)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    for b in range(B):
        if phase[b] == 1:
            assert_close(got[b], ref[b], what=f"chunk on slot {b}")
        else:
            assert (got[b] == 123.0).all(), f"off-phase slot {b} was written"


def test_prefill_workspace_too_small_is_refused(fa):
    B, H, G, Tq, D, W = 1, 8, 2, 128, 256, 1024
    q, k, v, o = make_case(B, H, G, Tq, D, W, seed=16)
    need = fa.workspace_bytes(B, H, G, Tq, D)
    assert need > 0
    small = torch.empty(need - 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError, match="workspace"):
        fa.flash_attention(q, k, v, o, i32([W]), u8([1]), W, 1, workspace=small)
    exact = torch.empty(need, dtype=torch.uint8, device="cuda")
    fa.flash_attention(q, k, v, o, i32([W]), u8([1]), W, 1, scale=1 / 16, workspace=exact)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), oracle(q, k, v, [W], [1], W, 1, scale=1 / 16), what="caller workspace")


def test_bound_plan_relaunches_with_new_device_data(fa):
    """A plan binds pointers, not values: lengths and queries updated in place are seen by the next launch."""
    B, H, G, D, W = 4, 8, 2, 256, 1024
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=17)
    tds = i32([100, 1024, 1024 + 5, 7])
    phase = u8([2, 2, 2, 2])
    ws = torch.empty(fa.workspace_bytes(B, H, G, 1, D), dtype=torch.uint8, device="cuda")
    plan = fa.plan_flash_attention(q, k, v, o, tds, phase, W, 2, scale=1 / 16, workspace=ws)
    plan.launch()
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), oracle(q, k, v, tds.tolist(), [2] * B, W, 2, scale=1 / 16), what="plan, first launch")
    tds += 3
    q.copy_(torch.roll(q, 1, dims=0))
    plan.launch()
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), oracle(q, k, v, tds.tolist(), [2] * B, W, 2, scale=1 / 16), what="plan, second launch")


def test_one_shot_causal_prefill_2048(fa):
    """Benchmark configuration 2: batch 1, seq 2048, 8 q heads / 2 kv heads, head dim 256, scale 1/16."""
    B, H, G, Tq, D = 1, 8, 2, 2048, 256
    q, k, v, o = make_case(B, H, G, Tq, D, Tq, seed=0)
    ref = oracle(q, k, v, [Tq], [1], Tq, 1, scale=1 / 16)
    fa.flash_attention(q, k, v, o, i32([Tq]), u8([1]), Tq, 1, scale=1 / 16)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what="config 2")


@pytest.mark.parametrize("qw,D", [(1, 256), (37, 256), (64, 256), (512, 256), (5000, 256), (1, 512), (37, 512), (500, 512)])
def test_per_query_sliding_window(fa, qw, D):
    """One-shot prefill longer than the window: key visible iff 0 <= q_pos - k_pos < query_window."""
    B, H, G, Tq = 1, 8, 2, 1024
    q, k, v, o = make_case(B, H, G, Tq, D, Tq, seed=5)
    ref = oracle(q, k, v, [Tq], [1], Tq, 1, scale=1 / 16, query_window=qw)
    fa.flash_attention(q, k, v, o, i32([Tq]), u8([1]), Tq, 1, scale=1 / 16, query_window=qw)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what=f"query_window={qw}")


@pytest.mark.parametrize("D", [256, 512])
def test_chunk_on_long_context_with_wrap(fa, D):
    """A 512-token chunk appended to an existing context in a ring of W + t - 1 rows (gemma4e.py:703-705)."""
    B, H, G, t, W = 2, 8, 2, 512, 2048
    kv_ctx = W + t - 1
    q, k, v, o = make_case(B, H, G, t, D, kv_ctx, seed=6)
    tds = [1500 + t, 9000 + t]  # second slot: window full, ring wrapped several times
    ref = oracle(q, k, v, tds, [1, 1], W, 1, scale=1 / 16)
    fa.flash_attention(q, k, v, o, i32(tds), u8([1, 1]), W, 1, scale=1 / 16)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, what="chunk on context")


def test_phase_skip_leaves_rows_untouched_and_empty_slots_are_zero(fa):
    B, H, G, D, W = 6, 8, 2, 256, 256
    for Tq in (1, 64):
        q, k, v, o = make_case(B, H, G, Tq, D, W, seed=7)
        phase = [1, 2, 0, 1, 2, 1]
        tds = [max(Tq, 100), 100, 100, 0, 0, 256 + 40]
        for launch_phase in (1, 2):
            o.fill_(777.0)
            parts = partials(4, B, H, Tq, D) if Tq == 1 else ()
            fa.flash_attention(q, k, v, o, i32(tds), u8(phase), W, launch_phase, *parts, scale=0.0625)
            torch.cuda.synchronize()
            got = o.float().cpu().numpy()
            ref = oracle(q, k, v, tds, phase, W, launch_phase, scale=0.0625)
            for b in range(B):
                if phase[b] != launch_phase:
                    assert (got[b] == 777.0).all(), f"slot {b} of an off-phase launch was written"
                elif tds[b] == 0:
                    assert (got[b] == 0).all(), "in-phase slot without keys must be zeros"
                else:
                    assert_close(got[b], ref[b], what=f"Tq={Tq} slot {b}")


@pytest.mark.parametrize("Tq", [1, 96])
def test_engine_layout_fp32_strided_views(fa, Tq):
    """q and o as the engine passes them: fp32, permuted views of [B, t, H, D] scratchpads (gemma4e.py:1031-1033)."""
    B, H, G, D, W = 3, 8, 2, 256, 700
    q, k, v, o = make_case(B, H, G, Tq, D, W, seed=8, q_dtype=torch.float32, engine_layout=True)
    assert not q.is_contiguous() or Tq == 1
    tds = [W, W + 17, max(Tq, 5)]
    phase_id = 2 if Tq == 1 else 1
    # the MFMA path rounds q to fp16 first; compare against the oracle on the rounded values
    ref = oracle(q.half(), k, v, tds, [phase_id] * B, W, phase_id, scale=0.0625)
    parts = partials(16, B, H, Tq, D) if Tq == 1 else ()
    fa.flash_attention(q, k, v, o, i32(tds), u8([phase_id] * B), W, phase_id, *parts, scale=0.0625, use_fp32_dot=True)
    torch.cuda.synchronize()
    assert o.dtype == torch.float32
    assert_close(o.cpu().numpy(), ref, what="engine layout")


@pytest.mark.parametrize("Tq,D", [(1, 256), (96, 256), (1, 512), (96, 512)])
def test_fp16_output_straight_into_the_token_major_activation_buffer(fa, Tq, D):
    """fp32 q scratchpad in, fp16 o out, o being the [B, t, H*D] buffer the next matmul reads: no cast or layout pass
    between the kernels (the reference keeps both sides fp32 and casts afterwards, gemma4e.py:1031-1033)."""
    B, H, G, W = 3, 8, 2, 700
    q, k, v, _ = make_case(B, H, G, Tq, D, W, seed=18, q_dtype=torch.float32, engine_layout=True)
    act = torch.full((B, Tq, H * D), 777.0, dtype=torch.float16, device="cuda")
    o = act.view(B, Tq, H, D).permute(0, 2, 1, 3)
    tds = [W, W + 17, max(Tq, 5)]
    phase_id = 2 if Tq == 1 else 1
    ref = oracle(q.half(), k, v, tds, [phase_id] * B, W, phase_id, scale=0.0625)
    fa.flash_attention(q, k, v, o, i32(tds), u8([phase_id] * B), W, phase_id, scale=0.0625)
    torch.cuda.synchronize()
    got = act.view(B, Tq, H, D).permute(0, 2, 1, 3).float().cpu().numpy()
    assert_close(got, ref, what="fp16 o in [B,t,H*D]")


@pytest.mark.parametrize("D", [256, 512])
@pytest.mark.parametrize("Tq", [1, 160])
def test_bf16_cache(fa, Tq, D):
    B, H, G, W = 2, 8, 2, 1024
    q, k, v, o = make_case(B, H, G, Tq, D, W, seed=9, dtype=torch.bfloat16)
    tds = [W, W + 17]
    phase_id = 2 if Tq == 1 else 1
    ref = oracle(q, k, v, tds, [phase_id] * B, W, phase_id, scale=0.0625)
    parts = partials(4, B, H, Tq, D) if Tq == 1 else ()
    fa.flash_attention(q, k, v, o, i32(tds), u8([phase_id] * B), W, phase_id, *parts, scale=0.0625)
    torch.cuda.synchronize()
    assert_close(o.float().cpu().numpy(), ref, atol=ATOL_BF16, rtol=RTOL_BF16, what="bf16")


@pytest.mark.parametrize("D", [256, 512])
@pytest.mark.parametrize("Tq", [1, 4, 40])
def test_visible_set_is_bit_exact(fa, Tq, D):
    """K = 0 makes the weights uniform; V row r = e_(r mod D) turns the output into the indicator of the
    ring rows that were read divided by their count, so the visible set is read back exactly."""
    B, H, G = 4, 8, 2
    kv_ctx, W = 251, 200  # W <= KV_CTX <= D so that every ring row has its own output column
    q = torch.randn(B, H, Tq, D, device="cuda").half()
    k = torch.zeros(B, G, kv_ctx, D, device="cuda", dtype=torch.float16)
    v = torch.zeros(B, G, kv_ctx, D, device="cuda", dtype=torch.float16)
    v[:, :, torch.arange(kv_ctx), torch.arange(kv_ctx)] = 1.0
    tds = [Tq, 57 + Tq, 200, 200 + 123]
    phase_id = 2 if Tq == 1 else 1
    for qw in (None, 7):
        o = torch.zeros(B, H, Tq, D, device="cuda", dtype=torch.float32)
        parts = partials(4, B, H, Tq, D) if Tq * 4 <= 16 else ()
        fa.flash_attention(q, k, v, o, i32(tds), u8([phase_id] * B), W, phase_id, *parts, query_window=qw)
        torch.cuda.synchronize()
        got = o.cpu().numpy()
        for b in range(B):
            for i in range(Tq):
                lo, hi = ix.visible_range(i, tds[b], W, Tq, ix.STAGE_CAUSAL, qw)
                rows = sorted(ix.ring_row(tds[b], W, kv_ctx, j) for j in range(lo, hi))
                for h in range(H):
                    read = np.nonzero(got[b, h, i])[0].tolist()
                    assert read == rows, (Tq, qw, b, h, i)
                    np.testing.assert_allclose(got[b, h, i, rows], 1.0 / len(rows), rtol=2e-3)


def test_dispatch_stamped_kernel_times(fa):
    """g4b_profile_begin / g4b_profile_end: one duration per call for its dominant kernel, -1 when that kernel is
    masked out, results unchanged, misuse reported."""
    import ctypes

    from g4b_amd import _native

    lib = _native.load()
    B, H, G, D, W = 4, 8, 2, 256, 2048
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=61)
    tds, ph = i32([W, 100, 1500, W + 9]), u8([2] * B)
    ws = torch.empty(fa.workspace_bytes(B, H, G, 1, D), dtype=torch.uint8, device="cuda")
    fa.flash_attention(q, k, v, o, tds, ph, W, 2, scale=1 / 16, workspace=ws)
    torch.cuda.synchronize()
    expect = o.clone()
    assert lib.g4b_profile_end(None, 0) == _native.G4B_ERR_INVALID_ARGUMENT
    assert lib.g4b_profile_begin() == 0
    assert lib.g4b_profile_begin() == _native.G4B_ERR_INVALID_ARGUMENT
    o.zero_()
    for mask in (0, 0, 2, 1):
        fa.flash_attention(q, k, v, o, tds, ph, W, 2, scale=1 / 16, workspace=ws, kernel_mask=mask)
    buf = (ctypes.c_float * 8)()
    assert lib.g4b_profile_end(buf, 8) == 4
    ts = list(buf[:4])
    assert ts[2] == -1.0 and all(0 < t < 5.0 for t in (ts[0], ts[1], ts[3])), ts
    torch.cuda.synchronize()
    assert torch.equal(o, expect)
    # a prefill-shaped call is timed the same way
    q2, k2, v2, o2 = make_case(1, H, G, 256, D, 512, seed=62)
    assert lib.g4b_profile_begin() == 0
    fa.flash_attention(q2, k2, v2, o2, i32([512]), u8([1]), 512, 1, scale=1 / 16)
    assert lib.g4b_profile_end(buf, 8) == 1 and 0 < buf[0] < 5.0


def test_argument_errors_follow_the_reference(fa):
    B, H, G, D, W = 2, 8, 2, 256, 64
    q, k, v, o = make_case(B, H, G, 1, D, W, seed=10)
    tds, ph = i32([10, 20]), u8([2, 2])
    po, pl, pm = partials(4, B, H, 1, D)
    with pytest.raises(ValueError):  # fa2.py:656-657
        fa.flash_attention(q, k, v, o, tds, ph, W, 2, po, None, pm)
    with pytest.raises(AssertionError):  # fa2.py:653
        fa.flash_attention(q, k, v, o, tds, ph, W, 2.0)
    with pytest.raises(ValueError):  # fa2.py:298 ctx_window_size <= KV_CTX
        fa.flash_attention(q, k, v, o, tds, ph, W + 1, 2)
    with pytest.raises(ValueError):  # fa2.py:293
        fa.flash_attention(q, k, v, o[:, :4], tds, ph, W, 2)
    with pytest.raises(ValueError, match="on_band_block"):  # the stage alone depends on the reference's tile size
        fa.flash_attention(q, k, v, o, tds, ph, W, 2, stage=fa.STAGE_ON_BAND)


@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("Tq", [1000, 400])
@pytest.mark.parametrize("case", ["from_scratch", "on_context", "two_active", "per_query_window", "full_stage", "bf16"])
def test_prefill_pairs_of_query_tiles_cut_into_key_spans(fa, D, case, Tq):
    """A slot that brings between a third of the chip's compute units and all of them in query tiles: the tiles are
    paired and the key tiles of every pair (heavy tile, then light tile) are cut into two to five spans of equal cost,
    one workgroup each; a tile that lies wholly in one span is written straight to o, the others are merged.  H/G = 16
    makes a query tile 8 tokens, so 1000 tokens are 125 tiles = 63 pairs per kv head (two spans each) and 400 tokens 50
    tiles = 25 pairs (five spans each)."""
    print(f"pair split {case} D={D} Tq={Tq}", flush=True)
    H, G, kv_ctx = 32, 2, 1300
    B = 3 if case == "two_active" else 2
    dtype = torch.bfloat16 if case == "bf16" else torch.float16
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=len(case) + D, dtype=dtype)
    tds = {"from_scratch": [Tq, 5], "on_context": [kv_ctx + 300, 5], "two_active": [Tq, 1250, Tq + 7]}.get(case, [Tq + 130, 5])
    phase = [1, 1, 0] if case == "two_active" else [1, 2]
    kw = {}
    if case == "per_query_window":
        kw["query_window"] = 200
    if case == "full_stage":
        kw["stage"] = ix.STAGE_FULL
    assert fa.workspace_bytes(B, H, G, Tq, D) > 0
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), kv_ctx, 1, scale=D**-0.5, **kw)
    torch.cuda.synchronize()
    ref = oracle(q, k, v, tds, phase, kv_ctx, 1, scale=D**-0.5, **kw)
    got = o.float().cpu().numpy()
    tol = dict(atol=ATOL_BF16, rtol=RTOL_BF16) if case == "bf16" else {}
    for b in range(B):
        if phase[b] == 1:
            assert_close(got[b], ref[b], what=f"slot {b}", **tol)
        else:
            assert (got[b] == torch.tensor(777.0, dtype=dtype).float().item()).all()  # 776 in bf16
    # the same launch without key splits
    o2 = torch.full_like(o, 777.0)
    fa.flash_attention(q, k, v, o2, i32(tds), u8(phase), kv_ctx, 1, scale=D**-0.5, workspace=False, **kw)
    torch.cuda.synchronize()
    assert (o.float() - o2.float()).abs().max().item() <= (6e-2 if case == "bf16" else 4e-3)


def test_prefill_3000_token_prompt_at_the_benchmark_head_shape(fa):
    """H=8, G=2, D=256 and 3000 tokens from an empty cache: 94 query tiles per kv head, 47 pairs, each cut into two spans
    (the range of prompt lengths, 2K to 4K tokens here, where neither the tile-by-tile split nor the pairs alone fill the
    chip).  Every output element against the fp64 oracle."""
    B, H, G, Tq, D = 1, 8, 2, 3000, 256
    q, k, v, o = make_case(B, H, G, Tq, D, Tq, seed=77)
    fa.flash_attention(q, k, v, o, i32([Tq]), u8([1]), Tq, 1, scale=1 / 16)
    torch.cuda.synchronize()
    ref = oracle(q, k, v, [Tq], [1], Tq, 1, scale=1 / 16)
    assert_close(o.float().cpu().numpy(), ref)


@pytest.mark.parametrize("case", ["from_scratch", "on_context", "two_active", "per_query_window", "bf16"])
def test_head_dim_512_query_tiles_cut_into_two_key_spans(fa, case):
    """Head dim 512 gives every workgroup one query tile; a slot whose tiles take more than half of the compute units
    but not all of them (H/G = 16: 1500 tokens are 188 tiles of 8 tokens) has the keys of every tile cut into two
    spans, so that the launch does not last as long as its heaviest tile with half of the chip idle.  With two slots in
    phase the same launch runs unsplit."""
    print(f"two key spans, D=512, {case}", flush=True)
    H, G, Tq, D, kv_ctx = 16, 1, 1500, 512, 1800
    B = 3 if case == "two_active" else 2
    dtype = torch.bfloat16 if case == "bf16" else torch.float16
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=len(case), dtype=dtype)
    tds = {"from_scratch": [Tq, 5], "on_context": [kv_ctx + 300, 5], "two_active": [Tq, 1750, Tq + 7]}.get(case, [Tq + 130, 5])
    phase = [1, 1, 0] if case == "two_active" else [1, 2]
    kw = {"query_window": 300} if case == "per_query_window" else {}
    assert fa.workspace_bytes(B, H, G, Tq, D) == 2 * H * Tq * (D * 2 + 8)
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), kv_ctx, 1, scale=D**-0.5, **kw)
    torch.cuda.synchronize()
    ref = oracle(q, k, v, tds, phase, kv_ctx, 1, scale=D**-0.5, **kw)
    got = o.float().cpu().numpy()
    tol = dict(atol=ATOL_BF16, rtol=RTOL_BF16) if case == "bf16" else {}
    for b in range(B):
        if phase[b] == 1:
            assert_close(got[b], ref[b], what=f"slot {b}", **tol)
        else:
            assert (got[b] == torch.tensor(777.0, dtype=dtype).float().item()).all()  # 776 in bf16


@pytest.mark.parametrize("n_active", [5, 8, 9])
def test_batch_of_prefill_chunks_one_query_tile_per_workgroup(fa, n_active):
    """Several slots with a 512-token chunk each (what the scheduler's prefill step looks like): too many for key splits,
    and up to eight of them are no more query tiles (8 x 2 kv heads x 16) than the chip has compute units, so every
    workgroup takes one tile; nine are paired again."""
    print(f"batch of chunks, {n_active} in phase", flush=True)
    B, H, G, Tq, D, kv_ctx = 10, 8, 2, 512, 256, 900
    q, k, v, o = make_case(B, H, G, Tq, D, kv_ctx, seed=n_active)
    phase = [1 if b < n_active else 2 for b in range(B)]
    tds = [Tq + 37 * b for b in range(B)]
    ws = torch.empty(fa.workspace_bytes(B, H, G, Tq, D), dtype=torch.uint8, device="cuda")
    fa.flash_attention(q, k, v, o, i32(tds), u8(phase), kv_ctx, 1, scale=1 / 16, workspace=ws)
    torch.cuda.synchronize()
    ref = oracle(q, k, v, tds, phase, kv_ctx, 1, scale=1 / 16)
    got = o.float().cpu().numpy()
    for b in range(B):
        if phase[b] == 1:
            assert_close(got[b], ref[b], what=f"slot {b}")
        else:
            assert (got[b] == 777.0).all()
