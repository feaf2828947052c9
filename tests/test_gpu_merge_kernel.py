"""The merge kernel of split prefill-shaped launches asks for partial rows before it knows which splits wrote any (the
heavier tile of a pair that was cut into key spans), and clamps the rows of its last block to the last token.  What a
split did not write is whatever the workspace held: these tests poison the workspace with bytes that read as NaN in
every type (0xFF) before each launch and compare with the unsplit launch of the same inputs, on shapes that take every
variant of the kernel: spans (2 .. 5 per pair, with and without a per-query window), uniform splits (4, 8, 16), head
dimensions 128 / 256 / 512, token counts that are no multiple of the kernel's 16 rows, fp32 and 16-bit outputs.
"""

import pytest
import torch

from helpers import i32, make_case, u8

pytestmark = pytest.mark.gpu
H, G = 8, 2


@pytest.fixture(scope="module")
def fa(gpu_device):
    from g4b_amd.kernels import fa2

    return fa2


CASES = [
    # B, Tq, context before the chunk, D, query window, in-phase slots
    (1, 1408, 0, 256, None, 1),   # pairs cut into key spans
    (1, 2048, 0, 256, None, 1),
    (1, 2560, 0, 256, None, 1),
    (1, 3000, 0, 256, None, 1),   # last row block of the merge holds 8 tokens
    (1, 4096, 0, 256, None, 1),
    (1, 2048, 0, 256, 512, 1),    # per-query window: neighbouring tiles paired
    (1, 2048, 0, 128, None, 1),
    (1, 1000, 0, 256, None, 1),   # uniform splits per tile, 1000 = 62 * 16 + 8
    (1, 1024, 0, 128, None, 1),
    (1, 250, 4096, 256, None, 1),  # chunk, 16 splits
    (3, 130, 2048, 256, None, 2),  # two in-phase slots of three
    (33, 512, 8192, 256, None, 1),  # one chunk in a batch of 33, 8 splits
    (1, 3072, 0, 512, None, 1),   # head dimension 512: two key spans per tile
    (1, 200, 4096, 512, None, 1),
]


@pytest.mark.parametrize("o_dtype", [torch.float16, torch.float32], ids=["o16", "o32"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_T%d_ctx%d_D%d_w%s_n%d" % c)
def test_split_launch_with_poisoned_workspace_agrees_with_unsplit(fa, case, o_dtype):
    B, Tq, ctx, D, qwin, n_in = case
    print(f"poisoned workspace {case} {o_dtype}", flush=True)
    kv = ctx + Tq
    q, k, v, _ = make_case(B, H, G, Tq, D, kv, seed=Tq + D)
    tds = i32([kv] * B)
    phases = u8([1] * n_in + [2] * (B - n_in))
    nbytes = fa.workspace_bytes(B, H, G, Tq, D)
    assert nbytes > 0, "the shape is meant to split"
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    kw = dict(scale=1 / 16, query_window=qwin)
    ref = torch.full((B, H, Tq, D), 777.0, dtype=o_dtype, device="cuda")
    fa.flash_attention(q, k, v, ref, tds, phases, kv, 1, workspace=False, **kw)
    for attempt in range(2):
        ws.fill_(0xFF)
        o = torch.full((B, H, Tq, D), 777.0, dtype=o_dtype, device="cuda")
        fa.flash_attention(q, k, v, o, tds, phases, kv, 1, workspace=ws, **kw)
        torch.cuda.synchronize()
        assert bool(torch.isfinite(o).all()), f"non-finite output, attempt {attempt}"
        assert bool((o[n_in:] == 777.0).all()), "rows of slots that are not in phase were written"
        d = (o[:n_in].float() - ref[:n_in].float()).abs()
        assert bool((d <= 1e-3 + 4e-3 * ref[:n_in].float().abs()).all()), (attempt, d.max().item())
