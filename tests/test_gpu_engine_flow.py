"""The caller contract of Gemma4E._attention (g4b/models/gemma4e.py:557-607) replayed on the GPU.

Per step and layer kind: K append, V append (with the fused weightless RMSNorm), flash_attention on
strided fp32 views of [B, t, H, D] scratchpads, and after a decode step advance_decode_state.  The
integers come from the scheduler's rules (g4b/scheduler.py:133-212): a prefilling slot gets
(offset, offset + t) with t the padded chunk width, a decoding slot (ctx, ctx + 1), an inactive
slot (0, 0).  The expectation is computed from the per-slot token streams by absolute position.
"""

import numpy as np
import pytest
import torch

from helpers import assert_close, ix

pytestmark = pytest.mark.gpu


def expected_from_stream(q_b, ks, vs, n_ctx, Tq, W, scale):
    """Attention of the last Tq positions of a stream of n_ctx tokens over its last W positions (fp64)."""
    H, _, D = q_b.shape
    G = ks.shape[0]
    lo = max(n_ctx - W, 0)
    k = np.repeat(ks[:, lo:n_ctx].astype(np.float64), H // G, axis=0)
    v = np.repeat(vs[:, lo:n_ctx].astype(np.float64), H // G, axis=0)
    s = np.einsum("htd,hnd->htn", q_b.astype(np.float64), k) * scale
    q_pos = np.arange(n_ctx - Tq, n_ctx)[:, None]
    k_pos = np.arange(lo, n_ctx)[None, :]
    s = np.where(q_pos < k_pos, -np.inf, s)
    p = np.exp(s - s.max(-1, keepdims=True))
    return np.einsum("htn,hnd->htd", p / p.sum(-1, keepdims=True), v)


@pytest.mark.parametrize("W,context_len", [(64, 4096), (4096, 4096)], ids=["swa", "global"])
def test_prefill_chunks_then_decode(gpu_device, W, context_len):
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache
    from g4b_amd.kernels.advance_decode_state import advance_decode_state
    from g4b_amd.kernels.fa2 import PHASE_DECODE, PHASE_PREFILL, flash_attention

    dev = gpu_device
    B, H, G, D, t = 4, 8, 2, 256, 32
    Wc = min(W, context_len)
    T = Wc + t - 1  # gemma4e.py:703-705
    eps, scale = 1e-6, 1.0 / 16
    rng = np.random.default_rng(0)
    prompt_len = [70, 32, 0, 45]  # slot 2 stays empty
    q_pad = torch.zeros(B, t, H, D, device=dev)  # fp32 scratchpads (DTA = float32)
    k_pad = torch.zeros(B, t, G, D, device=dev)
    v_pad = torch.zeros(B, t, G, D, device=dev)
    o_pad = torch.full((B, t, H, D), 777.0, device=dev)
    rs_pad = torch.zeros(B, t, G, device=dev)
    k_cache = torch.randn(B, G, T, D, device=dev).half()
    v_cache = torch.randn(B, G, T, D, device=dev).half()
    offsets = torch.zeros(B, dtype=torch.int32, device=dev)
    tds = torch.zeros(B, dtype=torch.int32, device=dev)
    phase = torch.zeros(B, dtype=torch.uint8, device=dev)
    streams_k = [np.zeros((G, 0, D), np.float16) for _ in range(B)]
    streams_v = [np.zeros((G, 0, D), np.float16) for _ in range(B)]
    ctx = [0] * B

    def view(x, t_now):  # _attn_view: [B, t_now, h, D] -> [B, h, t_now, D]
        return x[:, :t_now].permute(0, 2, 1, 3)

    def layer(t_now, phase_id, parts=()):
        k_in, v_in = view(k_pad, t_now), view(v_pad, t_now)
        rs = rs_pad[:, :t_now].permute(0, 2, 1)
        add_kv_to_cache(k_in, k_cache, offsets, eps, user_phase=phase, phase=phase_id)
        add_kv_to_cache(v_in, v_cache, offsets, eps, rs, user_phase=phase, phase=phase_id)
        flash_attention(view(q_pad, t_now), k_cache, v_cache, view(o_pad, t_now), tds, phase, Wc, phase_id, *parts,
                        use_grouped_query_tile=True, use_fp32_dot=True, scale=scale)

    def fill_inputs(b, n_tok, t_now):
        """New q/k/v rows for slot b; rows beyond n_tok are padding (repeat of the last token's values)."""
        q = rng.standard_normal((t_now, H, D)).astype(np.float32)
        k = rng.standard_normal((t_now, G, D)).astype(np.float32)
        v = rng.standard_normal((t_now, G, D)).astype(np.float32)
        q_pad[b, :t_now] = torch.from_numpy(q).to(dev)
        k_pad[b, :t_now] = torch.from_numpy(k).to(dev)
        v_pad[b, :t_now] = torch.from_numpy(v).to(dev)
        rs = (v * v).sum(-1)
        rs_pad[b, :t_now] = torch.from_numpy(rs).to(dev)
        vn = v * (1.0 / np.sqrt(rs / D + eps))[..., None]
        return q, k.astype(np.float16), vn.astype(np.float16)

    # ---- prefill: chunks of t tokens, the last one padded (scheduler.py:150-172) ----
    pos = [0] * B
    while any(pos[b] < prompt_len[b] for b in range(B)):
        step_q, active = {}, []
        offs, lens, ph = [], [], []
        for b in range(B):
            if pos[b] >= prompt_len[b]:
                # A slot that sits out a step is marked unallocated here (fa2.py:26-28) so that nothing of it is
                # touched.  (The engine marks every slot with the step's phase and zero offset / length,
                # gemma4e.py:224-248, which lets the append overwrite ring row 0.. of an idle slot; its scheduler
                # only idles slots whose cache is dead.)
                offs.append(0), lens.append(0), ph.append(0)
                continue
            real = min(t, prompt_len[b] - pos[b])
            q, k16, v16 = fill_inputs(b, real, t)
            o, n = ix.prefill_step_integers(ctx[b], t)
            offs.append(o), lens.append(n), ph.append(PHASE_PREFILL)
            # all t rows are written; only the first `real` become part of the stream
            step_q[b] = (q, real, k16, v16)
            active.append(b)
        offsets.copy_(torch.tensor(offs, dtype=torch.int32)), tds.copy_(torch.tensor(lens, dtype=torch.int32))
        phase.copy_(torch.tensor(ph, dtype=torch.uint8))
        o_pad.fill_(777.0)
        layer(t, PHASE_PREFILL)
        torch.cuda.synchronize()
        got = o_pad.permute(0, 2, 1, 3).cpu().numpy()
        for b in active:
            q, real, k16, v16 = step_q[b]
            # the kernel sees a stream in which the padded rows exist: ctx + t tokens
            ks = np.concatenate([streams_k[b], k16.transpose(1, 0, 2)], 1)
            vs = np.concatenate([streams_v[b], v16.transpose(1, 0, 2)], 1)
            exp = expected_from_stream(q.transpose(1, 0, 2).astype(np.float16), ks, vs, ctx[b] + t, t, Wc, scale)
            assert_close(got[b][:, :real], exp[:, :real], what=f"prefill slot {b} at ctx {ctx[b]}")
            streams_k[b] = ks[:, : ctx[b] + real]
            streams_v[b] = vs[:, : ctx[b] + real]
            ctx[b] += real
            pos[b] += real
        for b in range(B):
            if b not in active:
                assert (got[b] == 777.0).all()

    # ---- decode: 5 steps; the device advances its own offsets / lengths ----
    decoding = [b for b in range(B) if prompt_len[b] > 0]
    phase.copy_(torch.tensor([PHASE_DECODE if b in decoding else 0 for b in range(B)], dtype=torch.uint8))
    offs = [ix.decode_step_integers(ctx[b])[0] if b in decoding else 0 for b in range(B)]
    lens = [ix.decode_step_integers(ctx[b])[1] if b in decoding else 0 for b in range(B)]
    offsets.copy_(torch.tensor(offs, dtype=torch.int32)), tds.copy_(torch.tensor(lens, dtype=torch.int32))
    inp = torch.zeros(t, B, dtype=torch.int32, device=dev)
    out_tok = torch.zeros(B, 1, dtype=torch.int32, device=dev)
    S = 16
    parts = (
        torch.empty(S, B, H, t, D, dtype=torch.float16, device=dev)[:, :, :, :1],  # slice_until(3, 1) of the big buffer
        torch.empty(S, B, H, t, dtype=torch.float32, device=dev)[:, :, :, :1],
        torch.empty(S, B, H, t, dtype=torch.float32, device=dev)[:, :, :, :1],
    )
    for step in range(5):
        step_q = {}
        for b in decoding:
            step_q[b] = fill_inputs(b, 1, 1)
        out_tok.copy_(torch.arange(B, dtype=torch.int32).reshape(B, 1) + 100 * step)
        o_pad.fill_(777.0)
        layer(1, PHASE_DECODE, parts)
        advance_decode_state(inp, out_tok, offsets, tds, phase)
        torch.cuda.synchronize()
        got = o_pad[:, :1].permute(0, 2, 1, 3).cpu().numpy()
        for b in range(B):
            if b not in decoding:
                assert (got[b] == 777.0).all()
                continue
            q, k16, v16 = step_q[b]
            streams_k[b] = np.concatenate([streams_k[b], k16.transpose(1, 0, 2)], 1)
            streams_v[b] = np.concatenate([streams_v[b], v16.transpose(1, 0, 2)], 1)
            ctx[b] += 1
            exp = expected_from_stream(q.transpose(1, 0, 2).astype(np.float16), streams_k[b], streams_v[b], ctx[b], 1, Wc, scale)
            assert_close(got[b], exp, what=f"decode step {step} slot {b}")
        assert tds.tolist() == [ctx[b] + 1 if b in decoding else 0 for b in range(B)]
        assert offsets.tolist() == [ctx[b] if b in decoding else 0 for b in range(B)]
        assert inp[0].tolist() == [b + 100 * step if b in decoding else 0 for b in range(B)]


def test_rope_append_attention_by_absolute_position(gpu_device):
    """gemma4e.py:564-607 with the rope, both appends and the attention of a layer: a stream fed as two prefill chunks
    and three decode steps must give, at every new position, what the whole stream gives when it is normalised and
    rotated by absolute position on the CPU and attended in one piece."""
    from g4b_amd.kernels.advance_decode_state import advance_decode_state
    from g4b_amd.kernels.fa2 import PHASE_DECODE, PHASE_PREFILL, flash_attention
    from g4b_amd.kernels.rope import apply_rope_and_append
    from oracle import rope_ref as rr

    dev = gpu_device
    B, H, G, D, t = 2, 8, 2, 256, 48  # slot 1 is never allocated
    W = 4096
    T = W + t - 1
    eps, scale = 1e-6, 1.0
    rng = np.random.default_rng(7)
    n_total = 2 * t + 3
    q_all = rng.standard_normal((H, n_total, D)).astype(np.float32)
    k_all = rng.standard_normal((G, n_total, D)).astype(np.float32)
    v_all = rng.standard_normal((G, n_total, D)).astype(np.float32)
    freqs = rr.populate_rope_frequencies_ref(D // 2, 1e6).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    # whole stream on the CPU: positions 0 .. n_total - 1
    q_rot, k_rot = rr.apply_rope_ref(q_all[None], k_all[None], freqs, np.array([0]), (q_all * q_all).sum(-1)[None],
                                     (k_all * k_all).sum(-1)[None], qw, kw, eps)
    v_n = v_all / np.sqrt((v_all * v_all).mean(-1, keepdims=True) + eps)
    k16, v16 = k_rot[0].astype(np.float16), v_n.astype(np.float16)

    q_pad = torch.zeros(B, t, H, D, device=dev)
    k_pad = torch.zeros(B, t, G, D, device=dev)
    v_pad = torch.zeros(B, t, G, D, device=dev)
    o_pad = torch.zeros(B, t, H, D, device=dev)
    q_rs, k_rs, v_rs = (torch.ones(B, t, n, device=dev) for n in (H, G, G))
    k_cache = torch.zeros(B, G, T, D, device=dev, dtype=torch.float16)
    v_cache = torch.zeros(B, G, T, D, device=dev, dtype=torch.float16)
    freqs_d, qw_d, kw_d = (torch.from_numpy(x).to(dev) for x in (freqs, qw, kw))
    offsets = torch.zeros(B, dtype=torch.int32, device=dev)
    tds = torch.zeros(B, dtype=torch.int32, device=dev)
    phase = torch.zeros(B, dtype=torch.uint8, device=dev)

    def view(x, n):
        return x[:, :n].permute(0, 2, 1, 3)

    def step(lo, n, phase_id):
        q_pad[0, :n] = torch.from_numpy(q_all[:, lo : lo + n].transpose(1, 0, 2)).to(dev)
        k_pad[0, :n] = torch.from_numpy(k_all[:, lo : lo + n].transpose(1, 0, 2)).to(dev)
        v_pad[0, :n] = torch.from_numpy(v_all[:, lo : lo + n].transpose(1, 0, 2)).to(dev)
        for rs, x in ((q_rs, q_pad), (k_rs, k_pad), (v_rs, v_pad)):
            rs[:, :n] = (x[:, :n] ** 2).sum(-1)
        apply_rope_and_append(view(q_pad, n), view(k_pad, n), view(v_pad, n), freqs_d, offsets, q_rs[:, :n].permute(0, 2, 1),
                              k_rs[:, :n].permute(0, 2, 1), v_rs[:, :n].permute(0, 2, 1), qw_d, kw_d, eps, k_cache, v_cache,
                              phase, phase_id)
        flash_attention(view(q_pad, n), k_cache, v_cache, view(o_pad, n), tds, phase, W, phase_id, scale=scale)
        torch.cuda.synchronize()
        got = o_pad[0, :n].permute(1, 0, 2).cpu().numpy()
        # the kernel feeds the MFMA with q rounded to the cache's 16-bit type
        exp = expected_from_stream(q_rot[0][:, lo : lo + n].astype(np.float16), k16, v16, lo + n, n, W, scale)
        assert_close(got, exp, what=f"positions {lo}..{lo + n - 1}")

    phase.copy_(torch.tensor([PHASE_PREFILL, 0], dtype=torch.uint8))
    for c in range(2):
        o, n = ix.prefill_step_integers(c * t, t)
        offsets.copy_(torch.tensor([o, 0], dtype=torch.int32)), tds.copy_(torch.tensor([n, 0], dtype=torch.int32))
        step(c * t, t, PHASE_PREFILL)
    phase.copy_(torch.tensor([PHASE_DECODE, 0], dtype=torch.uint8))
    o, n = ix.decode_step_integers(2 * t)
    offsets.copy_(torch.tensor([o, 0], dtype=torch.int32)), tds.copy_(torch.tensor([n, 0], dtype=torch.int32))
    inp = torch.zeros(1, B, dtype=torch.int32, device=dev)
    out_tok = torch.zeros(B, 1, dtype=torch.int32, device=dev)
    for s in range(3):
        step(2 * t + s, 1, PHASE_DECODE)
        advance_decode_state(inp, out_tok, offsets, tds, phase)
    torch.cuda.synchronize()
    assert offsets.tolist() == [2 * t + 3, 0] and tds.tolist() == [2 * t + 4, 0]
