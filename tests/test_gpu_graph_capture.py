"""The calls of one attention layer recorded into a HIP graph and replayed, as the engine runs its steps
(g4b/lifecycle.py:29-53): rope + append, attention, decode-state advance.  The wrappers allocate nothing when the
workspace is passed in, read no device memory on the host and launch static grids whose work split is computed on the
device from time_dim_sizes, so one recording serves every later step.  Every replay is compared bit for bit with the
same step run eagerly on a second copy of the state, with eager work and synchronisations between the replays.
"""

import pytest
import torch

from helpers import i32, u8

pytestmark = pytest.mark.gpu

H, G, EPS, SCALE = 8, 2, 1e-6, 1 / 16


class LayerState:
    """Static tensors of one layer for B slots and t new tokens per step."""

    def __init__(self, B, t, D, W, T, tds, phase, seed):
        from g4b_amd.kernels import fa2

        g = torch.Generator(device="cuda").manual_seed(seed)
        self.B, self.t, self.D, self.W = B, t, D, W
        self.q = torch.zeros(B, t, H, D, device="cuda")
        self.k = torch.zeros(B, t, G, D, device="cuda")
        self.v = torch.zeros(B, t, G, D, device="cuda")
        self.o = torch.zeros(B, t, H, D, device="cuda")
        self.q_rs, self.k_rs, self.v_rs = (torch.ones(B, t, n, device="cuda") for n in (H, G, G))
        self.kc = torch.randn(B, G, T, D, generator=g, device="cuda").half()
        self.vc = torch.randn(B, G, T, D, generator=g, device="cuda").half()
        self.freqs = torch.rand(D // 2, generator=g, device="cuda") * 0.1
        self.qw = 1 + 0.1 * torch.randn(D, generator=g, device="cuda")
        self.kw = 1 + 0.1 * torch.randn(D, generator=g, device="cuda")
        self.tds = i32(tds)
        self.offsets = i32([x - t for x in tds])
        self.phase = u8(phase)
        self.inp = torch.zeros(1, B, dtype=torch.int32, device="cuda")
        self.out_tok = torch.arange(B, dtype=torch.int32, device="cuda").view(B, 1).contiguous()
        self.ws = torch.empty(max(fa2.workspace_bytes(B, H, G, t, D), 16), dtype=torch.uint8, device="cuda")

    def clone(self):
        other = object.__new__(LayerState)
        for name, val in vars(self).items():
            setattr(other, name, val.clone() if torch.is_tensor(val) else val)
        return other

    def feed(self, q, k, v):
        """New activations of a step (eager copies into the static scratchpads)."""
        self.q.copy_(q), self.k.copy_(k), self.v.copy_(v)
        for rs, x in ((self.q_rs, self.q), (self.k_rs, self.k), (self.v_rs, self.v)):
            rs.copy_((x * x).sum(-1))

    def layer(self, phase_id):
        from g4b_amd.kernels.advance_decode_state import advance_decode_state
        from g4b_amd.kernels.fa2 import PHASE_DECODE, flash_attention
        from g4b_amd.kernels.rope import apply_rope_and_append

        def hv(x):  # [B, t, heads, D] scratchpad as [B, heads, t, D]
            return x.permute(0, 2, 1, 3)

        def rv(x):
            return x.permute(0, 2, 1)

        apply_rope_and_append(hv(self.q), hv(self.k), hv(self.v), self.freqs, self.offsets, rv(self.q_rs), rv(self.k_rs),
                              rv(self.v_rs), self.qw, self.kw, EPS, self.kc, self.vc, self.phase, phase_id)
        flash_attention(hv(self.q), self.kc, self.vc, hv(self.o), self.tds, self.phase, self.W, phase_id, scale=SCALE,
                        workspace=self.ws)
        if phase_id == PHASE_DECODE:
            advance_decode_state(self.inp, self.out_tok, self.offsets, self.tds, self.phase)

    def same_as(self, other):
        for name in ("q", "o", "kc", "vc", "tds", "offsets", "inp"):
            a, b = getattr(self, name), getattr(other, name)
            assert torch.equal(a, b), f"{name} differs after a replay"


@pytest.mark.parametrize("D", [256, 512])
def test_decode_layer_graph_replays_follow_the_device_state(gpu_device, D):
    """Six slots (four decoding at very different lengths, one on the ring seam, one off phase); the recorded step is
    replayed five times while time_dim_sizes and cache_offsets advance on the device."""
    B, W = 6, 1024
    tds = [1, 300, 1024, 1021, 777, 50]  # slot 3 crosses the ring seam during the replays
    phase = [2, 2, 2, 2, 0, 2]
    eager = LayerState(B, 1, D, W, W, tds, phase, seed=21)
    gen = torch.Generator(device="cuda").manual_seed(22)
    new = lambda: [torch.randn(B, 1, n, D, generator=gen, device="cuda") for n in (H, G, G)]  # noqa: E731
    eager.feed(*new())
    eager.layer(2)  # first step eagerly: first-call set-up happens here, not in the recording
    torch.cuda.synchronize()
    replayed = eager.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        replayed.layer(2)
    for step in range(5):
        acts = new()
        eager.feed(*acts), replayed.feed(*acts)
        eager.layer(2)
        graph.replay()
        torch.cuda.synchronize()
        replayed.same_as(eager)
    assert replayed.tds.tolist() == [t + 6 if p == 2 else t for t, p in zip(tds, phase)]


def test_prefill_chunk_graph_replays_with_host_updated_offsets(gpu_device):
    """A 96-token chunk per replay on one slot of three; the host moves cache_offsets / time_dim_sizes between the
    replays with eager copies into the static tensors, as the scheduler does for prefill steps."""
    B, t, D, W = 3, 96, 256, 1024
    T = W + t - 1
    phase = [2, 1, 0]
    eager = LayerState(B, t, D, W, T, [400, t, 9], phase, seed=23)
    gen = torch.Generator(device="cuda").manual_seed(24)
    new = lambda: [torch.randn(B, t, n, D, generator=gen, device="cuda") for n in (H, G, G)]  # noqa: E731
    eager.feed(*new())
    eager.layer(1)
    torch.cuda.synchronize()
    replayed = eager.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        replayed.layer(1)
    for chunk in range(1, 14):  # 13 more chunks: the window fills and the ring wraps
        acts = new()
        for st in (eager, replayed):
            st.feed(*acts)
            st.offsets.copy_(i32([399, chunk * t, 0]))
            st.tds.copy_(i32([400, (chunk + 1) * t, 9]))
        eager.layer(1)
        graph.replay()
        torch.cuda.synchronize()
        replayed.same_as(eager)
