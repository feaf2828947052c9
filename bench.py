#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra] [--no-cpu-baseline]

A "step" is one pass of the hot path over one batch of synthetic input: one ``flash_attention``
call (all of its kernels) on inputs that already sit in HBM, issued through a bound plan (the arguments are
validated once, every step is the bare C-ABI call -- what a graph replay costs the engine).  The default workload is the batched
decode configuration of the metric (64 sequences, KV lengths U{128..32768}, half of them with a
512-token sliding window); ``value`` is its algorithmic KV bytes per second.  The other synthetic
configurations (single-sequence decode, causal prefill 2048 / 8192, sliding-window prefill 8192, the
mixed chunked-prefill step) are timed as well and reported under ``extra`` unless ``--no-extra``.

One JSON line is printed at the end.  ``roofline`` describes the dominant kernel of the primary
workload: algorithmic bytes (or flops) per launch divided by that kernel's average duration,
measured here with HIP events on the launch stream: the library dispatches the kernel with a start and a
stop event of its own (``g4b_profile_begin`` / ``g4b_profile_end``), so the figure is the kernel's duration
as a kernel trace reports it; the duration of an event pair recorded around the call, which also spans the
launch gaps, is logged beside it.  ``cpu_baseline`` is the CPU restatement of the
reference attention timed on the host cores on a bounded sample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "decode attn GB/s (% HBM peak); prefill attn TFLOP/s (% fp16 MFMA peak)"
HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E
FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA

# HBM bytes per launch of the dominant kernel come from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of these
# same seeded workloads (KiB per dispatch), each scaled by what the same counter reads for a 1 GiB copy kernel in the
# same run.  Counters cannot be read from inside the timed run, so `--traffic-from DIR` turns the counter CSVs of
# such runs into profiles/traffic.json and every later run reads the figures from there; a workload without a
# counter run reports null.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
SETTLE_MS = 30.0  # untimed launches of the same workload before anything is timed: the clocks settle under load
DOMINANT_KERNEL = ("attn_decode_worker", "attn_decode_pair", "attn_decode_single", "attn_prefill_kernel",
                   "attn_prefill_wide_kernel", "attn_mixed", "rope_kernel")


def measured_traffic_bytes(name: str):
    try:
        with open(TRAFFIC_JSON) as f:
            t = json.load(f).get(name)
    except (OSError, ValueError):
        return None
    return None if t is None else int(t["bytes"])


def traffic_from_counters(prof_dir: str) -> dict:
    """Read DIR/pmc_FETCH_SIZE_<workload>/**/*counter_collection.csv and DIR/pmc_WRITE_SIZE_<workload>/... (runs of
    `bench.py --workload <workload> --no-extra --no-cpu-baseline --copy-calibration` under rocprofv3 --pmc) and
    merge per-launch HBM bytes of each workload's dominant kernel into profiles/traffic.json."""
    import collections
    import csv
    import glob

    try:
        with open(TRAFFIC_JSON) as f:
            table = json.load(f)
    except (OSError, ValueError):
        table = {}
    found = collections.defaultdict(dict)
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        for d in sorted(glob.glob(os.path.join(prof_dir, f"pmc_{counter}_*"))):
            wl_key = os.path.basename(d)[len(f"pmc_{counter}_"):]
            per_kernel = collections.defaultdict(list)
            for path in glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True):
                with open(path) as f:
                    for r in csv.DictReader(f):
                        if r["Counter_Name"] == counter:
                            per_kernel[r["Kernel_Name"]].append(float(r["Counter_Value"]))
            copies = [v for k, vs in per_kernel.items() if "copyBuffer" in k for v in vs if v > 1e5]
            if not copies:
                continue
            # the calibration copy reads 1 GiB and writes 1 GiB: 1 048 576 KiB of each
            scale = 1048576.0 / (sum(copies) / len(copies))
            dom = [(k, vs) for k, vs in per_kernel.items() if any(n in k for n in DOMINANT_KERNEL)]
            if not dom:
                continue
            k, vs = max(dom, key=lambda kv: sum(kv[1]))
            found[wl_key][counter] = {"kernel": k.split("(")[0], "kib": sum(vs) / len(vs), "scale": scale, "dispatches": len(vs)}
    for wl_key, c in found.items():
        if "FETCH_SIZE" not in c or "WRITE_SIZE" not in c:
            continue
        name = wl_key
        fe, wr = c["FETCH_SIZE"], c["WRITE_SIZE"]
        table[name] = {
            "kernel": fe["kernel"], "fetch_kib": round(fe["kib"], 1), "fetch_scale": round(fe["scale"], 4),
            "write_kib": round(wr["kib"], 1), "write_scale": round(wr["scale"], 4),
            "bytes": int(round((fe["kib"] * fe["scale"] + wr["kib"] * wr["scale"]) * 1024)),
            "source": f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, bench.py --workload {wl_key} --copy-calibration",
        }
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")
    return table
H, G, D = 8, 2, 256
SCALE = 1.0 / 16.0

# Where split partials go: "caller" = a workspace tensor sized with workspace_bytes() next to the engine's own partial
# buffers (what the integration notes recommend), "static" = the library's own scratch array (what the wrappers take
# when no workspace is passed: same kernels, a few microseconds slower per split launch on this board).
WORKSPACE_MODE = "caller"


def WORKSPACE_OF(ws):
    return "static" if WORKSPACE_MODE == "static" or ws is None else ws



def host_cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# --------------------------------------------------------------------------- workloads
class Workload:
    """Device tensors plus the closures that launch the hot path on them."""

    name = ""
    key = ""  # the --workload name; profiles/traffic.json is keyed by it
    bound = "hbm"

    def launch(self, i: int = 0, kernel_mask: int = 0):
        raise NotImplementedError

    def cpu_sample(self):
        """-> (seconds, units_done, description) for the CPU baseline on a bounded sample."""
        raise NotImplementedError


def _randn_f16(shape, seed, device, dtype=None):
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randn(shape, generator=g, device=device, dtype=dtype or torch.float16)


class BatchedDecode(Workload):
    """64 sequences x 1 query token against per-sequence ring caches; lengths U{lo..hi}; even slots SWA-512."""

    bound = "hbm"

    def __init__(self, device, B=64, kv_ctx=32768, len_lo=128, len_hi=32768, swa_every=2, seed=0, name="decode_batched_b64",
                 heads=H, groups=G, dim=D, layer_window=None):
        import numpy as np
        import torch

        from g4b_amd.kernels import fa2

        self.name = name
        self.fa2 = fa2
        self.B, self.kv_ctx = B, kv_ctx
        H_, G_, D_ = heads, groups, dim
        self.G_, self.D_ = G_, D_
        rng = np.random.default_rng(seed)
        self.tds_list = rng.integers(len_lo, len_hi + 1, B).tolist()
        self.win_list = [512 if (swa_every and b % swa_every == 0) else kv_ctx for b in range(B)]
        # layer_window: a sliding-window layer of the engine -- one window for every slot (ctx_window_size), no per-slot
        # windows, rings of kv_ctx rows
        self.layer_window = layer_window
        if layer_window:
            self.win_list = [layer_window] * B
        self.n_keys = [min(t, w) for t, w in zip(self.tds_list, self.win_list)]
        self.q = _randn_f16((B, H_, 1, D_), seed + 1, device)
        self.k = _randn_f16((B, G_, kv_ctx, D_), seed + 2, device)
        self.v = _randn_f16((B, G_, kv_ctx, D_), seed + 3, device)
        self.o = torch.empty_like(self.q)
        self.tds = torch.tensor(self.tds_list, dtype=torch.int32, device=device)
        self.win = torch.tensor(self.win_list, dtype=torch.int32, device=device)
        self.phase = torch.full((B,), fa2.PHASE_DECODE, dtype=torch.uint8, device=device)
        self.ws = torch.empty(fa2.workspace_bytes(B, H_, G_, 1, D_), dtype=torch.uint8, device=device)
        self.plans = {}  # bound calls (arguments validated once), one per kernel_mask
        # algorithmic bytes: every visible K and V row once per kv head (2 * G * D * 2 bytes per key)
        self.bytes = 2 * G_ * D_ * 2 * sum(self.n_keys)
        self.flops = 4 * H_ * D_ * sum(self.n_keys)
        self.units = self.bytes

    def launch(self, i=0, kernel_mask=0):
        plan = self.plans.get(kernel_mask)
        if plan is None:
            plan = self.plans[kernel_mask] = self.fa2.plan_flash_attention(
                self.q, self.k, self.v, self.o, self.tds, self.phase, self.layer_window or self.kv_ctx, self.fa2.PHASE_DECODE,
                scale=SCALE, window_sizes=None if self.layer_window else self.win, workspace=WORKSPACE_OF(self.ws),
                kernel_mask=kernel_mask,
            )
        plan.launch()

    def cpu_sample(self):
        from oracle import attention_ref as ar

        if self.layer_window:
            raise NotImplementedError
        # the whole batch, as many passes as fit in about ten seconds of CPU time (the first pass warms the thread pool)
        q, k, v = self.q.cpu(), self.k.cpu(), self.v.cpu()
        phase = [2] * self.B
        ar.attention_cpu_baseline(q[:2], k[:2], v[:2], self.tds_list[:2], phase[:2], self.kv_ctx, 2, scale=SCALE,
                                  window_sizes=self.win_list[:2])
        passes, t0 = 0, time.perf_counter()
        while True:
            ar.attention_cpu_baseline(q, k, v, self.tds_list, phase, self.kv_ctx, 2, scale=SCALE, window_sizes=self.win_list)
            passes += 1
            dt = time.perf_counter() - t0
            if dt >= 10.0 or passes >= 64:
                break
        done = passes * self.bytes
        return dt, done, f"all {self.B} slots ({self.bytes / 1e6:.1f} MB of KV per pass), {passes} passes"


class SingleDecode(Workload):
    """Config 1: one sequence, KV length 2048.  64 distinct caches are rotated so that the 4 MiB do not sit in cache."""

    bound = "hbm"

    def __init__(self, device, n=2048, copies=64, seed=0):
        import torch

        from g4b_amd.kernels import fa2

        self.name = "decode_single_kv2048"
        self.fa2 = fa2
        self.n, self.copies = n, copies
        self.q = _randn_f16((copies, H, 1, D), seed + 1, device)
        self.k = _randn_f16((copies, G, n, D), seed + 2, device)
        self.v = _randn_f16((copies, G, n, D), seed + 3, device)
        self.o = torch.empty_like(self.q)
        self.tds = torch.full((1,), n, dtype=torch.int32, device=device)
        self.phase = torch.full((1,), fa2.PHASE_DECODE, dtype=torch.uint8, device=device)
        self.ws = torch.empty(fa2.workspace_bytes(1, H, G, 1, D), dtype=torch.uint8, device=device)
        # one bound call per cache copy and kernel mask, made here so that no timed step pays for the binding
        self.plans = {
            (c, km): fa2.plan_flash_attention(
                self.q[c : c + 1], self.k[c : c + 1], self.v[c : c + 1], self.o[c : c + 1], self.tds, self.phase,
                n, fa2.PHASE_DECODE, scale=SCALE, workspace=WORKSPACE_OF(self.ws), kernel_mask=km,
            )
            for c in range(copies) for km in (0, 1)
        }
        self.bytes = 2 * G * n * D * 2
        self.flops = 4 * H * n * D
        self.units = self.bytes

    def launch(self, i=0, kernel_mask=0):
        self.plans[(i % self.copies, kernel_mask)].launch()

    def graph_replay_ms(self, replays=20):
        """The same launches recorded once into a graph (all cache copies, in order) and replayed, which is how the
        engine runs its decode step (g4b/lifecycle.py:29-53): wall time per launch without the host's share."""
        import torch

        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for c in range(self.copies):
                self.plans[(c, 0)].launch()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / (replays * self.copies)

    def cpu_sample(self):
        from oracle import attention_ref as ar

        q, k, v = self.q[:1].cpu(), self.k[:1].cpu(), self.v[:1].cpu()
        reps, t0 = 0, time.perf_counter()
        while True:  # about ten seconds of CPU time
            for _ in range(20):
                ar.attention_cpu_baseline(q, k, v, [self.n], [2], self.n, 2, scale=SCALE)
            reps += 20
            dt = time.perf_counter() - t0
            if dt >= 10.0:
                break
        return dt, reps * self.bytes, f"{reps} passes over one cache"


class Prefill(Workload):
    """One-shot prefill: batch 1, Tq = S tokens, causal; ``query_window`` turns it into the per-query sliding window."""

    bound = "mfma"

    def __init__(self, device, S, query_window=None, seed=0, dim=D, bf16=False, engine_call=False):
        import torch

        from g4b_amd.kernels import fa2

        self.fa2 = fa2
        self.S, self.qw = S, query_window
        self.name = f"prefill_causal_{S}" if query_window is None else f"prefill_swa{query_window}_{S}"
        D_ = self.D_ = dim
        if dim != D:
            self.name += f"_d{dim}"
        dt = torch.bfloat16 if bf16 else torch.float16
        if bf16:
            self.name += "_bf16"
        self.engine_call = engine_call
        if engine_call:
            # what the engine passes (gemma4e.py:593-607): fp32 q and o as [B, H, t, D] views of [B, t, H, D] scratchpads,
            # use_fp32_dot=True, so q enters K Q^T as a pair of 16-bit operands
            self.name += "_fp32q"
            self.q = _randn_f16((1, S, H, D_), seed + 1, device, torch.float32).permute(0, 2, 1, 3)
            self.o = torch.empty((1, S, H, D_), dtype=torch.float32, device=device).permute(0, 2, 1, 3)
        else:
            self.q = _randn_f16((1, H, S, D_), seed + 1, device, dt)
            self.o = torch.empty_like(self.q)
        self.k = _randn_f16((1, G, S, D_), seed + 2, device, dt)
        self.v = _randn_f16((1, G, S, D_), seed + 3, device, dt)
        self.tds = torch.full((1,), S, dtype=torch.int32, device=device)
        self.phase = torch.full((1,), fa2.PHASE_PREFILL, dtype=torch.uint8, device=device)
        if query_window is None:
            pairs = S * (S + 1) // 2
        else:
            w = query_window
            pairs = w * (w + 1) // 2 + (S - w) * w
        self.pairs = pairs
        self.plan = None
        need = fa2.workspace_bytes(1, H, G, S, D_)
        self.ws = torch.empty(need, dtype=torch.uint8, device=device) if need and WORKSPACE_MODE == "caller" else None
        self.flops = 4 * H * D_ * pairs
        self.bytes = 2 * H * S * D_ * (4 if engine_call else 2) + 2 * G * S * D_ * 2
        self.units = self.flops

    def launch(self, i=0, kernel_mask=0):
        if self.plan is None:
            self.plan = self.fa2.plan_flash_attention(
                self.q, self.k, self.v, self.o, self.tds, self.phase, self.S, self.fa2.PHASE_PREFILL,
                scale=SCALE, query_window=self.qw, workspace=WORKSPACE_OF(self.ws), use_fp32_dot=self.engine_call,
            )
        self.plan.launch()

    def cpu_sample(self, seconds: float = 10.0):
        from oracle import attention_ref as ar

        # the last `rows` query rows only (they are the most expensive ones): bounded work, stated in the report
        rows = min(self.S, 1024)
        q = self.q[:, :, self.S - rows :].cpu()
        k, v = self.k.cpu(), self.v.cpu()
        ar.retrieve_ref_torch(q[:, :, :8], k, v, scale=SCALE, query_window=self.qw)  # warms the thread pool
        passes, t0 = 0, time.perf_counter()
        while True:
            ar.retrieve_ref_torch(q, k, v, scale=SCALE, query_window=self.qw)
            passes += 1
            dt = time.perf_counter() - t0
            if dt >= seconds or passes >= 64:
                break
        if self.qw is None:
            pairs = sum(self.S - rows + i + 1 for i in range(rows))
        else:
            pairs = sum(min(self.qw, self.S - rows + i + 1) for i in range(rows))
        # the dense CPU formulation computes every (row, key) score, masked or not
        return dt, passes * 4 * H * self.D_ * pairs, f"last {rows} query rows against all {self.S} keys (dense scores), {passes} passes"


class MixedStep(Workload):
    """Config 5: 32 decode slots (lengths U{1024..16384}) + one 512-token chunk on a 16384-token context,
    35 layers alternating sliding-window-512 and global attention.  ``one_launch``: every layer is one mixed launch
    (``decode_q=`` / ``decode_o=``: the chunk and the decode stream share a grid); otherwise one prefill-phase and one
    decode-phase launch per layer over the same batch tensors, as the reference would issue them.  The same cache
    pair is reused by all layers of a kind."""

    bound = "hbm"

    def __init__(self, device, seed=0, layers=35, one_launch=True, global_dim=D):
        import numpy as np
        import torch

        from g4b_amd.kernels import fa2

        self.name = "mixed_step_35_layers" if one_launch else "mixed_step_35_layers_two_launches"
        if global_dim != D:
            self.name += f"_global_d{global_dim}"  # Gemma-4's global-attention layers use head dimension 512
        Dg = self.Dg = global_dim
        self.fa2 = fa2
        self.layers = layers
        self.one_launch = one_launch
        B, t, ctx = 33, 512, 16384
        self.B, self.t = B, t
        rng = np.random.default_rng(seed)
        dec_len = rng.integers(1024, 16384 + 1, 32).tolist()
        self.tds_list = dec_len + [ctx + t]
        self.T_global, self.T_swa, self.W_swa = 32768 + t - 1, 512 + t - 1, 512
        self.W_global = 32768
        self.qp = _randn_f16((B, H, t, D), seed + 1, device)
        self.qd = _randn_f16((B, H, 1, D), seed + 2, device)
        self.op, self.od = torch.empty_like(self.qp), torch.empty_like(self.qd)
        if Dg != D:  # the global layers' own scratchpads
            self.qpg, self.qdg = _randn_f16((B, H, t, Dg), seed + 7, device), _randn_f16((B, H, 1, Dg), seed + 8, device)
            self.opg, self.odg = torch.empty_like(self.qpg), torch.empty_like(self.qdg)
        else:
            self.qpg, self.qdg, self.opg, self.odg = self.qp, self.qd, self.op, self.od
        self.kg = _randn_f16((B, G, self.T_global, Dg), seed + 3, device)
        self.vg = _randn_f16((B, G, self.T_global, Dg), seed + 4, device)
        self.ks = _randn_f16((B, G, self.T_swa, D), seed + 5, device)
        self.vs = _randn_f16((B, G, self.T_swa, D), seed + 6, device)
        self.tds = torch.tensor(self.tds_list, dtype=torch.int32, device=device)
        self.phase = torch.tensor([2] * 32 + [1], dtype=torch.uint8, device=device)
        self.ws = torch.empty(max(fa2.workspace_bytes(B, H, G, 1, Dg), fa2.workspace_bytes(B, H, G, t, Dg),
                                  fa2.mixed_workspace_bytes(B, H, G, t, 1, Dg, self.T_global, self.W_global),
                                  fa2.mixed_workspace_bytes(B, H, G, t, 1, D, self.T_swa, self.W_swa)),
                              dtype=torch.uint8, device=device)
        self.plans = {}
        n_swa, n_glob = (layers + 1) // 2, layers // 2
        dec_g = 2 * G * Dg * 2 * sum(min(x, self.W_global) for x in dec_len)
        dec_s = 2 * G * D * 2 * sum(min(x, self.W_swa) for x in dec_len)
        pre_g_pairs = t * ctx + t * (t + 1) // 2
        pre_s_pairs = t * (t + 1) // 2  # anchored window: a chunk of W tokens sees only itself
        self.bytes = n_glob * dec_g + n_swa * dec_s
        self.flops = 4 * H * (Dg * n_glob * pre_g_pairs + D * n_swa * pre_s_pairs)
        self.units = self.bytes
        self.detail = {
            "launches_per_layer": 1 if one_launch else 2,
            "decode_bytes_global_layer": dec_g, "decode_bytes_swa_layer": dec_s,
            "prefill_flops_global_layer": 4 * H * Dg * pre_g_pairs, "prefill_flops_swa_layer": 4 * H * D * pre_s_pairs,
        }

    def launch(self, i=0, kernel_mask=0):
        fa2 = self.fa2
        if not self.plans:
            for swa in (True, False):
                k, v, W = (self.ks, self.vs, self.W_swa) if swa else (self.kg, self.vg, self.W_global)
                qp, qd, op, od = (self.qp, self.qd, self.op, self.od) if swa else (self.qpg, self.qdg, self.opg, self.odg)
                if self.one_launch:
                    self.plans[swa] = (fa2.plan_flash_attention(qp, k, v, op, self.tds, self.phase, W, fa2.PHASE_PREFILL,
                                                                scale=SCALE, workspace=self.ws, decode_q=qd, decode_o=od),)
                    continue
                self.plans[swa] = (
                    fa2.plan_flash_attention(qp, k, v, op, self.tds, self.phase, W, fa2.PHASE_PREFILL, scale=SCALE),
                    fa2.plan_flash_attention(qd, k, v, od, self.tds, self.phase, W, fa2.PHASE_DECODE, scale=SCALE,
                                             workspace=self.ws),
                )
        for layer in range(self.layers):
            for plan in self.plans[layer % 2 == 0]:
                plan.launch()

    def cpu_sample(self):
        raise NotImplementedError


class RopeAppend(Workload):
    """The step in front of the attention of a prefill chunk: q/k RMSNorm + rotary embedding on fp32 scratchpads in
    engine layout ([B, t, heads, D] viewed as [B, heads, t, D]) with rotated K and normalised V written to fp16 rings,
    one launch.  Algorithmic bytes: q read and written, k and v read, both new cache rows written."""

    bound = "hbm"

    def __init__(self, device, t=8192, seed=0):
        import torch

        from g4b_amd.kernels import rope

        self.rope = rope
        self.name = f"rope_append_t{t}"
        self.t = t
        g = torch.Generator(device=device).manual_seed(seed)
        self.q = torch.randn(1, t, H, D, generator=g, device=device).permute(0, 2, 1, 3)
        self.k = torch.randn(1, t, G, D, generator=g, device=device).permute(0, 2, 1, 3)
        self.v = torch.randn(1, t, G, D, generator=g, device=device).permute(0, 2, 1, 3)
        self.q_rsos, self.k_rsos, self.v_rsos = (torch.full(x.shape[:3], float(D), device=device) for x in (self.q, self.k, self.v))
        self.freqs = torch.empty(D // 2, device=device)
        rope.populate_rope_frequencies(self.freqs, None, 1e6)
        self.qw = torch.ones(D, device=device)
        self.kw = torch.ones(D, device=device)
        self.kc = torch.zeros(1, G, t, D, dtype=torch.float16, device=device)
        self.vc = torch.zeros(1, G, t, D, dtype=torch.float16, device=device)
        self.offs = torch.zeros(1, dtype=torch.int32, device=device)
        self.bytes = t * D * (2 * H * 4 + 2 * G * 4 + 2 * G * 2)
        self.flops = 0
        self.units = self.bytes

    def launch(self, i=0, kernel_mask=0):
        # rsos = D and unit weights: the normalisation is the identity, so repeated in-place launches stay bounded
        self.rope.apply_rope_and_append(self.q, self.k, self.v, self.freqs, self.offs, self.q_rsos, self.k_rsos, self.v_rsos,
                                        self.qw, self.kw, 0.0, self.kc, self.vc)

    def cpu_sample(self):
        raise NotImplementedError


WORKLOADS = {
    "decode_batched": lambda dev: BatchedDecode(dev),
    # head dimension 512 (global-attention layers): 32 sequences, every slot attends its whole history
    "decode_batched_d512": lambda dev: BatchedDecode(dev, B=32, swa_every=0, dim=512, name="decode_batched_b32_d512"),
    # a sliding-window layer of a decode step: 64 sequences, window 512 in rings of 1023 rows (one kernel, no merge)
    "decode_swa512": lambda dev: BatchedDecode(dev, kv_ctx=1023, len_lo=1024, len_hi=16384, swa_every=0, layer_window=512,
                                               name="decode_swa512_b64"),
    "decode_single": lambda dev: SingleDecode(dev),
    "prefill_causal_2048": lambda dev: Prefill(dev, 2048),
    "prefill_causal_4096": lambda dev: Prefill(dev, 4096),  # between the configs: pairs of query tiles cut into key spans
    "prefill_causal_8192": lambda dev: Prefill(dev, 8192),
    "prefill_swa_8192": lambda dev: Prefill(dev, 8192, query_window=512),
    "prefill_causal_8192_d512": lambda dev: Prefill(dev, 8192, dim=512),
    "prefill_causal_8192_bf16": lambda dev: Prefill(dev, 8192, bf16=True),
    # the engine's own call: fp32 q / o scratchpads in token-major layout, use_fp32_dot=True (flops counted as for fp16 q)
    "prefill_causal_8192_fp32q": lambda dev: Prefill(dev, 8192, engine_call=True),
    "prefill_causal_8192_d512_fp32q": lambda dev: Prefill(dev, 8192, dim=512, engine_call=True),
    "mixed_step": lambda dev: MixedStep(dev),
    "mixed_step_two_launches": lambda dev: MixedStep(dev, one_launch=False),
    # the same step with Gemma-4's layer shapes: head dimension 256 on sliding-window layers, 512 on global ones
    "mixed_step_global_d512": lambda dev: MixedStep(dev, global_dim=512),
    "mixed_step_global_d512_two_launches": lambda dev: MixedStep(dev, global_dim=512, one_launch=False),
    "rope_append": lambda dev: RopeAppend(dev),
}


# --------------------------------------------------------------------------- timing
def settle(wl: Workload, ms: float = SETTLE_MS) -> int:
    """Untimed launches of the workload for at least ``ms`` milliseconds of device time (the board's clocks take
    some 20 ms of load to settle, whatever --warmup says); returns the number of launches."""
    import torch

    n, t0 = 0, time.perf_counter()
    while True:
        for _ in range(8):
            wl.launch(n)
            n += 1
        torch.cuda.synchronize()
        if (time.perf_counter() - t0) * 1e3 >= ms:
            return n


def time_steps(wl: Workload, steps: int, warmup: int):
    """Wall-clock of exactly ``steps`` steps between two device synchronisations -> ms per step."""
    import torch

    for i in range(warmup):
        wl.launch(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        wl.launch(warmup + i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_kernel_events(wl: Workload, steps: int, kernel_mask: int):
    """Average GPU duration (ms) of one launch of the selected kernel(s), HIP events on the launch stream."""
    import torch

    stream = torch.cuda.current_stream()
    pairs = []
    for i in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        wl.launch(i, kernel_mask)
        b.record(stream)
        pairs.append((a, b))
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in pairs)
    return sum(ts) / len(ts), ts[len(ts) // 2]


def time_dominant_kernel(wl: Workload, steps: int):
    """Average / median GPU duration (ms) of the dominant kernel over ``steps`` complete launches: the library
    dispatches it with a pair of HIP events that the runtime stamps with the begin and the end of that dispatch
    (hipExtLaunchKernelGGL), so launch gaps are not part of the figure and it agrees with a kernel trace."""
    import ctypes

    import torch

    from g4b_amd import _native

    lib = _native.load()
    torch.cuda.synchronize()
    _native.check(lib.g4b_profile_begin())
    try:
        for i in range(steps):
            wl.launch(i)
    finally:
        buf = (ctypes.c_float * (steps * 128))()
        n = lib.g4b_profile_end(buf, len(buf))
    if n < 0:
        _native.check(n)
    ts = sorted(t for t in buf[:n] if t >= 0)
    if not ts:
        return None, None, 0
    per_step = len(ts) / steps  # a step of several launches (the mixed step) sums its kernels
    left_out = 0
    if per_step == 1:
        # a dispatch that took more than five times the median was held up by something outside the kernel (seen once
        # in a while on 10 us kernels: one launch of 20 at over a millisecond); it is logged, not averaged
        med = ts[len(ts) // 2]
        held_up = [t for t in ts if t > 5 * med]
        if held_up and len(held_up) * 10 <= len(ts):
            log(f"{wl.name}: {len(held_up)} of {len(ts)} timed dispatches left out of the average: {[round(t, 4) for t in held_up]} ms "
                f"against a median of {med:.4f} ms")
            ts = [t for t in ts if t <= 5 * med]
            left_out = len(held_up)
    return sum(ts) / len(ts) * per_step, ts[len(ts) // 2], left_out


def measure(wl: Workload, steps: int, warmup: int):
    settle(wl)
    ms = time_steps(wl, steps, warmup)
    k_avg, k_med, k_left_out = time_dominant_kernel(wl, max(steps, 10))
    kmask = 1 if wl.bound == "hbm" and not isinstance(wl, MixedStep) else 0
    e_avg, _ = time_kernel_events(wl, max(steps, 10), kmask)  # event pairs around the launch: includes the gaps
    if k_avg is None:
        k_avg, k_med = e_avg, e_avg
    wl.launch(0, 0)  # leave complete results behind after kernel-only launches
    res = {"ms_per_step": ms, "kernel_ms_avg": k_avg, "kernel_ms_median": k_med, "event_pair_ms_avg": e_avg,
           "kernel_dispatches_left_out": k_left_out}
    res["GBps"] = wl.bytes / (ms * 1e-3) / 1e9
    res["TFLOPs"] = wl.flops / (ms * 1e-3) / 1e12
    if wl.bound == "hbm":
        ach = wl.bytes / (k_avg * 1e-3) / 1e9
        res["roofline"] = {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": measured_traffic_bytes(wl.key)}
    else:
        ach = wl.flops / (k_avg * 1e-3) / 1e12
        res["roofline"] = {"bound": "mfma", "achieved": round(ach, 1), "peak": FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                           "frac": round(ach / FP16_PEAK_TFLOPS, 4), "traffic": measured_traffic_bytes(wl.key)}
    if isinstance(wl, MixedStep):
        # two rooflines in one step: the decode slots' KV bytes at the HBM peak and the chunk's flops at the MFMA peak.
        # One after the other is the floor of a step that overlaps nothing; the larger of the two is the floor of a
        # step that overlaps them completely, which is what one launch for both is for: `frac` is quoted against it.
        hbm_ms = wl.bytes / (HBM_PEAK_GBPS * 1e9) * 1e3
        mfma_ms = wl.flops / (FP16_PEAK_TFLOPS * 1e12) * 1e3
        res["roofline"] = {"bound": "hbm+mfma", "decode_bytes": wl.bytes, "prefill_flops": wl.flops,
                           "floor_ms_no_overlap": round(hbm_ms + mfma_ms, 4), "floor_ms_overlap": round(max(hbm_ms, mfma_ms), 4),
                           "kernel_ms": round(k_avg, 4), "frac": round(max(hbm_ms, mfma_ms) / k_avg, 4),
                           "frac_no_overlap": round((hbm_ms + mfma_ms) / k_avg, 4),
                           # the counters give the main kernel's average bytes per dispatch over both layer kinds
                           "traffic": None if measured_traffic_bytes(wl.key) is None else measured_traffic_bytes(wl.key) * wl.layers}
    return res


def sample_power(wl, seconds):
    """Board power and shader clock while ``wl`` runs back to back for ``seconds``: power from the amdgpu hwmon node
    (microwatts, sampled between batches of launches), the shader clock from ``rocm-smi --showclocks`` (a child
    process per sample).  The second half of the samples is averaged, after the power controller has settled."""
    import glob
    import re
    import subprocess
    import threading

    import torch

    def read(path):
        try:
            with open(path) as f:
                return float(f.read().strip())
        except (OSError, ValueError):
            return None

    nodes = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")
    power_file = next((f"{n}/{leaf}" for n in nodes for leaf in ("power1_input", "power1_average") if read(f"{n}/{leaf}") is not None), None)
    cap = next((read(f"{n}/power1_cap") for n in nodes if read(f"{n}/power1_cap") is not None), None)
    watts, mhz, stop = [], [], threading.Event()

    def sampler():
        while not stop.is_set():
            if power_file:
                w = read(power_file)
                if w is not None:
                    watts.append(w / 1e6)
            try:
                out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
                m = re.search(r"sclk clock level: \S+ \((\d+)Mhz\)", out)
                if m:
                    mhz.append(int(m.group(1)))
            except (OSError, subprocess.SubprocessError):
                stop.wait(0.05)

    th = threading.Thread(target=sampler)
    th.start()
    t0, n = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            wl.launch()
        n += 20
        torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stop.set()
    th.join()
    half = lambda xs: xs[len(xs) // 2:]  # noqa: E731
    mean = lambda xs: round(sum(xs) / len(xs), 1) if xs else None  # noqa: E731
    return {"seconds": round(elapsed, 2), "ms_per_launch": round(elapsed / n * 1e3, 4), "watts": mean(half(watts)),
            "cap_watts": None if cap is None else round(cap / 1e6, 1), "sclk_mhz": mean(half(mhz)),
            "power_samples": len(watts), "clock_samples": len(mhz)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=100,
                    help="untimed steps first; the board needs some 20 ms of load before its clocks settle")
    ap.add_argument("--workload", default="decode_batched", choices=sorted(WORKLOADS))
    ap.add_argument("--no-extra", action="store_true", help="time the primary workload only")
    ap.add_argument("--workspace", choices=("static", "caller"), default="caller",
                    help="split partials in a caller-owned workspace tensor (default) or in the library's static scratch "
                         "(what the wrappers take when no workspace is passed)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-from", metavar="DIR",
                    help="no GPU work: read DIR/pmc_FETCH_SIZE_<workload> and DIR/pmc_WRITE_SIZE_<workload> (rocprofv3 "
                         "--pmc runs of this script with --copy-calibration) and update profiles/traffic.json")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 1 GiB device-to-device copies (a kernel of known traffic, used to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--sample-power", type=float, default=0.0, metavar="SECONDS",
                    help="afterwards run the primary workload back to back for SECONDS and report board power and "
                         "shader clock under it (\"power\" in the JSON line)")
    args = ap.parse_args()
    if args.traffic_from:
        print(json.dumps(traffic_from_counters(args.traffic_from), indent=1, sort_keys=True))
        return
    global WORKSPACE_MODE
    WORKSPACE_MODE = args.workspace
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the attention path shards by slot or kv head with "
                 "no exchange; nothing here uses a second device). Run with --gpus 1.")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import g4b_amd.kernels  # noqa: F401  raises when libg4b_attn.so is missing

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    log(f"device: {props.name}, {props.multi_processor_count} CUs, {props.total_memory / 2**30:.0f} GiB")
    log(f"peaks used: HBM {HBM_PEAK_GBPS:.0f} GB/s, fp16 dense MFMA {FP16_PEAK_TFLOPS:.0f} TFLOP/s")

    if args.copy_calibration:
        src = torch.empty(1 << 29, dtype=torch.float16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        log("copy calibration: 3 copies, each reads 1 GiB and writes 1 GiB")
        del src, dst

    wl = WORKLOADS[args.workload](dev)
    wl.key = args.workload
    res = measure(wl, args.steps, args.warmup)
    log(f"{wl.name}: {res['ms_per_step']:.4f} ms/step, {res['GBps']:.1f} GB/s, {res['TFLOPs']:.2f} TFLOP/s, "
        f"kernel {res['kernel_ms_avg']:.4f} ms avg (event pair around the launch: {res['event_pair_ms_avg']:.4f}) -> {res['roofline']}")

    def cpu_baseline_of(w, *sample_args):
        try:
            torch.set_num_threads(min(os.cpu_count() or 1, 16))  # the box gives one GPU 16 host cores
            secs, done, desc = w.cpu_sample(*sample_args)
        except NotImplementedError:
            return None
        unit, val = ("GB/s", done / secs / 1e9) if w.bound == "hbm" else ("TFLOP/s", done / secs / 1e12)
        c = {"value": round(val, 4), "unit": unit, "cores": torch.get_num_threads(), "kind": "port",
             "sample": f"{desc}; {secs:.2f} s; torch CPU fp32 restatement of scripts/reference_impl.py:421-443",
             "cpu_model": host_cpu_model()}
        log(f"cpu baseline ({w.name}): {c}")
        return c

    cpu = None if args.no_cpu_baseline else cpu_baseline_of(wl)
    power = None
    if args.sample_power > 0:
        power = sample_power(wl, args.sample_power)
        log(f"power under {wl.name}: {power}")

    extra = {}
    if not args.no_extra:
        del wl
        torch.cuda.empty_cache()
        for name, make in WORKLOADS.items():
            if name == args.workload:
                continue
            w = make(dev)
            w.key = name
            steps = min(max(args.steps, 10), 20)
            r = measure(w, steps, 2 if name.startswith("mixed_step") else min(args.warmup, 60))
            entry = {"ms_per_step": round(r["ms_per_step"], 4), "GB/s": round(r["GBps"], 1),
                     "TFLOP/s": round(r["TFLOPs"], 2), "roofline": r["roofline"],
                     "kernel_dispatches_left_out": r["kernel_dispatches_left_out"]}
            if isinstance(w, MixedStep):
                entry["detail"] = w.detail
            if hasattr(w, "graph_replay_ms"):
                entry["graph_replay_ms_per_step"] = round(w.graph_replay_ms(), 4)
            if name == "prefill_causal_8192" and not args.no_cpu_baseline:
                # the prefill half of the metric carries its own CPU baseline (a three-second sample)
                entry["cpu_baseline"] = cpu_baseline_of(w, 3.0)
            extra[w.name] = entry
            log(f"{w.name}: {entry}")
            del w
            torch.cuda.empty_cache()

    primary_is_hbm = res["roofline"]["bound"] == "hbm"
    head_dim = 512 if "_d512" in args.workload else D
    line = {
        "metric": METRIC,
        "value": round(res["GBps"] if primary_is_hbm else res["TFLOPs"], 2),
        "unit": "GB/s" if primary_is_hbm else "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.workload.endswith("_bf16") else ("f32" if args.workload == "rope_append" else "f16"),
        "data": "synthetic",
        "config": {"workload": args.workload, "H": H, "G": G, "D": head_dim, "scale": SCALE, "workspace": args.workspace,
                   "detail": "Q/K/V ~ N(0,1) seeded, fp32 softmax accumulation"},
        "roofline": res["roofline"],
        "cpu_baseline": cpu,
        "kernel_ms": {"avg": round(res["kernel_ms_avg"], 5), "median": round(res["kernel_ms_median"], 5),
                      "event_pair_avg": round(res["event_pair_ms_avg"], 5), "launches": max(args.steps, 10),
                      # dispatches that took more than five times the median and were left out of `avg`
                      "left_out": res["kernel_dispatches_left_out"]},
        "settle_ms": SETTLE_MS,
        "device": props.name,
        "extra": extra,
    }
    if power is not None:
        line["power"] = power
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
