"""Flash attention over the per-slot ring KV cache -- drop-in for ``g4b/kernels/fa2.py``.

Same public surface as the reference module: the ``STAGE_*`` / ``PHASE_*`` constants
(``fa2.py:14-34``) and :func:`flash_attention` with the reference's positional signature
(``fa2.py:634-652``).  The work is done by ``g4b_attn_forward`` of ``libg4b_attn.so``
(hand-written HIP for gfx950); there is no other code path.
"""

from __future__ import annotations

import ctypes as C
import warnings

from .. import _native
from . import utils as U

# g4b/kernels/fa2.py:14-19
STAGE_FULL = 1
STAGE_ON_BAND = 2
STAGE_CAUSAL = STAGE_FULL | STAGE_ON_BAND
INNER_STAGE_OFF_BAND = 1
INNER_STAGE_ON_BAND = 2
INNER_STAGE_FULL = 3
# g4b/kernels/fa2.py:29-31 -- per-slot phase: 0 unallocated (skipped by every launch), 1 prefill, 2 decode
PHASE_UNALLOCATED = 0
PHASE_PREFILL = 1
PHASE_DECODE = 2

MAX_DECODE_ROWS = 16  # (H/G) * Tq up to which a launch takes the split-KV streaming kernel

_warned = set()


def _warn_once(key: str, message: str) -> None:
    if key not in _warned:
        _warned.add(key)
        warnings.warn(message, RuntimeWarning, stacklevel=3)


def _launch(entry, args_ref, stream, implicit_static: bool) -> None:
    """The C call.  A call that took the library's static scratch by default (``workspace=None``) and finds it in use
    by unfinished work on another stream runs without scratch instead (no key split: correct, slower) and says so
    once; a call that asked for it (``workspace="static"``) gets the error."""
    rc = entry(args_ref, stream)
    if rc == _native.G4B_ERR_BUSY and implicit_static:
        _warn_once("busy", "flash_attention: the library's static scratch is in use on another stream; this launch runs "
                   "without a key split.  Pass workspace= (see workspace_bytes) to calls that overlap on one GPU.")
        rc = _native.load().g4b_attn_forward(args_ref, stream)
    if rc:
        _native.check(rc)


def workspace_bytes(B: int, H: int, G: int, Tq: int, D: int, num_workers: int = 0) -> int:
    """Bytes of scratch that let a launch of this shape split keys: over ``num_workers`` waves when it is
    decode-shaped, over workgroups when it is a prefill shape that would not fill the chip (0 otherwise)."""
    return int(_native.load().g4b_attn_workspace_bytes(B, H, G, Tq, D, num_workers))


def mixed_workspace_bytes(B: int, H: int, G: int, Tq_prefill: int, Tq_decode: int, D: int, KV_CTX: int, ctx_window_size: int,
                          has_window_sizes: bool = False, num_workers: int = 0) -> int:
    """Bytes of scratch that let both halves of a mixed launch (``decode_q=`` / ``decode_o=``) split keys."""
    return int(_native.load().g4b_attn_mixed_workspace_bytes(B, H, G, Tq_prefill, Tq_decode, D, KV_CTX, ctx_window_size,
                                                             1 if has_window_sizes else 0, num_workers))


def _bind_mixed(q, k_cache, v_cache, o, time_dim_sizes, user_phase, ctx_window_size, phase, decode_q, decode_o, decode_phase,
                workspace, **kw):
    """Argument blocks of the two halves of a mixed launch and the call that launches them as one grid."""
    if decode_q is None or decode_o is None:
        raise ValueError("decode_q and decode_o go together")
    if isinstance(workspace, str):
        raise ValueError("a mixed launch takes workspace=<uint8 tensor> (see mixed_workspace_bytes) or none")
    kw = dict(kw)
    num_workers = kw.pop("num_workers", 0)
    a, keep_a, _ = _bind(q, k_cache, v_cache, o, time_dim_sizes, user_phase, ctx_window_size, phase, workspace=False, **kw)
    d, keep_d, _ = _bind(decode_q, k_cache, v_cache, decode_o, time_dim_sizes, user_phase, ctx_window_size, decode_phase,
                         workspace=False, num_workers=num_workers, **kw)
    ws = None if workspace is False else workspace
    if ws is not None:
        a.workspace = ws.data_ptr()
        a.workspace_bytes = int(ws.numel()) * int(ws.element_size())
    lib = _native.load()
    d_ref = C.byref(d)

    def entry(a_ref, stream):
        return lib.g4b_attn_forward_mixed(a_ref, d_ref, stream)

    return a, (keep_a, keep_d, d, ws), entry


def _bind(
    q,
    k_cache,
    v_cache,
    o,
    time_dim_sizes,
    user_phase,
    ctx_window_size: int,
    phase: int,
    partial_o=None,
    partial_l=None,
    partial_m=None,
    *,
    use_grouped_query_tile: bool = True,
    warp_specialize: bool = False,
    is_hopper: bool = False,
    use_fp32_dot: bool = False,
    stage: int = STAGE_CAUSAL,
    scale: float = 1.0,
    query_window: int | None = None,
    window_sizes=None,
    workspace=None,
    num_workers: int = 0,
    kernel_mask: int = 0,
    on_band_block: int | None = None,
    limit_kv_splits: bool = False,
):
    """Validate the arguments like the reference and fill the C argument block (plus the objects it points into)."""
    assert isinstance(phase, int)  # fa2.py:653
    if (partial_o is None) != (partial_l is None) or (partial_o is None) != (partial_m is None):
        raise ValueError("partial_o, partial_l, and partial_m must be provided together")

    U.require_tensor(q, "q", 4)
    U.require_tensor(o, "o", 4)
    U.require_tensor(k_cache, "k_cache", 4)
    U.require_tensor(v_cache, "v_cache", 4)
    U.require_tensor(time_dim_sizes, "time_dim_sizes", 1)
    U.require_tensor(user_phase, "user_phase", 1)
    B, H, Tq, D = U.shape_of(q)
    Bk, G, KV_CTX, Dk = U.shape_of(k_cache)
    # the reference's static asserts (fa2.py:289-320)
    if U.shape_of(o) != [B, H, Tq, D]:
        raise ValueError(f"o shape {tuple(o.shape)} must equal q shape {tuple(q.shape)}")
    if U.shape_of(v_cache) != [Bk, G, KV_CTX, Dk]:
        raise ValueError("k_cache and v_cache must have the same shape")
    if Bk != B or Dk != D:
        raise ValueError("q and the caches must agree in batch size and head dim")
    if U.shape_of(time_dim_sizes) != [B] or U.shape_of(user_phase) != [B]:
        raise ValueError("time_dim_sizes and user_phase must have shape [B]")
    if G == 0 or H % G:
        raise ValueError("number of query heads must be a multiple of the number of kv heads")
    U.int_itemsize(time_dim_sizes, "time_dim_sizes", {"int32"})
    U.int_itemsize(user_phase, "user_phase", {"uint8"})
    ks, vs = U.strides_of(k_cache), U.strides_of(v_cache)
    for name, s in (("k_cache", ks), ("v_cache", vs)):
        if s[3] != 1 or s[2] != D or s[1] != KV_CTX * D:  # fa2.py:315-320
            raise ValueError(f"{name} must be contiguous inside a slot")
    kv_dt = U.float_dtype_code(k_cache, "k_cache")
    if U.float_dtype_code(v_cache, "v_cache") != kv_dt:
        raise ValueError("k_cache and v_cache must have the same dtype")
    max_kv_splits = 1
    if partial_o is not None:
        max_kv_splits = min(int(partial_o.shape[0]), int(partial_l.shape[0]), int(partial_m.shape[0]))  # fa2.py:658

    lib = _native.load()
    if limit_kv_splits and max_kv_splits > 1 and (H // G) * Tq <= MAX_DECODE_ROWS:
        # MAX_KV_SPLITS of the reference (fa2.py:658) as a bound: no more workers than max_kv_splits per (slot, kv head)
        cap = B * G * max_kv_splits
        default = int(lib.g4b_attn_default_workers()) * 256 // max(D, 256)  # a worker at head dimension 512 is two waves
        num_workers = min(num_workers or default, cap)
    a = _native.AttnArgs()
    a.q, a.k_cache, a.v_cache, a.o = q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), o.data_ptr()
    a.time_dim_sizes, a.user_phase = time_dim_sizes.data_ptr(), user_phase.data_ptr()
    a.q_stride = (C.c_int64 * 4)(*U.strides_of(q))
    a.o_stride = (C.c_int64 * 4)(*U.strides_of(o))
    a.k_stride_b, a.v_stride_b = ks[0], vs[0]
    a.time_dim_sizes_stride = U.strides_of(time_dim_sizes)[0]
    a.user_phase_stride = U.strides_of(user_phase)[0]
    if window_sizes is not None:
        U.require_tensor(window_sizes, "window_sizes", 1)
        U.int_itemsize(window_sizes, "window_sizes", {"int32"})
        if U.shape_of(window_sizes) != [B]:
            raise ValueError("window_sizes must have shape [B]")
        a.window_sizes = window_sizes.data_ptr()
        a.window_sizes_stride = U.strides_of(window_sizes)[0]
    a.q_dtype = U.float_dtype_code(q, "q")
    a.o_dtype = U.float_dtype_code(o, "o")
    a.kv_dtype = kv_dt
    a.B, a.H, a.G, a.Tq, a.D, a.KV_CTX = B, H, G, Tq, D, KV_CTX
    a.ctx_window_size = int(ctx_window_size)
    a.phase = phase
    a.stage = int(stage)
    a.query_window = 0 if query_window is None else int(query_window)
    if query_window is not None and a.query_window < 1:
        raise ValueError("query_window must be a positive int or None")
    a.num_workers = int(num_workers)
    a.kernel_mask = int(kernel_mask)
    a.use_fp32_dot = 1 if use_fp32_dot else 0
    if int(stage) == STAGE_ON_BAND and on_band_block is None:
        raise ValueError("STAGE_ON_BAND alone needs on_band_block= (the reference's autotuned Q_BLOCKSIZE_T)")
    a.on_band_block = 0 if on_band_block is None else int(on_band_block)
    a.scale = float(scale)

    if isinstance(workspace, str) and workspace != "static":
        raise ValueError('workspace must be a uint8 tensor, None, False or "static"')
    static = False
    ws = None
    if workspace is False:
        pass  # no scratch at all: nothing is split
    elif workspace is None or isinstance(workspace, str):
        # Nothing is ever allocated here: the split partials go to the library's own scratch array
        # (g4b_attn_forward_static_scratch).  A decode-shaped launch splits only when the reference's split buffers
        # were passed (fa2.py:658) or the array was asked for by name; a prefill shape whose in-phase slots may bring fewer workgroups than the chip has
        # compute units (chunked prefill, short prompts) splits every item's keys.  A launch whose partials would not
        # fit the array runs unsplit.
        decode_shaped = (H // G) * Tq <= MAX_DECODE_ROWS
        need = workspace_bytes(B, H, G, Tq, D, num_workers if decode_shaped else 0)
        wanted = need > 0 and (workspace == "static" or not decode_shaped or max_kv_splits > 1)
        static = wanted and need <= int(lib.g4b_static_scratch_bytes())
        if wanted and not static:
            _warn_once("too big", f"flash_attention: this launch would split keys through {need} bytes of partials, more than "
                       f"the library's static scratch holds ({int(lib.g4b_static_scratch_bytes())}); it runs without a key "
                       "split.  Pass workspace= (see workspace_bytes) to split it.")
    else:
        ws = workspace
    if ws is not None:
        a.workspace = ws.data_ptr()
        a.workspace_bytes = int(ws.numel()) * int(ws.element_size()) if hasattr(ws, "numel") else int(ws.nbytes)

    entry = lib.g4b_attn_forward_static_scratch if static else lib.g4b_attn_forward
    return a, (q, k_cache, v_cache, o, time_dim_sizes, user_phase, window_sizes, ws), entry


def flash_attention(
    q,
    k_cache,
    v_cache,
    o,
    time_dim_sizes,
    user_phase,
    ctx_window_size: int,
    phase: int,
    partial_o=None,
    partial_l=None,
    partial_m=None,
    *,
    use_grouped_query_tile: bool = True,
    warp_specialize: bool = False,
    is_hopper: bool = False,
    use_fp32_dot: bool = False,
    stage: int = STAGE_CAUSAL,
    scale: float = 1.0,
    query_window: int | None = None,
    window_sizes=None,
    workspace=None,
    num_workers: int = 0,
    kernel_mask: int = 0,
    on_band_block: int | None = None,
    limit_kv_splits: bool = False,
    stream=None,
    decode_q=None,
    decode_o=None,
    decode_phase: int = PHASE_DECODE,
):
    """``o[b, h, i] = softmax(scale * q[b, h, i] . K_b^T + mask) V_b`` for every in-phase slot ``b``.

    Positional arguments and the first five keywords are the reference's (``fa2.py:634-652``):

    * ``q``, ``o``: ``[B, H, Tq, D]`` (strided views allowed, unit stride in ``D``);
      ``k_cache``, ``v_cache``: ``[B, G, KV_CTX, D]`` rings; ``time_dim_sizes``: ``[B]`` int32;
      ``user_phase``: ``[B]`` uint8 -- slots with ``user_phase[b] != phase`` are skipped and their
      rows of ``o`` stay untouched.
    * ``partial_o/l/m``: the reference's split-KV scratch.  All three or none
      (``ValueError`` otherwise, ``fa2.py:656-657``).  Passing them allows a decode launch to
      split keys across workgroups, as in the reference; the partials themselves live in
      ``workspace=`` (or the library's static scratch) with this library's own layout, and the
      contents of ``partial_*`` are left unspecified.
    * ``use_grouped_query_tile``, ``warp_specialize``, ``is_hopper``: tuning knobs of the Triton
      kernel; accepted and ignored (the GQA group is always packed).
    * ``use_fp32_dot`` (``fa2.py:85-88``): ``False`` rounds a wider query to the cache's 16-bit type
      before ``K Q^T``, as the reference's ``q.to(tl.float16)`` does; ``True`` (what the engine passes
      with its fp32 scratchpads, ``g4b/models/gemma4e.py:606``) feeds the product with the query as
      the sum of two 16-bit operands, value and rounding error, so the scores are those of the
      unrounded query.  The products run on fp16/bf16 MFMA with fp32 accumulation either way.
    * ``stage``: ``STAGE_CAUSAL``, ``STAGE_FULL``, or ``STAGE_ON_BAND`` together with ``on_band_block=``.

    The tuned kernels serve head dimensions 128, 256 and 512 on fp16 / bf16 caches; other head dimensions
    (multiples of 8 up to 1024), query-head groups that do not divide a workgroup's 128 rows, an fp32 cache
    (the reference's ``G4B_DTKV_FP32`` switch, ``g4b/models/gemma4e.py:32``) and ``STAGE_ON_BAND`` run on a plain
    fp32 kernel: same results, a fraction of the speed.

    Keyword-only extensions, with defaults that reproduce the reference:

    * ``scale`` (1.0, ``fa2.py:89``); ``query_window`` (None = anchored window; an int hides keys with
      ``q_pos - k_pos >= query_window`` as ``scripts/reference_impl.py:440-441`` does);
      ``window_sizes`` (``[B]`` int32 per-slot ``ctx_window_size``); ``workspace`` (uint8 tensor
      holding the split partials of this call -- size it with :func:`workspace_bytes` next to the engine's
      ``fa_gqa_partial_o`` (``g4b/models/gemma4e.py:819-821``); ``None`` or ``"static"`` = the library's built-in
      scratch array through ``g4b_attn_forward_static_scratch``: nothing is allocated, a launch whose partials exceed
      ``g4b_static_scratch_bytes()`` runs unsplit, and calls that overlap on one GPU (two streams) must not share it,
      so give every stream but one a workspace of its own; ``False`` = no scratch, never split); ``num_workers``; ``kernel_mask`` (profiling:
      bit 0 main kernel, bit 1 merge kernel, 0 = both); ``stream``; ``on_band_block`` (with ``STAGE_ON_BAND``: the
      reference's ``Q_BLOCKSIZE_T``, ``fa2.py:56,61`` -- query ``i`` sees the keys of its own block of that many
      positions up to itself; the reference's result for this stage depends on what its autotuner picked).
    * ``decode_q``, ``decode_o`` (``[B, H, 1, D]``), ``decode_phase``: a mixed step in one launch.  The reference
      serves a step that holds prefill-phase and decode-phase slots with two calls over the same batch tensors,
      because its kernel skips per slot on ``user_phase[b] != PHASE`` (``fa2.py:332-335``), and its scheduler avoids
      such steps (``g4b/scheduler.py:66,96-98``).  With these two tensors given, this call (the chunk: ``q``, ``o``,
      ``phase``) also computes ``decode_o`` from ``decode_q`` for the slots in ``decode_phase``, in the same grid:
      the chunk's workgroups and the decode stream's run on different compute units at the same time.  Same results
      as the two calls.  ``workspace`` must then be a tensor of :func:`mixed_workspace_bytes` bytes (or absent: no
      half splits its keys).  Head dimensions 256 and 512.

    Returns ``(None, None)`` in place of the reference's two launch handles, which its callers
    ignore (``g4b/models/gemma4e.py:593-607``).
    """
    a, _keep, entry = _bind_call(
        q, k_cache, v_cache, o, time_dim_sizes, user_phase, ctx_window_size, phase, partial_o, partial_l, partial_m,
        use_grouped_query_tile=use_grouped_query_tile, warp_specialize=warp_specialize, is_hopper=is_hopper,
        use_fp32_dot=use_fp32_dot, stage=stage, scale=scale, query_window=query_window, window_sizes=window_sizes,
        workspace=workspace, num_workers=num_workers, kernel_mask=kernel_mask, on_band_block=on_band_block,
        limit_kv_splits=limit_kv_splits, decode_q=decode_q, decode_o=decode_o, decode_phase=decode_phase,
    )
    _launch(entry, C.byref(a), C.c_void_p(U.current_stream() if stream is None else U.stream_handle(stream)), workspace is None)
    return None, None


def _bind_call(q, k_cache, v_cache, o, time_dim_sizes, user_phase, ctx_window_size, phase, partial_o=None, partial_l=None,
               partial_m=None, *, workspace=None, decode_q=None, decode_o=None, decode_phase=PHASE_DECODE, **kw):
    """Arguments of :func:`flash_attention` (without ``stream``) -> (argument block, objects to keep alive, entry point)."""
    if decode_q is not None or decode_o is not None:
        if partial_o is not None or partial_l is not None or partial_m is not None:
            raise ValueError("a mixed launch takes its scratch through workspace=, not partial_o/l/m")
        return _bind_mixed(q, k_cache, v_cache, o, time_dim_sizes, user_phase, ctx_window_size, phase,
                           decode_q, decode_o, decode_phase, workspace, **kw)
    return _bind(q, k_cache, v_cache, o, time_dim_sizes, user_phase, ctx_window_size, phase,
                 partial_o, partial_l, partial_m, workspace=workspace, **kw)


class AttentionPlan:
    """A bound ``flash_attention`` call: arguments validated once, every ``launch()`` is the bare C call.

    The engine records its steps into graphs (``g4b/lifecycle.py:29-53``), which is how the reference keeps
    Python out of the decode loop; outside a graph this gives the same effect for callers whose tensors do not
    move between steps (the caches, scratchpads and per-slot integer tensors of a serving engine never do).  The
    plan holds references to the tensors it points into.
    """

    def __init__(self, args, keep, entry, implicit_static=False):
        self._args, self._keep, self._entry = args, keep, entry
        self._implicit_static = implicit_static
        self._ref = C.byref(args)

    def launch(self, stream=None) -> None:
        st = C.c_void_p(U.current_stream() if stream is None else U.stream_handle(stream))
        rc = self._entry(self._ref, st)
        if rc:
            _launch(self._entry, self._ref, st, self._implicit_static)  # the slow path: fall back or raise


def plan_flash_attention(*args, **kwargs) -> AttentionPlan:
    """Same arguments as :func:`flash_attention`, positional or by keyword (``stream`` is ignored: it is given to
    ``launch``); returns an :class:`AttentionPlan`."""
    kwargs.pop("stream", None)
    return AttentionPlan(*_bind_call(*args, **kwargs), implicit_static=kwargs.get("workspace") is None)
