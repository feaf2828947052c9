"""Ring append of new K or V rows -- drop-in for ``g4b/kernels/add_kv_to_cache.py``."""

from __future__ import annotations

import ctypes as C

from .. import _native
from . import utils as U


def add_kv_to_cache(
    x,
    cache,
    cache_offsets,
    rmsnorm_eps: float,
    x_rsos=None,
    user_phase=None,
    phase: int = 0,
    *,
    stream=None,
):
    """``cache[b, g, (t + cache_offsets[b]) % T, :] = x[b, g, t, :]`` for every in-phase slot.

    Signature of the reference wrapper (``add_kv_to_cache.py:162-170``).  ``x``: ``[B, G, t, D]``
    strided view; ``cache``: ``[B, G, T, D]``; ``cache_offsets``: ``[B]`` int32 (or int64, as the
    reference's test passes); ``x_rsos``: optional ``[B, G, t]`` row sums of squares which turn the
    copy into the weightless RMSNorm ``x * rsqrt(x_rsos / D + rmsnorm_eps)``
    (``add_kv_to_cache.py:148-151``); with ``user_phase`` given, slots whose phase differs from
    ``phase`` are skipped (``add_kv_to_cache.py:124-126``).
    """
    assert isinstance(phase, int)  # add_kv_to_cache.py:171
    U.require_tensor(x, "x", 4)
    U.require_tensor(cache, "cache", 4)
    U.require_tensor(cache_offsets, "cache_offsets", 1)
    B, G, t, D = U.shape_of(x)
    Bc, Gc, T, Dc = U.shape_of(cache)
    # add_kv_to_cache.py:105-119
    if (Bc, Gc, Dc) != (B, G, D):
        raise ValueError(f"x {tuple(x.shape)} and cache {tuple(cache.shape)} must agree in B, G and D")
    if U.shape_of(cache_offsets) != [B]:
        raise ValueError("cache_offsets must have shape [B]")
    if t > T:
        raise ValueError(f"cannot append t={t} tokens to a ring of T={T} rows")
    cs = U.strides_of(cache)
    if cs[3] != 1 or cs[2] != D or cs[1] != T * D:
        raise ValueError("cache must be contiguous inside a slot")

    a = _native.KvAppendArgs()
    a.x, a.cache, a.cache_offsets = x.data_ptr(), cache.data_ptr(), cache_offsets.data_ptr()
    a.x_stride = (C.c_int64 * 4)(*U.strides_of(x))
    a.cache_stride_b = cs[0]
    a.cache_offsets_stride = U.strides_of(cache_offsets)[0]
    a.cache_offsets_is_int64 = 1 if U.int_itemsize(cache_offsets, "cache_offsets", {"int32", "int64"}) == 8 else 0
    if x_rsos is not None:
        U.require_tensor(x_rsos, "x_rsos", 3)
        if U.shape_of(x_rsos) != [B, G, t]:
            raise ValueError("x_rsos must have shape [B, G, t]")
        if U.float_dtype_code(x_rsos, "x_rsos") != _native.DT_F32:
            raise ValueError("x_rsos must be float32")
        a.x_rsos = x_rsos.data_ptr()
        a.x_rsos_stride = (C.c_int64 * 3)(*U.strides_of(x_rsos))
    if user_phase is not None:
        U.require_tensor(user_phase, "user_phase", 1)
        U.int_itemsize(user_phase, "user_phase", {"uint8"})
        if U.shape_of(user_phase) != [B]:
            raise ValueError("user_phase must have shape [B]")
        a.user_phase = user_phase.data_ptr()
        a.user_phase_stride = U.strides_of(user_phase)[0]
    a.x_dtype = U.float_dtype_code(x, "x")
    a.cache_dtype = U.float_dtype_code(cache, "cache")
    a.B, a.G, a.t, a.T, a.D = B, G, t, T, D
    a.phase = phase
    a.rmsnorm_eps = float(rmsnorm_eps)
    lib = _native.load()
    _native.check(lib.g4b_kv_append(C.byref(a), C.c_void_p(U.current_stream() if stream is None else U.stream_handle(stream))))
    return None
