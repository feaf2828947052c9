"""q/k RMSNorm + rotary embedding -- drop-in for ``g4b/kernels/rope.py``, plus the fused ring append."""

from __future__ import annotations

import ctypes as C

from .. import _native
from . import utils as U


def _f32_vector(t, what: str, n: int):
    U.require_tensor(t, what, 1)
    if U.shape_of(t) != [n]:
        raise ValueError(f"{what} must have shape [{n}], got {tuple(t.shape)}")
    if U.float_dtype_code(t, what) != _native.DT_F32:
        raise ValueError(f"{what} must be float32")
    return t.data_ptr(), U.strides_of(t)[0]


def _rsos(t, what: str, shape):
    U.require_tensor(t, what, 3)
    if U.shape_of(t) != list(shape):
        raise ValueError(f"{what} must have shape {list(shape)}, got {tuple(t.shape)}")
    if U.float_dtype_code(t, what) != _native.DT_F32:
        raise ValueError(f"{what} must be float32")
    return t.data_ptr(), (C.c_int64 * 3)(*U.strides_of(t))


def _bind(q, k, rope_freqs, time_dim_offsets, q_rsos, k_rsos, q_rmsnorm_w, k_rmsnorm_w, rmsnorm_eps):
    U.require_tensor(q, "q", 4)
    U.require_tensor(k, "k", 4)
    U.require_tensor(time_dim_offsets, "time_dim_offsets", 1)
    B, H, t, D = U.shape_of(q)
    Bk, G, tk, Dk = U.shape_of(k)
    # the reference's static asserts (rope.py:149-164)
    if (Bk, tk, Dk) != (B, t, D):
        raise ValueError(f"q {tuple(q.shape)} and k {tuple(k.shape)} must agree in batch, tokens and head dim")
    if D % 2:
        raise ValueError("head dim must be even")
    if U.shape_of(time_dim_offsets) != [B]:
        raise ValueError("time_dim_offsets must have shape [B]")
    U.int_itemsize(time_dim_offsets, "time_dim_offsets", {"int32"})
    a = _native.RopeArgs()
    a.q, a.k = q.data_ptr(), k.data_ptr()
    a.q_stride = (C.c_int64 * 4)(*U.strides_of(q))
    a.k_stride = (C.c_int64 * 4)(*U.strides_of(k))
    a.rope_freqs, a.rope_freqs_stride = _f32_vector(rope_freqs, "rope_freqs", D // 2)
    a.q_rmsnorm_w, a.q_rmsnorm_w_stride = _f32_vector(q_rmsnorm_w, "q_rmsnorm_w", D)
    a.k_rmsnorm_w, a.k_rmsnorm_w_stride = _f32_vector(k_rmsnorm_w, "k_rmsnorm_w", D)
    a.q_rsos, a.q_rsos_stride = _rsos(q_rsos, "q_rsos", (B, H, t))
    a.k_rsos, a.k_rsos_stride = _rsos(k_rsos, "k_rsos", (B, G, t))
    a.time_dim_offsets = time_dim_offsets.data_ptr()
    a.time_dim_offsets_stride = U.strides_of(time_dim_offsets)[0]
    a.q_dtype = U.float_dtype_code(q, "q")
    a.k_dtype = U.float_dtype_code(k, "k")
    a.B, a.H, a.G, a.t, a.D = B, H, G, t, D
    a.rmsnorm_eps = float(rmsnorm_eps)
    return a, (B, H, G, t, D)


def apply_rope(q, k, rope_freqs, time_dim_offsets, q_rsos, k_rsos, q_rmsnorm_w, k_rmsnorm_w, rmsnorm_eps: float, *, stream=None):
    """In place, for ``x`` in ``(q, k)``: ``x <- rope(x * rsqrt(x_rsos / D + eps) * x_rmsnorm_w)``.

    Signature of the reference wrapper (``rope.py:207-217``).  ``q``: ``[B, H, t, D]``, ``k``: ``[B, G, t, D]`` strided
    views; ``rope_freqs``: ``[D/2]`` fp32; ``time_dim_offsets``: ``[B]`` int32 position of each slot's first new token;
    ``*_rsos``: ``[B, heads, t]`` fp32 row sums of squares; ``*_rmsnorm_w``: ``[D]`` fp32.  Column ``j < D/2`` is
    rotated with column ``j + D/2`` by the angle ``(time_dim_offsets[b] + t) * rope_freqs[j]`` (``rope.py:177-186,36-37``).
    """
    a, _ = _bind(q, k, rope_freqs, time_dim_offsets, q_rsos, k_rsos, q_rmsnorm_w, k_rmsnorm_w, rmsnorm_eps)
    lib = _native.load()
    _native.check(lib.g4b_rope(C.byref(a), C.c_void_p(U.current_stream() if stream is None else U.stream_handle(stream))))
    return None


def apply_rope_and_append(
    q, k, v, rope_freqs, cache_offsets, q_rsos, k_rsos, v_rsos, q_rmsnorm_w, k_rmsnorm_w, rmsnorm_eps: float,
    k_cache, v_cache, user_phase=None, phase: int = 0, *, k_writeback: bool = False, stream=None,
):
    """One launch for the engine's ``apply_rope`` + ``add_kv_to_cache(k)`` + ``add_kv_to_cache(v, v_rsos)``
    (``g4b/models/gemma4e.py:564-590``): q is rotated in place, rotated K and (weightlessly normalised) V go to ring
    row ``(t + cache_offsets[b]) % T`` of every slot with ``user_phase[b] == phase`` (all slots without ``user_phase``).
    The K scratchpad itself is left alone unless ``k_writeback`` -- nothing reads it after the append.
    """
    assert isinstance(phase, int)  # add_kv_to_cache.py:171
    a, (B, H, G, t, D) = _bind(q, k, rope_freqs, cache_offsets, q_rsos, k_rsos, q_rmsnorm_w, k_rmsnorm_w, rmsnorm_eps)
    U.require_tensor(v, "v", 4)
    U.require_tensor(k_cache, "k_cache", 4)
    U.require_tensor(v_cache, "v_cache", 4)
    Bv, Gv, tv, Dv = U.shape_of(v)
    if (Bv, Gv, tv) != (B, G, t):
        raise ValueError(f"v {tuple(v.shape)} must agree with k in batch, heads and tokens")
    Bc, Gc, T, Dc = U.shape_of(k_cache)
    if (Bc, Gc, Dc) != (B, G, D):  # add_kv_to_cache.py:105-107
        raise ValueError(f"k {tuple(k.shape)} and k_cache {tuple(k_cache.shape)} must agree in B, G and D")
    if U.shape_of(v_cache) != [B, G, T, Dv]:
        raise ValueError(f"v_cache {tuple(v_cache.shape)} must be [B, G, T, Dv] = {[B, G, T, Dv]}")
    if t > T:  # add_kv_to_cache.py:119
        raise ValueError(f"cannot append t={t} tokens to a ring of T={T} rows")
    for name, c, d in (("k_cache", k_cache, D), ("v_cache", v_cache, Dv)):
        cs = U.strides_of(c)
        if cs[3] != 1 or cs[2] != d or cs[1] != T * d:
            raise ValueError(f"{name} must be contiguous inside a slot")
    cdt = U.float_dtype_code(k_cache, "k_cache")
    if U.float_dtype_code(v_cache, "v_cache") != cdt:
        raise ValueError("k_cache and v_cache must have the same dtype")
    a.v, a.k_cache, a.v_cache = v.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr()
    a.v_stride = (C.c_int64 * 4)(*U.strides_of(v))
    a.v_dtype = U.float_dtype_code(v, "v")
    a.cache_dtype = cdt
    a.k_cache_stride_b, a.v_cache_stride_b = U.strides_of(k_cache)[0], U.strides_of(v_cache)[0]
    if v_rsos is not None:
        a.v_rsos, a.v_rsos_stride = _rsos(v_rsos, "v_rsos", (B, G, t))
    if user_phase is not None:
        U.require_tensor(user_phase, "user_phase", 1)
        U.int_itemsize(user_phase, "user_phase", {"uint8"})
        if U.shape_of(user_phase) != [B]:
            raise ValueError("user_phase must have shape [B]")
        a.user_phase = user_phase.data_ptr()
        a.user_phase_stride = U.strides_of(user_phase)[0]
    a.Dv, a.T, a.phase, a.k_writeback = Dv, T, phase, 1 if k_writeback else 0
    lib = _native.load()
    _native.check(lib.g4b_rope(C.byref(a), C.c_void_p(U.current_stream() if stream is None else U.stream_handle(stream))))
    return None


def populate_rope_frequencies(out, freq_scalars, freq_base: float, *, stream=None):
    """``out[j] = 1 / freq_base ** (j / n)`` [``/ freq_scalars[j]``] (``rope.py:262-293``); run once at load."""
    U.require_tensor(out, "out", 1)
    n = U.shape_of(out)[0]
    if U.float_dtype_code(out, "out") != _native.DT_F32:
        raise ValueError("out must be float32")
    sc_ptr, sc_stride = None, 0
    if freq_scalars is not None:
        assert out.shape[-1] == freq_scalars.shape[-1]  # rope.py:291
        sc_ptr, sc_stride = _f32_vector(freq_scalars, "freq_scalars", n)
    lib = _native.load()
    _native.check(
        lib.g4b_rope_frequencies(
            C.c_void_p(out.data_ptr()), C.c_void_p(sc_ptr), n, U.strides_of(out)[0], sc_stride, float(freq_base),
            C.c_void_p(U.current_stream() if stream is None else U.stream_handle(stream)),
        )
    )
    return None
