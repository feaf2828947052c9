"""Per-slot decode bookkeeping on the device -- drop-in for ``g4b/kernels/advance_decode_state.py``."""

from __future__ import annotations

import ctypes as C

from .. import _native
from . import utils as U


def advance_decode_state(input_token_ids, out_token_ids, cache_offsets, time_dim_sizes, user_phase, *, stream=None):
    """For slots with ``user_phase[b] == PHASE_DECODE``: ``input_token_ids[0, b] = out_token_ids[b, 0]``,
    ``cache_offsets[b] += 1``, ``time_dim_sizes[b] += 1`` (``advance_decode_state.py:52-63``).

    ``input_token_ids``: ``[t, B]`` int32; ``out_token_ids``: ``[B, >=1]`` int32; the rest ``[B]``.
    """
    U.require_tensor(input_token_ids, "input_token_ids", 2)
    U.require_tensor(out_token_ids, "out_token_ids", 2)
    for name, t in (("cache_offsets", cache_offsets), ("time_dim_sizes", time_dim_sizes), ("user_phase", user_phase)):
        U.require_tensor(t, name, 1)
    t_rows, B = U.shape_of(input_token_ids)
    # advance_decode_state.py:45-50
    if t_rows < 1 or U.shape_of(out_token_ids)[0] != B or U.shape_of(out_token_ids)[1] < 1:
        raise ValueError("input_token_ids must be [t>=1, B] and out_token_ids [B, >=1]")
    if U.shape_of(cache_offsets) != [B] or U.shape_of(time_dim_sizes) != [B] or U.shape_of(user_phase) != [B]:
        raise ValueError("cache_offsets, time_dim_sizes and user_phase must have shape [B]")
    for name, t in (
        ("input_token_ids", input_token_ids),
        ("out_token_ids", out_token_ids),
        ("cache_offsets", cache_offsets),
        ("time_dim_sizes", time_dim_sizes),
    ):
        U.int_itemsize(t, name, {"int32"})
    U.int_itemsize(user_phase, "user_phase", {"uint8"})

    a = _native.AdvanceArgs()
    a.input_token_ids, a.out_token_ids = input_token_ids.data_ptr(), out_token_ids.data_ptr()
    a.cache_offsets, a.time_dim_sizes, a.user_phase = (
        cache_offsets.data_ptr(),
        time_dim_sizes.data_ptr(),
        user_phase.data_ptr(),
    )
    a.input_token_ids_stride1 = U.strides_of(input_token_ids)[1]
    a.out_token_ids_stride0 = U.strides_of(out_token_ids)[0]
    a.cache_offsets_stride = U.strides_of(cache_offsets)[0]
    a.time_dim_sizes_stride = U.strides_of(time_dim_sizes)[0]
    a.user_phase_stride = U.strides_of(user_phase)[0]
    a.B = B
    lib = _native.load()
    _native.check(
        lib.g4b_advance_decode_state(C.byref(a), C.c_void_p(U.current_stream() if stream is None else U.stream_handle(stream)))
    )
    return None
