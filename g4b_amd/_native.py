"""ctypes binding of libg4b_attn.so (declarations mirror ``include/g4b_attn.h``)."""

from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libg4b_attn.so"

G4B_OK = 0
G4B_ERR_INVALID_ARGUMENT = -1
G4B_ERR_UNSUPPORTED = -2
G4B_ERR_WORKSPACE = -3
G4B_ERR_LAUNCH = -4
G4B_ERR_BUSY = -5

DT_F16, DT_BF16, DT_F32 = 0, 1, 2
ABI_VERSION = 4


class AttnArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p),
        ("k_cache", C.c_void_p),
        ("v_cache", C.c_void_p),
        ("o", C.c_void_p),
        ("time_dim_sizes", C.c_void_p),
        ("user_phase", C.c_void_p),
        ("window_sizes", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_uint64),
        ("q_stride", C.c_int64 * 4),
        ("o_stride", C.c_int64 * 4),
        ("k_stride_b", C.c_int64),
        ("v_stride_b", C.c_int64),
        ("time_dim_sizes_stride", C.c_int64),
        ("user_phase_stride", C.c_int64),
        ("window_sizes_stride", C.c_int64),
        ("q_dtype", C.c_int32),
        ("o_dtype", C.c_int32),
        ("kv_dtype", C.c_int32),
        ("B", C.c_int32),
        ("H", C.c_int32),
        ("G", C.c_int32),
        ("Tq", C.c_int32),
        ("D", C.c_int32),
        ("KV_CTX", C.c_int32),
        ("ctx_window_size", C.c_int32),
        ("phase", C.c_int32),
        ("stage", C.c_int32),
        ("query_window", C.c_int32),
        ("num_workers", C.c_int32),
        ("kernel_mask", C.c_int32),
        ("use_fp32_dot", C.c_int32),
        ("on_band_block", C.c_int32),
        ("scale", C.c_float),
    ]


class KvAppendArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p),
        ("cache", C.c_void_p),
        ("cache_offsets", C.c_void_p),
        ("x_rsos", C.c_void_p),
        ("user_phase", C.c_void_p),
        ("x_stride", C.c_int64 * 4),
        ("x_rsos_stride", C.c_int64 * 3),
        ("cache_stride_b", C.c_int64),
        ("cache_offsets_stride", C.c_int64),
        ("user_phase_stride", C.c_int64),
        ("x_dtype", C.c_int32),
        ("cache_dtype", C.c_int32),
        ("cache_offsets_is_int64", C.c_int32),
        ("B", C.c_int32),
        ("G", C.c_int32),
        ("t", C.c_int32),
        ("T", C.c_int32),
        ("D", C.c_int32),
        ("phase", C.c_int32),
        ("rmsnorm_eps", C.c_float),
    ]


class AdvanceArgs(C.Structure):
    _fields_ = [
        ("input_token_ids", C.c_void_p),
        ("out_token_ids", C.c_void_p),
        ("cache_offsets", C.c_void_p),
        ("time_dim_sizes", C.c_void_p),
        ("user_phase", C.c_void_p),
        ("input_token_ids_stride1", C.c_int64),
        ("out_token_ids_stride0", C.c_int64),
        ("cache_offsets_stride", C.c_int64),
        ("time_dim_sizes_stride", C.c_int64),
        ("user_phase_stride", C.c_int64),
        ("B", C.c_int32),
    ]


class RopeArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p),
        ("k", C.c_void_p),
        ("rope_freqs", C.c_void_p),
        ("time_dim_offsets", C.c_void_p),
        ("q_rsos", C.c_void_p),
        ("k_rsos", C.c_void_p),
        ("q_rmsnorm_w", C.c_void_p),
        ("k_rmsnorm_w", C.c_void_p),
        ("v", C.c_void_p),
        ("v_rsos", C.c_void_p),
        ("k_cache", C.c_void_p),
        ("v_cache", C.c_void_p),
        ("user_phase", C.c_void_p),
        ("q_stride", C.c_int64 * 4),
        ("k_stride", C.c_int64 * 4),
        ("v_stride", C.c_int64 * 4),
        ("q_rsos_stride", C.c_int64 * 3),
        ("k_rsos_stride", C.c_int64 * 3),
        ("v_rsos_stride", C.c_int64 * 3),
        ("rope_freqs_stride", C.c_int64),
        ("q_rmsnorm_w_stride", C.c_int64),
        ("k_rmsnorm_w_stride", C.c_int64),
        ("time_dim_offsets_stride", C.c_int64),
        ("user_phase_stride", C.c_int64),
        ("k_cache_stride_b", C.c_int64),
        ("v_cache_stride_b", C.c_int64),
        ("q_dtype", C.c_int32),
        ("k_dtype", C.c_int32),
        ("v_dtype", C.c_int32),
        ("cache_dtype", C.c_int32),
        ("B", C.c_int32),
        ("H", C.c_int32),
        ("G", C.c_int32),
        ("t", C.c_int32),
        ("D", C.c_int32),
        ("Dv", C.c_int32),
        ("T", C.c_int32),
        ("phase", C.c_int32),
        ("k_writeback", C.c_int32),
        ("rmsnorm_eps", C.c_float),
    ]


EXPORTS = {
    "g4b_attn_forward": (C.c_int, [C.POINTER(AttnArgs), C.c_void_p]),
    "g4b_attn_forward_static_scratch": (C.c_int, [C.POINTER(AttnArgs), C.c_void_p]),
    "g4b_static_scratch_init": (C.c_int, []),
    "g4b_static_scratch_bytes": (C.c_uint64, []),
    "g4b_attn_forward_mixed": (C.c_int, [C.POINTER(AttnArgs), C.POINTER(AttnArgs), C.c_void_p]),
    "g4b_attn_mixed_workspace_bytes": (C.c_uint64, [C.c_int32] * 10),
    "g4b_attn_workspace_bytes": (C.c_uint64, [C.c_int32] * 6),
    "g4b_attn_default_workers": (C.c_int32, []),
    "g4b_kv_append": (C.c_int, [C.POINTER(KvAppendArgs), C.c_void_p]),
    "g4b_advance_decode_state": (C.c_int, [C.POINTER(AdvanceArgs), C.c_void_p]),
    "g4b_rope": (C.c_int, [C.POINTER(RopeArgs), C.c_void_p]),
    "g4b_rope_frequencies": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_float, C.c_void_p]),
    "g4b_profile_begin": (C.c_int, []),
    "g4b_profile_end": (C.c_int, [C.POINTER(C.c_float), C.c_int32]),
    "g4b_last_error": (C.c_char_p, []),
    "g4b_abi_version": (C.c_int32, []),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library; raise loudly when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m g4b_amd.build` "
            "(g4b_amd has no CPU or eager fallback for the attention path)"
        )
    lib = C.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in EXPORTS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.g4b_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} has ABI version {lib.g4b_abi_version()}, expected {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def last_error() -> str:
    return load().g4b_last_error().decode()


class ScratchBusyError(ValueError):
    """g4b_attn_forward_static_scratch found the static scratch in use by unfinished work on another stream."""


def check(status: int) -> None:
    """Map a g4b_status to the exception the reference raises for the same mistake."""
    if status == G4B_OK:
        return
    msg = last_error()
    if status == G4B_ERR_BUSY:
        raise ScratchBusyError(msg)
    if status in (G4B_ERR_INVALID_ARGUMENT, G4B_ERR_WORKSPACE):
        raise ValueError(msg)
    if status == G4B_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
