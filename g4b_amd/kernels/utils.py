"""Tensor protocol and stream plumbing shared by the kernel wrappers.

The reference's launch adapter accepts its own ``Tensor`` dataclass or any object with
``shape``, ``stride`` (sequence or callable), ``dtype`` and ``data_ptr()``
(``g4b/kernels/utils.py:51-60,87-127``); strides are in elements.  The same objects are
accepted here and reduced to (pointer, shape, strides, dtype code).
"""

from __future__ import annotations

from .. import _native

_DTYPE_NAMES = {
    "float16": _native.DT_F16,
    "half": _native.DT_F16,
    "bfloat16": _native.DT_BF16,
    "float32": _native.DT_F32,
    "float": _native.DT_F32,
}
_INT_NAMES = {"int32": 4, "int64": 8, "uint8": 1, "int8": 1}


def _is_tensor_like(t) -> bool:
    return hasattr(t, "shape") and hasattr(t, "stride") and hasattr(t, "dtype") and hasattr(t, "data_ptr")


def dtype_name(t) -> str:
    """'float16', 'int32', ... for torch dtypes (``torch.float16``) and g4b DTypes (``.name``)."""
    dt = t.dtype
    name = getattr(dt, "name", None)
    if not isinstance(name, str):
        name = str(dt)
    return name.rsplit(".", 1)[-1]


def float_dtype_code(t, what: str) -> int:
    name = dtype_name(t)
    if name not in _DTYPE_NAMES:
        raise ValueError(f"{what}: unsupported dtype {name}")
    return _DTYPE_NAMES[name]


def int_itemsize(t, what: str, allowed) -> int:
    name = dtype_name(t)
    if name not in allowed:
        raise ValueError(f"{what}: dtype must be one of {sorted(allowed)}, got {name}")
    return _INT_NAMES[name]


def strides_of(t) -> list[int]:
    s = t.stride
    if isinstance(s, (list, tuple)):
        return [int(x) for x in s]
    if callable(s):
        return [int(s(i)) for i in range(len(t.shape))]
    raise RuntimeError("Failed to normalize tensor stride into list[int]")


def shape_of(t) -> list[int]:
    return [int(x) for x in t.shape]


def require_tensor(t, what: str, ndim: int):
    if not _is_tensor_like(t):
        raise TypeError(f"{what} must expose shape, stride, dtype and data_ptr()")
    if len(t.shape) != ndim:
        raise ValueError(f"{what} must have {ndim} dimensions, got shape {tuple(t.shape)}")


_stream_override = None


def set_stream(stream) -> None:
    """Pin the HIP stream kernels are enqueued on (an int / hipStream_t handle, or None).

    The reference launches everything on one engine-owned stream (``g4b/device.py:99,117-124``).
    Without an override the current PyTorch stream is used when torch has a GPU, else the
    default stream.
    """
    global _stream_override
    _stream_override = stream


def stream_handle(stream) -> int:
    """hipStream_t of a ``stream=`` argument: an int, a ``torch.cuda.Stream`` (``cuda_stream``) or a g4b stream
    (``handle``, ``g4b/device.py:99``)."""
    return int(getattr(stream, "cuda_stream", getattr(stream, "handle", stream)))


def current_stream() -> int:
    if _stream_override is not None:
        return stream_handle(_stream_override)
    try:
        import torch

        if torch.cuda.is_available():
            return int(torch.cuda.current_stream().cuda_stream)
    except ImportError:
        pass
    return 0
