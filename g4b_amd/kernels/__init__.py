"""Kernel wrappers with the reference's module layout (``g4b/kernels/{fa2,add_kv_to_cache,advance_decode_state,rope}.py``).

Importing this package loads ``libg4b_attn.so`` and raises if it has not been built.
"""

from .. import _native

_native.load()

from . import add_kv_to_cache, advance_decode_state, fa2, rope, utils  # noqa: E402,F401
from .add_kv_to_cache import add_kv_to_cache as add_kv_to_cache_fn  # noqa: E402,F401
from .advance_decode_state import advance_decode_state as advance_decode_state_fn  # noqa: E402,F401
from .fa2 import flash_attention  # noqa: E402,F401
