"""g4b_amd -- MI355X-native attention hot path of the g4b inference engine.

Drop-in replacements for ``g4b.kernels.fa2.flash_attention``,
``g4b.kernels.add_kv_to_cache.add_kv_to_cache`` and
``g4b.kernels.advance_decode_state.advance_decode_state`` backed by hand-written HIP kernels
for gfx950 behind a C ABI (``include/g4b_attn.h``, ``libg4b_attn.so``).  There is no CPU or
eager fallback: importing :mod:`g4b_amd.kernels` raises if the shared library is not built.
"""

__version__ = "0.1.0"
