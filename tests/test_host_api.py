"""CPU-side checks of the C ABI and the Python boundary (no GPU, no compute calls)."""

import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def native():
    from g4b_amd import _native

    if not _native.LIB_PATH.exists():
        from g4b_amd.build import build

        build()
    _native.load()
    return _native


def test_library_exports_every_declared_symbol(native):
    header = (ROOT / "include" / "g4b_attn.h").read_text()
    declared = set(re.findall(r"\b(g4b_[a-z_]+)\s*\(", header))
    assert declared == set(native.EXPORTS), declared ^ set(native.EXPORTS)
    lib = ctypes.CDLL(str(native.LIB_PATH))
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.g4b_abi_version() == native.ABI_VERSION


def test_struct_layouts_match_the_header(native):
    """Field order and C types of the ctypes mirrors follow the header's structs."""
    header = (ROOT / "include" / "g4b_attn.h").read_text()
    ctype_of = {
        "void*": ctypes.c_void_p,
        "int32_t*": ctypes.c_void_p,
        "uint8_t*": ctypes.c_void_p,
        "float*": ctypes.c_void_p,
        "uint64_t": ctypes.c_uint64,
        "int64_t": ctypes.c_int64,
        "int32_t": ctypes.c_int32,
        "float": ctypes.c_float,
    }
    for cname, mirror in (
        ("g4b_attn_args", native.AttnArgs),
        ("g4b_kv_append_args", native.KvAppendArgs),
        ("g4b_advance_args", native.AdvanceArgs),
        ("g4b_rope_args", native.RopeArgs),
    ):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), header, re.S).group(1)
        fields = []
        for line in body.splitlines():
            line = line.split("/*")[0].strip().rstrip(";")
            if not line:
                continue
            m = re.match(r"(?:const\s+)?([a-z0-9_]+\s*\*?)\s*(.*)", line)
            ctype = m.group(1).replace(" ", "")
            for decl in m.group(2).split(","):
                decl = decl.strip()
                arr = re.match(r"(\w+)\[(\d+)\]", decl)
                if arr:
                    fields.append((arr.group(1), ctype_of[ctype] * int(arr.group(2))))
                else:
                    fields.append((decl, ctype_of[ctype]))
        got = [(n, t) for n, t in mirror._fields_]
        assert [n for n, _ in got] == [n for n, _ in fields], cname
        for (n, t), (_, t2) in zip(got, fields):
            assert ctypes.sizeof(t) == ctypes.sizeof(t2), (cname, n)


def test_workspace_size_formula(native):
    lib = native.load()
    nw = lib.g4b_attn_default_workers()
    assert nw > 0
    # (workers + B*G) partial slots of rows x (D + 2) floats
    assert lib.g4b_attn_workspace_bytes(64, 8, 2, 1, 256, 0) == (nw + 128) * 4 * 258 * 4
    assert lib.g4b_attn_workspace_bytes(3, 8, 2, 2, 128, 10) == (10 + 6) * 8 * 130 * 4
    # prefill-shaped: (slot, key split) pairs x H x Tq rows x (D 16-bit values + 2 floats) when one slot brings fewer
    # than 256 workgroups (16 query tiles x 2 kv heads here -> 8 pairs), nothing when the shape fills the chip by itself
    assert lib.g4b_attn_workspace_bytes(1, 8, 2, 512, 256, 0) == 8 * 8 * 512 * (256 * 2 + 8)
    assert lib.g4b_attn_workspace_bytes(33, 8, 2, 512, 256, 0) == 8 * 8 * 512 * (256 * 2 + 8)  # independent of B
    assert lib.g4b_attn_workspace_bytes(1, 8, 2, 1024, 256, 0) == 4 * 8 * 1024 * (256 * 2 + 8)  # 32 tiles x 2 kv heads -> 4 pairs
    # from a third of the chip's units in query tiles on, the tiles are paired and the pairs cut into spans:
    # 2048 tokens are 32 pairs x 2 kv heads -> 4 spans each
    assert lib.g4b_attn_workspace_bytes(1, 8, 2, 2048, 256, 0) == 4 * 8 * 2048 * (256 * 2 + 8)
    assert lib.g4b_attn_workspace_bytes(1, 8, 2, 8192, 256, 0) == 0


def _decode_args():
    q = torch.zeros(2, 8, 1, 256, dtype=torch.float16)
    k = torch.zeros(2, 2, 64, 256, dtype=torch.float16)
    return q, k, k.clone(), q.clone(), torch.zeros(2, dtype=torch.int32), torch.zeros(2, dtype=torch.uint8)


def test_integration_stub_lists_the_argument_block_as_the_library_has_it(native):
    """The ctypes structure printed in the integration notes at the repository root is what a maintainer would paste:
    same fields, order and types as the structure this package binds (which the test above holds against the header)."""
    import re
    from pathlib import Path

    text = (Path(__file__).resolve().parent.parent / "INTEGRATION.md").read_text()
    body = text[text.index("class g4b_attn_args(C.Structure)"):text.index("lib.g4b_attn_forward.argtypes")]
    doc = []
    for name, ctype, length in re.findall(r'\("(\w+)", C\.(c_\w+)(?: \* (\d+))?\)', body):
        doc.append((name, getattr(ctypes, ctype), int(length or 0)))  # c_int32 and c_int are one type
    ours = [(name, getattr(ctype, "_type_", ctype) if hasattr(ctype, "_length_") else ctype, getattr(ctype, "_length_", 0))
            for name, ctype in native.AttnArgs._fields_]
    assert doc == ours


def test_python_boundary_validates_like_the_reference(native):
    from g4b_amd.kernels.fa2 import PHASE_DECODE, STAGE_CAUSAL, STAGE_FULL, STAGE_ON_BAND, flash_attention

    assert (STAGE_FULL, STAGE_ON_BAND, STAGE_CAUSAL) == (1, 2, 3)  # fa2.py:14-16
    q, k, v, o, tds, ph = _decode_args()
    with pytest.raises(ValueError, match="provided together"):  # fa2.py:656-657
        flash_attention(q, k, v, o, tds, ph, 64, PHASE_DECODE, torch.zeros(4, 2, 8, 1, 256))
    with pytest.raises(AssertionError):  # fa2.py:653
        flash_attention(q, k, v, o, tds, ph, 64, "decode")
    with pytest.raises(ValueError, match="ctx_window_size"):  # fa2.py:298
        flash_attention(q, k, v, o, tds, ph, 65, PHASE_DECODE)
    with pytest.raises(ValueError):  # fa2.py:296
        flash_attention(q[:, :7], k, v, o[:, :7], tds, ph, 64, PHASE_DECODE)
    with pytest.raises(ValueError, match="contiguous"):  # fa2.py:315-320
        flash_attention(q, k[:, :, ::2], v[:, :, ::2], o, tds, ph, 32, PHASE_DECODE)
    with pytest.raises(ValueError):
        flash_attention(q, k, v, o, tds.long(), ph, 64, PHASE_DECODE)
    with pytest.raises(ValueError, match="on_band_block"):  # the stage alone depends on the reference's tile size
        flash_attention(q, k, v, o, tds, ph, 64, PHASE_DECODE, stage=STAGE_ON_BAND)
    with pytest.raises(ValueError, match="on_band_block"):
        flash_attention(q, k, v, o, tds, ph, 64, PHASE_DECODE, stage=STAGE_ON_BAND, on_band_block=0)
    with pytest.raises(ValueError, match="stage"):
        flash_attention(q, k, v, o, tds, ph, 64, PHASE_DECODE, stage=4)
    q5, k5 = torch.zeros(2, 8, 1, 2048, dtype=torch.float16), torch.zeros(2, 2, 64, 2048, dtype=torch.float16)
    with pytest.raises(NotImplementedError, match="head_dim"):
        flash_attention(q5, k5, k5, q5.clone(), tds, ph, 64, PHASE_DECODE)


def test_c_abi_rejects_bad_arguments_before_launching(native):
    lib = native.load()
    assert lib.g4b_attn_forward(None, None) == native.G4B_ERR_INVALID_ARGUMENT
    assert "NULL" in native.last_error()
    a = native.AttnArgs()
    assert lib.g4b_attn_forward(ctypes.byref(a), None) == native.G4B_ERR_INVALID_ARGUMENT
    k = native.KvAppendArgs()
    assert lib.g4b_kv_append(ctypes.byref(k), None) == native.G4B_ERR_INVALID_ARGUMENT
    adv = native.AdvanceArgs()
    assert lib.g4b_advance_decode_state(ctypes.byref(adv), None) == native.G4B_ERR_INVALID_ARGUMENT
    # workspace too small is reported, not launched
    q, kk, v, o, tds, ph = _decode_args()
    from g4b_amd.kernels.fa2 import flash_attention

    with pytest.raises(ValueError, match="workspace"):
        flash_attention(q, kk, v, o, tds, ph, 64, 2, workspace=torch.zeros(64, dtype=torch.uint8))


def test_kv_append_and_advance_validation(native):
    from g4b_amd.kernels.add_kv_to_cache import add_kv_to_cache
    from g4b_amd.kernels.advance_decode_state import advance_decode_state

    x = torch.zeros(2, 4, 7, 256)
    cache = torch.zeros(2, 4, 17, 256, dtype=torch.float16)
    offs = torch.tensor([15, 3])
    with pytest.raises(AssertionError):  # add_kv_to_cache.py:171
        add_kv_to_cache(x, cache, offs, 1e-6, phase=1.0)
    with pytest.raises(ValueError):  # add_kv_to_cache.py:119
        add_kv_to_cache(torch.zeros(2, 4, 18, 256), cache, offs, 1e-6)
    with pytest.raises(ValueError):  # add_kv_to_cache.py:105-107
        add_kv_to_cache(x, cache[:, :2], offs, 1e-6)
    with pytest.raises(ValueError):
        add_kv_to_cache(x, cache, offs, 1e-6, x_rsos=torch.zeros(2, 4, 6))
    with pytest.raises(ValueError):  # advance_decode_state.py:45-50
        advance_decode_state(
            torch.zeros(1, 3, dtype=torch.int32),
            torch.zeros(4, 1, dtype=torch.int32),
            torch.zeros(3, dtype=torch.int32),
            torch.zeros(3, dtype=torch.int32),
            torch.zeros(3, dtype=torch.uint8),
        )


def test_tensor_protocol_accepts_g4b_style_tensors(native):
    """Objects with shape / stride sequence / dtype.name / data_ptr() (g4b/tensor.py:71-80) are accepted."""
    from g4b_amd.kernels import utils as U

    class DT:
        def __init__(self, name):
            self.name = name

    class T:
        def __init__(self, t, name):
            self._t, self.shape, self.stride, self.dtype = t, list(t.shape), list(t.stride()), DT(name)

        def data_ptr(self):
            return self._t.data_ptr()

    t = torch.zeros(2, 3, 4, 8, dtype=torch.float16).permute(0, 2, 1, 3)
    w = T(t, "float16")
    assert U.strides_of(w) == list(t.stride()) == U.strides_of(t)
    assert U.float_dtype_code(w, "w") == U.float_dtype_code(t, "t") == native.DT_F16
    assert U.dtype_name(torch.zeros(1, dtype=torch.int32)) == "int32"


def test_plan_validates_at_bind_time(native):
    from g4b_amd.kernels.fa2 import PHASE_DECODE, plan_flash_attention

    q, k, v, o, tds, ph = _decode_args()
    plan = plan_flash_attention(q, k, v, o, tds, ph, 64, PHASE_DECODE, scale=0.5)
    assert plan._args.B == 2 and plan._args.H == 8 and plan._args.KV_CTX == 64 and plan._args.scale == 0.5
    with pytest.raises(ValueError):  # shape checks run when the plan is made (fa2.py:296)
        plan_flash_attention(q[:, :7], k, v, o, tds, ph, 64, PHASE_DECODE)
    bad = plan_flash_attention(q, k, v, o, tds, ph, 65, PHASE_DECODE)
    with pytest.raises(ValueError, match="ctx_window_size"):  # value checks live in the library (fa2.py:298)
        bad.launch(stream=0)


def test_pipelined_kernels_keep_foreign_memory_traffic_out_of_their_wait_regions():
    """The prefill kernels retire LDS reads with hand-counted lgkmcnt waits and direct-to-LDS loads with one vmcnt(0)
    per tile; a compiler-made scalar, LDS, global or scratch access between the first and the last MFMA would break
    the counts (a spill is enough).  The build module scans the generated assembly."""
    from g4b_amd.build import check_wait_discipline

    seen = check_wait_discipline()
    # head dims 128, 256 and 512, fp16 and bf16 caches, each with the query rounded or split into two operands
    assert len(seen) == 20, seen
    assert all(n >= 48 for n in seen.values()), seen


def test_decode_stream_keeps_its_non_temporal_loads():
    """K and V of a decode launch are read once, with `global_load_dwordx4 ... nt`; the marking is optimiser metadata
    (merging such a load with an ordinary one drops it without a word), so the generated assembly is scanned."""
    from g4b_amd.build import check_stream_loads

    seen = check_stream_loads()
    # worker: head dims 128 / 256 / 512 x three row classes x fp16 / bf16 x query rounded or split; pair: 128 / 256
    assert len(seen) == 36 + 24, sorted(seen)


def test_mixed_launch_is_validated_before_launching(native):
    """g4b_attn_forward_mixed checks both argument blocks and their agreement on the host (no GPU needed)."""
    from g4b_amd.kernels.fa2 import PHASE_DECODE, PHASE_PREFILL, flash_attention, mixed_workspace_bytes

    lib = native.load()
    assert lib.g4b_attn_forward_mixed(None, None, None) == native.G4B_ERR_INVALID_ARGUMENT
    B, H, G, D, T, t = 2, 8, 2, 256, 600, 64
    qp, qd = torch.zeros(B, H, t, D, dtype=torch.float16), torch.zeros(B, H, 1, D, dtype=torch.float16)
    k = torch.zeros(B, G, T, D, dtype=torch.float16)
    tds, ph = torch.zeros(B, dtype=torch.int32), torch.zeros(B, dtype=torch.uint8)
    with pytest.raises(ValueError, match="go together"):
        flash_attention(qp, k, k, qp.clone(), tds, ph, T, PHASE_PREFILL, decode_q=qd)
    with pytest.raises(ValueError, match="different phases"):
        flash_attention(qp, k, k, qp.clone(), tds, ph, T, PHASE_DECODE, decode_q=qd, decode_o=qd.clone())
    with pytest.raises(ValueError, match="prefill-shaped"):
        flash_attention(qd, k, k, qd.clone(), tds, ph, T, PHASE_PREFILL, decode_q=qd, decode_o=qd.clone())
    with pytest.raises(ValueError, match="partial_o"):
        flash_attention(qp, k, k, qp.clone(), tds, ph, T, PHASE_PREFILL, torch.zeros(4, B, H, t, D), torch.zeros(4, B, H, t),
                        torch.zeros(4, B, H, t), decode_q=qd, decode_o=qd.clone())
    with pytest.raises(ValueError, match="workspace holds"):
        flash_attention(qp, k, k, qp.clone(), tds, ph, T, PHASE_PREFILL, decode_q=qd, decode_o=qd.clone(),
                        workspace=torch.zeros(64, dtype=torch.uint8))
    q128, k128 = torch.zeros(B, H, t, 128, dtype=torch.float16), torch.zeros(B, G, T, 128, dtype=torch.float16)
    with pytest.raises(NotImplementedError, match="head_dim"):
        flash_attention(q128, k128, k128, q128.clone(), tds, ph, T, PHASE_PREFILL, decode_q=torch.zeros(B, H, 1, 128, dtype=torch.float16),
                        decode_o=torch.zeros(B, H, 1, 128, dtype=torch.float16))
    # sizing: the chunk's partials ((slot, split) pairs x H x t x (D 16-bit values + 2 floats), rounded up to 256 bytes) followed by the
    # decode partials ((workers + B*G) x rows x (D + 2) floats).  64-token chunks bring 2 tiles x 2 kv heads = 4 workgroups
    # per slot; the default share-out leaves 256 - 112 = 144 units to the chunk -> 36 pairs, and the decode half gets the
    # remaining 112 workgroups of four workers.
    n = mixed_workspace_bytes(B, H, G, t, 1, D, T, T)
    assert n == 36 * H * t * (D * 2 + 8) + (448 + B * G) * 4 * (D + 2) * 4
    # a short window takes the one-workgroup-per-pair decode path: no decode partials, 256 - B*G units for the chunk
    n_swa = mixed_workspace_bytes(B, H, G, t, 1, D, 512 + t - 1, 512)
    assert n_swa == 63 * H * t * (D * 2 + 8)
    assert mixed_workspace_bytes(B, H, G, t, 1, D, 512 + t - 1, 512, True) == n  # per-slot windows: streaming workers again


def test_static_scratch_entry_point_checks_its_arguments(native):
    lib = native.load()
    assert lib.g4b_static_scratch_bytes() == 68 << 20
    assert lib.g4b_attn_forward_static_scratch(None, None) == native.G4B_ERR_INVALID_ARGUMENT
    a = native.AttnArgs()
    a.workspace = 4096
    assert lib.g4b_attn_forward_static_scratch(ctypes.byref(a), None) == native.G4B_ERR_INVALID_ARGUMENT
    assert "workspace must be NULL" in native.last_error()


def test_c_abi_rejects_a_tile_count_beyond_32_bits(native):
    """The streaming kernels count the 32-key tiles of all (slot, kv head) pairs in 32 bits; the host refuses what
    could overflow that before anything is launched (the pointers are never dereferenced on the host)."""
    lib = native.load()
    a = native.AttnArgs()
    for name in ("q", "k_cache", "v_cache", "o", "time_dim_sizes", "user_phase"):
        setattr(a, name, 256)
    a.B, a.H, a.G, a.Tq, a.D, a.KV_CTX = 60000, 40000, 40000, 1, 8, 1 << 20
    a.ctx_window_size, a.phase, a.stage, a.scale = 1 << 20, 2, 3, 1.0
    a.q_stride = (ctypes.c_int64 * 4)(8, 8, 8, 1)
    a.o_stride = (ctypes.c_int64 * 4)(8, 8, 8, 1)
    a.k_stride_b = a.v_stride_b = 40000 * (1 << 20) * 8
    a.time_dim_sizes_stride = a.user_phase_stride = 1
    assert lib.g4b_attn_forward(ctypes.byref(a), None) == native.G4B_ERR_UNSUPPORTED
    assert "2^31" in native.last_error()
    a.B, a.G, a.H = 4, 2, 8
    a.k_stride_b = a.v_stride_b = 2 * (1 << 20) * 8
    a.q_dtype = 7  # the next check in line fails instead: the tile count passed
    assert lib.g4b_attn_forward(ctypes.byref(a), None) == native.G4B_ERR_INVALID_ARGUMENT


def test_limit_kv_splits_turns_the_partials_leading_dimension_into_a_bound(native):
    """The reference's MAX_KV_SPLITS (fa2.py:658) does not bound the split by default; with limit_kv_splits=True a
    decode launch gets at most that many workers per (slot, kv head)."""
    from g4b_amd.kernels import fa2

    q, k, v, o, tds, ph = _decode_args()
    parts = (torch.zeros(4, 2, 8, 1, 256, dtype=torch.float16), torch.zeros(4, 2, 8, 1), torch.zeros(5, 2, 8, 1))
    a, _, _ = fa2._bind(q, k, v, o, tds, ph, 64, 2, *parts, workspace=False)
    assert a.num_workers == 0
    a, _, _ = fa2._bind(q, k, v, o, tds, ph, 64, 2, *parts, workspace=False, limit_kv_splits=True)
    assert a.num_workers == 2 * 2 * 4  # B * G * min of the leading dimensions
    a, _, _ = fa2._bind(q, k, v, o, tds, ph, 64, 2, *parts, workspace=False, limit_kv_splits=True, num_workers=7)
    assert a.num_workers == 7
    a, _, _ = fa2._bind(q, k, v, o, tds, ph, 64, 2, workspace=False, limit_kv_splits=True)  # no partials: no bound
    assert a.num_workers == 0
