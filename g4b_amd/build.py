"""Build libg4b_attn.so (HIP kernels for gfx950 + the C ABI) in-tree with hipcc.

    python -m g4b_amd.build            # compile every translation unit, link
    python -m g4b_amd.build --verbose  # also print the per-kernel register / LDS usage remarks
    python -m g4b_amd.build --check-waits  # also verify that nothing foreign sits in the hand-counted wait regions
    python -m g4b_amd.build --asan     # host code of the C ABI under AddressSanitizer + UBSan (no GPU needed), and run it

The shared library lands next to this file so that it travels with the source tree; nothing
is installed.  hipcc cross-compiles for gfx950 without a GPU present.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
BUILD_DIR = PKG_DIR / "build"
LIB_PATH = PKG_DIR / "libg4b_attn.so"
ARCH = "gfx950"

SOURCES = ["api.hip", "attn_decode.hip", "attn_prefill.hip", "attn_prefill_wide.hip", "attn_mixed_f16.hip",
           "attn_mixed_bf16.hip", "attn_mixed_d512_f16.hip", "attn_mixed_d512_bf16.hip", "attn_generic.hip", "cache_ops.hip",
           "rope.hip"]

# packed-fp32 VALU forms are kept off: the compiler must not form v_pk_{add,mul,fma}_f32
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fno-honor-nans", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-variable", "-Wno-unknown-pragmas",
                "-Wno-inline-asm"]  # the M0 clobber of dma_set_base is deliberate


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build g4b_amd")
    return exe


def _compile(src: str, verbose: bool) -> Path:
    obj = BUILD_DIR / (src + ".o")
    cmd = [hipcc(), *COMMON_FLAGS, *DEVICE_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    if verbose:
        cmd.insert(1, "-Rpass-analysis=kernel-resource-usage")
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = False, jobs: int | None = None) -> Path:
    BUILD_DIR.mkdir(exist_ok=True)
    jobs = jobs or min(len(SOURCES), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


# Kernels whose LDS operand reads are retired with hand-counted `s_waitcnt lgkmcnt(n)` and whose direct-to-LDS loads
# are waited for with one `s_waitcnt vmcnt(0)` per tile.  The counts are only exact while the compiler keeps its own
# memory traffic out of the region between the first and the last MFMA: a scalar load or a compiler-made LDS access
# there shares lgkmcnt (and scalar loads return out of order), a global or scratch access brings a vmcnt(0) that also
# waits for the direct loads in flight.
PIPELINED_SOURCES = {"attn_prefill.hip": "attn_prefill_kernel", "attn_prefill_wide.hip": "attn_prefill_wide_kernel"}


def check_wait_discipline() -> dict:
    """Compile the pipelined kernels to assembly and scan the MFMA region of each instantiation.

    Returns {kernel symbol: number of MFMAs}; raises RuntimeError naming the first foreign memory instruction."""
    import re
    import tempfile

    foreign = re.compile(r"\b(s_load|s_buffer_load|scratch_|global_load_dword|global_store|buffer_|flat_|ds_)")
    allowed = ("ds_read_b128", "ds_read_b64_tr_b16", "global_load_lds_dwordx4")
    seen = {}
    with tempfile.TemporaryDirectory() as tmp:
        for src, stem in PIPELINED_SOURCES.items():
            out = Path(tmp) / (src + ".s")
            cmd = [hipcc(), *COMMON_FLAGS, *DEVICE_FLAGS, "-S", "--cuda-device-only", str(CSRC / src), "-o", str(out)]
            res = subprocess.run(cmd, capture_output=True, text=True)
            if res.returncode != 0:
                raise RuntimeError(f"hipcc -S failed on {src}:\n{res.stderr}")
            lines = out.read_text().splitlines()
            i = 0
            while i < len(lines):
                m = re.match(r"(_ZN3g4b\d+%s\w*):" % stem, lines[i])
                if not m:
                    i += 1
                    continue
                end = next(j for j in range(i, len(lines)) if lines[j].startswith(".Lfunc_end"))
                body = lines[i:end]
                mfma = [j for j, l in enumerate(body) if "v_mfma" in l]
                # A foreign access is harmless only if its counter is drained again before the next MFMA (the epilogue
                # of a workgroup's first query tile and the set-up of its second sit between two MFMAs).  Every
                # hand-counted wait stands directly in front of the MFMA that consumes what it waited for, so a wait
                # that counted next to a foreign access is caught at that MFMA; a wait whose MFMA comes only after the
                # drain has, by then, everything it counted on.  (The epilogue's own LDS traffic and the waits the
                # compiler counts for it use the same mnemonics as the operand reads and cannot be told apart here.)
                # A flat access holds a slot of both counters until it has completed, i.e. until vmcnt(0).
                dirty_lgkm = dirty_vm = None
                for l in body[mfma[0] : mfma[-1] + 1]:
                    ins = l.strip()
                    if "v_mfma" in ins:
                        if dirty_lgkm or dirty_vm:
                            raise RuntimeError(f"{m.group(1)}: `{dirty_lgkm or dirty_vm}` inside the hand-counted wait region")
                    elif ins.startswith("s_waitcnt"):
                        if "lgkmcnt(0)" in ins and not (dirty_lgkm or "").startswith("flat_"):
                            dirty_lgkm = None
                        if "vmcnt(0)" in ins:
                            dirty_vm = None
                            if (dirty_lgkm or "").startswith("flat_"):
                                dirty_lgkm = None
                    elif foreign.search(ins) and not ins.startswith(allowed):
                        if ins.startswith(("s_load", "s_buffer_load", "ds_", "flat_")):
                            dirty_lgkm = ins
                        if not ins.startswith(("s_load", "s_buffer_load", "ds_")):
                            dirty_vm = ins
                # M0 carries the LDS destination of the direct loads from one dma_set_base (`s_mov_b32 m0` + `s_nop 0`,
                # one asm block) to the loads that follow it: any other write to M0 in the kernel would misplace a tile.
                code = [l.strip() for l in body if l.strip() and not l.strip().startswith((";", ".", "//"))]
                for j, ins in enumerate(code):
                    ops = ins.split(None, 1)
                    writes_m0 = len(ops) == 2 and ops[0].startswith(("s_", "v_readlane", "v_readfirstlane")) and \
                        re.match(r"m0\b", ops[1]) is not None
                    if writes_m0 and not (ops[0] == "s_mov_b32" and j + 1 < len(code) and code[j + 1].startswith("s_nop 0")):
                        raise RuntimeError(f"{m.group(1)}: `{ins}` writes M0 outside dma_set_base")
                    if ops[0].startswith(("s_movrel", "v_movrel")):
                        raise RuntimeError(f"{m.group(1)}: `{ins}` uses M0 as an index next to the direct loads")
                seen[m.group(1)] = len(mfma)
                i = end
    return seen


def check_stream_loads() -> dict:
    """The decode kernels read K and V with non-temporal loads (a fifth of their throughput hangs on it) and q with
    ordinary ones.  The marking is metadata the optimiser may drop when it merges loads, so the generated assembly is
    checked: every worker / pair instantiation must carry `global_load_dwordx4 ... nt` for its stream.

    Returns {kernel symbol: (non-temporal 16-byte loads, ordinary 16-byte loads)}."""
    import re
    import tempfile

    seen = {}
    with tempfile.TemporaryDirectory() as tmp:
        out = Path(tmp) / "attn_decode.s"
        cmd = [hipcc(), *COMMON_FLAGS, *DEVICE_FLAGS, "-S", "--cuda-device-only", str(CSRC / "attn_decode.hip"), "-o", str(out)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc -S failed on attn_decode.hip:\n{res.stderr}")
        cur = None
        for line in out.read_text().splitlines():
            m = re.match(r"(_ZN3g4b\d+attn_decode_(?:worker|pair)\w*):", line)
            if m:
                cur = m.group(1)
                seen[cur] = [0, 0]
            elif line.startswith(".Lfunc_end"):
                cur = None
            elif cur and "global_load_dwordx4" in line:
                seen[cur][0 if re.search(r"\bnt\b", line) else 1] += 1
    if not seen:
        raise RuntimeError("no decode kernel found in the assembly of attn_decode.hip")
    for sym, (nt, plain) in seen.items():
        if nt < 24 or nt <= plain:
            raise RuntimeError(f"{sym}: {nt} non-temporal and {plain} ordinary 16-byte loads; the K/V stream lost its nt marking")
    return {k: tuple(v) for k, v in seen.items()}


# The host pass under AddressSanitizer and UndefinedBehaviorSanitizer (GPU sanitizers are not available here): the C ABI's
# entry points and their validation (api.hip) linked with tests/host_api_check.hip, whose stand-in launchers abort, and
# the share-out arithmetic of tests/tile_shares_check.hip.  Returns the two executables; they need no GPU.
SANITIZE = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host", "-fno-sanitize-recover=undefined",
            "-Xarch_host", "-fno-omit-frame-pointer", "-g"]


def build_asan() -> list[Path]:
    out_dir = BUILD_DIR / "asan"
    out_dir.mkdir(parents=True, exist_ok=True)
    tests = PKG_DIR.parent / "tests"
    flags = ["-O1", "-std=c++17", "-fPIE", f"--offload-arch={ARCH}", "-Wno-inline-asm", "-Wno-unknown-pragmas", *DEVICE_FLAGS, *SANITIZE]

    def run(cmd):
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"{' '.join(map(str, cmd[:3]))} ... failed:\n{res.stderr[-3000:]}")

    api_check = out_dir / "host_api_check"
    run([hipcc(), *flags, "-I", str(CSRC), str(CSRC / "api.hip"), str(tests / "host_api_check.hip"), "-o", str(api_check)])
    shares_check = out_dir / "tile_shares_check"
    run([hipcc(), *flags, "-I", str(CSRC), str(tests / "tile_shares_check.hip"), "-o", str(shares_check)])
    return [api_check, shares_check]


if __name__ == "__main__":
    if "--asan" in sys.argv:
        for exe in build_asan():
            res = subprocess.run([str(exe)], capture_output=True, text=True, env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
            print(f"{exe.name}: exit {res.returncode}: {(res.stdout.strip().splitlines() or [''])[-1]}")
            if res.returncode:
                print(res.stderr[-3000:], file=sys.stderr)
                sys.exit(1)
        sys.exit(0)
    path = build(verbose="--verbose" in sys.argv)
    print(path)
    if "--check-waits" in sys.argv:
        for sym, n in check_wait_discipline().items():
            print(f"wait discipline ok: {sym} ({n} MFMAs)")
        for sym, (nt, plain) in check_stream_loads().items():
            print(f"stream loads ok: {sym} ({nt} non-temporal, {plain} ordinary)")
