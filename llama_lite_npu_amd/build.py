"""Builds liblitekv.so (HIP, gfx950) in-tree with hipcc.

Usage: ``python -m llama_lite_npu_amd.build`` or ``build_library(force=True)``.
hipcc cross-compiles for gfx950 without a GPU, so this also runs on a CPU-only
machine. The library lands next to its sources (``csrc/liblitekv.so``); nothing
is installed outside the tree.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_PATH = CSRC / "liblitekv.so"
OBJ_DIR = CSRC / "build"

SOURCES = (
    "status.hip",
    "kv_append.hip",
    "kv_fp8.hip",
    "qk_rope_append.hip",
    "page_ops.hip",
    "paged_decode.hip",
    "paged_decode_hd64.hip",
    "decode_advance.hip",
    "paged_prefill.hip",
    "paged_prefill_hd64.hip",
    "generic_attention.hip",
)

# Packed fp32 VALU forms are switched off for device code: the compiler would
# otherwise form them on its own from scalar float arithmetic.
HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)


# Extra flags per source. The prefill kernel takes maxima of MFMA results: without NaN
# semantics to honour, the compiler drops the self-max that quiets each operand and fuses the
# rest into v_max3_f32. Nothing in that file relies on NaN propagation (masking uses -inf).
# Its direct HBM -> LDS loads set m0 in inline assembly and list it as clobbered; the compiler
# remarks on every such statement that m0 is a reserved register, which is the point of listing it.
PER_FILE_FLAGS = {
    "paged_prefill.hip": ("-fno-honor-nans", "-Wno-inline-asm"),
    "paged_prefill_hd64.hip": ("-fno-honor-nans", "-Wno-inline-asm"),
    # the decode step behind a shared prefix runs the same tile kernel as one role of its launch
    "paged_decode.hip": ("-Wno-inline-asm",),
    "paged_decode_hd64.hip": ("-Wno-inline-asm",),
}


def _hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; liblitekv needs the ROCm toolchain to build")
    return found


def _headers() -> list[Path]:
    return sorted(CSRC.glob("*.h")) + sorted(CSRC.glob("*.inc")) + sorted((CSRC.parents[1] / "include").glob("*.h"))


def is_stale() -> bool:
    if not LIB_PATH.exists():
        return True
    built = LIB_PATH.stat().st_mtime
    deps = [CSRC / s for s in SOURCES] + _headers()
    return any(d.stat().st_mtime > built for d in deps)


def _compile(hipcc: str, src: Path, obj: Path, extra: tuple[str, ...]) -> None:
    cmd = [hipcc, *HIPCC_FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature"
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{log}")
    if log.strip():
        print(log, file=sys.stderr)


def build_library(force: bool = False, extra_flags: tuple[str, ...] = ()) -> Path:
    """Compiles every source and links liblitekv.so; returns its path."""
    if not force and not is_stale():
        return LIB_PATH
    hipcc = _hipcc()
    OBJ_DIR.mkdir(exist_ok=True)
    objs = [OBJ_DIR / (Path(s).stem + ".o") for s in SOURCES]
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as pool:
        jobs = [
            pool.submit(_compile, hipcc, CSRC / s, o, PER_FILE_FLAGS.get(s, ()) + tuple(extra_flags))
            for s, o in zip(SOURCES, objs)
        ]
        for j in jobs:
            j.result()
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link of liblitekv.so failed:\n{proc.stdout}{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True))
