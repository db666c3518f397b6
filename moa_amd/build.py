"""Builds moa_amd/libmoa_hip.so from moa_amd/csrc/*.hip with hipcc for gfx950.

    python -m moa_amd.build            # build if sources are newer than the library
    python -m moa_amd.build --force    # always rebuild
    python -m moa_amd.build --experiment -DNAME ...   # rebuild with extra hipcc flags (measurements only)

hipcc cross-compiles without a GPU.  The library is kept in-tree next to this
file so that it travels with the source tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from typing import Sequence

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "csrc", "build")
LIB_PATH = os.path.join(HERE, "libmoa_hip.so")

SOURCES = ["moa_capi.hip", "moa_cache.hip", "moa_decode.hip", "moa_prefill.hip", "moa_rope.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # no kernel relies on NaN propagation (masks use -inf): lets fmax compile to one instruction
    "-fno-honor-nans",
    # packed-FP32 instructions are switched off for all device code of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# moa_rope.hip reproduces torch's per-operation rounding bit for bit: no multiply-add contraction there
PER_SOURCE_FLAGS = {"moa_rope.hip": ["-ffp-contract=off"]}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _deps_mtime() -> float:
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h"))]
    paths.append(os.path.join(HERE, "..", "include", "moa_hip.h"))
    return max(os.path.getmtime(p) for p in paths if os.path.exists(p))


def is_stale() -> bool:
    return (not os.path.exists(LIB_PATH)) or os.path.getmtime(LIB_PATH) < _deps_mtime()


def _compile(src: str, extra: Sequence[str] = ()) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_SOURCE_FLAGS.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    noise = "is not a recognized feature for this target"
    warn = "\n".join(l for l in r.stderr.splitlines() if noise not in l).strip()
    if warn:
        sys.stderr.write(f"[moa_amd.build] {src}:\n{warn}\n")
    return obj


def build(force: bool = False, verbose: bool = True, experiment_flags: Sequence[str] = ()) -> str:
    """Compiles every source and links the library.  ``experiment_flags`` (extra hipcc arguments) are for
    measurement builds only and must be asked for explicitly: the environment never changes the build."""
    if not force and not experiment_flags and not is_stale():
        return LIB_PATH
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    missing = set(SOURCES) - set(srcs)
    if missing:
        raise RuntimeError(f"missing sources: {sorted(missing)}")
    with ThreadPoolExecutor(max_workers=min(4, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, experiment_flags), srcs))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"[moa_amd.build] built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    argv = sys.argv[1:]
    flags = argv[argv.index("--experiment") + 1:] if "--experiment" in argv else []
    build(force="--force" in argv or bool(flags), experiment_flags=flags)
