"""Build the gfx950 kernel library (``merak_amd/lib/libmerak_tp_gfx950.so``).

Plain hipcc, one object per source file, compiled in parallel and linked into
one shared library that exports the C ABI declared in
``include/merak_tp_gfx950.h``.  The library is built in-tree so that it
travels with the source tree; nothing is installed.

    python -m merak_amd.build            # build (always recompiles)
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
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libmerak_tp_gfx950.so"

SOURCES = [
    "api.hip",
    "vocab_ce.hip",
    "embedding.hip",
    "gemv.hip",
    "elementwise.hip", "sampling.hip",
    "gemm_bf16_fwd.hip", "gemm_f16_fwd.hip",
    "gemm_bf16_dgrad.hip",
    "gemm_bf16_wgrad.hip",
    "gemm_generic.hip", "gemm_f32.hip", "decode_attn.hip",
    "linear.hip",
]

# -packed-fp32-ops off: packed fp32 VALU forms are not to be generated for this target pool.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the gfx950 kernel library cannot be built")
    return exe


def _compile(src: Path, obj: Path, extra: list[str]) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops' is not a recognized feature"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = True, jobs: int | None = None, extra_flags: list[str] | None = None) -> Path:
    """Compile every kernel source for gfx950 and link the shared library."""
    LIB_DIR.mkdir(exist_ok=True)
    extra = list(extra_flags or [])
    jobs = jobs or min(8, len(SOURCES), os.cpu_count() or 1)
    objs = [LIB_DIR / (Path(s).stem + ".o") for s in SOURCES]
    if verbose:
        print(f"[merak_amd.build] hipcc x{jobs}: {', '.join(SOURCES)}", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _compile(CSRC / so[0], so[1], extra), zip(SOURCES, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(tmp), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[merak_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
