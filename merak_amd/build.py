"""Build the gfx950 kernel library (``merak_amd/lib/libmerak_tp_gfx950.so``).

Plain hipcc, one object per source file, compiled in parallel and linked into
one shared library that exports the C ABI declared in
``include/merak_tp_gfx950.h``.  The library is built in-tree so that it
travels with the source tree; nothing is installed.

    python -m merak_amd.build            # build (always recompiles)
    python -m merak_amd.build --measure  # the same sources with -DMTP_MEASURE into libmerak_tp_gfx950_measure.so:
                                         # kernels with their measurement switches (MTP_GEMM_DEBUG: parts of the
                                         # product switched off, results wrong); point MERAK_AMD_LIB at it
    python -m merak_amd.build --registers gemm_bf16_fwd.hip [...]
                                         # compile the named sources and print registers, scratch, LDS and
                                         # occupancy of every kernel in them (the compiler's own resource remarks)
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
    "gemm_bf16_bwd.hip",
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


# Per-source additions.  gemv.hip: MFMA accumulators in arch VGPRs.  Its single-set loop pins the instruction order;
# with accumulators in the other register file the compiler copies them back and forth around every pinned section
# and the largest configuration loses half its occupancy (314 registers instead of 254).
SOURCE_FLAGS = {
    "gemv.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the gfx950 kernel library cannot be built")
    return exe


def _compile(src: Path, obj: Path, extra: list[str]) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, *SOURCE_FLAGS.get(src.name, []), *extra, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops' is not a recognized feature"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = True, jobs: int | None = None, extra_flags: list[str] | None = None,
          lib_path: Path | None = None) -> Path:
    """Compile every kernel source for gfx950 and link the shared library."""
    LIB_DIR.mkdir(exist_ok=True)
    extra = list(extra_flags or [])
    out_path = Path(lib_path) if lib_path else LIB_PATH
    jobs = jobs or min(8, len(SOURCES), os.cpu_count() or 1)
    tag = "" if out_path == LIB_PATH else "." + out_path.stem
    objs = [LIB_DIR / (Path(s).stem + tag + ".o") for s in SOURCES]
    if verbose:
        print(f"[merak_amd.build] hipcc x{jobs}: {', '.join(SOURCES)}", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _compile(CSRC / so[0], so[1], extra), zip(SOURCES, objs)))
    tmp = out_path.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(tmp), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, out_path)
    if verbose:
        print(f"[merak_amd.build] wrote {out_path}", flush=True)
    return out_path


def kernel_registers(sources: list[str]) -> list[dict]:
    """Compile `sources` (names under csrc/) with -Rpass-analysis=kernel-resource-usage and return, per kernel,
    what the compiler reports: arch and accumulator VGPRs, SGPRs, scratch bytes per lane, LDS bytes, occupancy."""
    import re
    import tempfile
    rows = []
    for name in sources:
        with tempfile.TemporaryDirectory() as td:
            cmd = [_hipcc(), *HIPCC_FLAGS, *SOURCE_FLAGS.get(name, []), "-Rpass-analysis=kernel-resource-usage", "-c",
                   str(CSRC / name), "-o",
                   os.path.join(td, "o.o")]
            r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {name}:\n{r.stderr[-2000:]}")
        cur = None
        for line in r.stderr.splitlines():
            m = re.search(r"remark:\s+([A-Za-z \[\]/]+): (.*?) \[-Rpass-analysis", line)
            if not m:
                continue
            key, val = m.group(1).strip(), m.group(2)
            if key == "Function Name":
                filt = subprocess.run(["c++filt", val], capture_output=True, text=True).stdout.strip() or val
                filt = filt.replace("(anonymous namespace)::", "").replace("void ", "").split("(")[0]
                cur = {"source": name, "kernel": filt}
                rows.append(cur)
            elif cur is not None:
                cur[key] = val
    return rows


def _print_registers(sources: list[str]) -> None:
    for r in kernel_registers(sources):
        print(f"{r['kernel']:62s} vgpr={r.get('VGPRs', '?'):>3s} agpr={r.get('AGPRs', '?'):>3s} "
              f"sgpr={r.get('TotalSGPRs', '?'):>3s} scratch={r.get('ScratchSize [bytes/lane]', '?'):>3s} "
              f"lds={r.get('LDS Size [bytes/block]', '?'):>6s} occupancy={r.get('Occupancy [waves/SIMD]', '?')}")


if __name__ == "__main__":
    if "--registers" in sys.argv:
        _print_registers(sys.argv[sys.argv.index("--registers") + 1:])
    elif "--measure" in sys.argv:
        build(extra_flags=["-DMTP_MEASURE"], lib_path=LIB_DIR / "libmerak_tp_gfx950_measure.so")
    else:
        build()
