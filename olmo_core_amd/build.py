"""
Build recipe for libmi8.so (the float8 linear path) and libmi8_diag.so (measurement kernels used by bench.py only):
plain ``hipcc`` for gfx950, no torch headers (the libraries have a C ABI).

    python -m olmo_core_amd.build            # compile if sources are newer than the library
    python -m olmo_core_amd.build --force    # always compile
"""

from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "lib" / "libmi8.so"
DIAG_LIB_PATH = PKG_DIR / "lib" / "libmi8_diag.so"
OBJ_DIR = PKG_DIR / "lib" / "obj"

SOURCES = ["mi8_api.hip", "mi8_cast.hip", "mi8_gemm.hip", "mi8_gemm_m16.hip", "mi8_gemm_skinny.hip", "mi8_pointwise.hip", "mi8_swiglu_amax.hip", "mi8_grouped.hip", "mi8_permute.hip"]
# the diagnostics library: the probe kernels plus the error-text / launch helpers they share with the main library
DIAG_SOURCES = ["mi8_api.hip", "mi8_probe.hip"]
# ... and the persistent GEMM once more, compiled with time stamps at fixed points of every tile (object name, source, flag)
DIAG_EXTRA = [("mi8_gemm_m16_timeline", "mi8_gemm_m16.hip", "-DMI8_TILE_TIMELINE")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    # hipcc must not form packed-fp32 instructions on its own
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; libmi8.so cannot be built on this machine")
    return exe


def sources() -> list[Path]:
    names = SOURCES + [s for s in DIAG_SOURCES if s not in SOURCES]
    return [CSRC / s for s in names if (CSRC / s).exists()]


def is_stale() -> bool:
    if not LIB_PATH.exists() or not DIAG_LIB_PATH.exists():
        return True
    built = min(LIB_PATH.stat().st_mtime, DIAG_LIB_PATH.stat().st_mtime)
    deps = list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h")) + list((PKG_DIR.parent / "include").glob("*.h"))
    return any(d.stat().st_mtime > built for d in deps)


def build(force: bool = True, verbose: bool = False) -> Path:
    if not force and not is_stale():
        return LIB_PATH
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    cc = hipcc()

    def compile_one(job) -> Path:
        stem, src, extra = job
        obj = OBJ_DIR / (stem + ".o")
        cmd = [cc, *HIPCC_FLAGS, *extra, "-c", str(src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {Path(src).name}:\n{res.stdout}\n{res.stderr}")
        noise = "unknown target feature"  # host pass does not know the device-only feature flag
        warn = "\n".join(line for line in res.stderr.splitlines() if line.strip() and noise not in line and "-packed-fp32-ops" not in line)
        if warn and verbose:
            print(warn, file=sys.stderr)
        return obj

    work = [(src.stem, src, []) for src in sources()] + [(stem, CSRC / name, [flag]) for stem, name, flag in DIAG_EXTRA]
    jobs = min(len(work), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=max(jobs, 1)) as pool:
        objs = {o.stem: o for o in pool.map(compile_one, work)}
    diag_names = DIAG_SOURCES + [stem for stem, _, _ in DIAG_EXTRA]
    # (-Bsymbolic: the diagnostics library binds its own copies of the helpers it shares with libmi8.so)
    for target, names, link_flags in ((LIB_PATH, SOURCES, []), (DIAG_LIB_PATH, diag_names, ["-Wl,-Bsymbolic"])):
        tmp = target.with_suffix(".so.tmp")
        cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", *link_flags, "-o", str(tmp), *(str(objs[Path(n).stem]) for n in names)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link of {target.name} failed:\n{res.stdout}\n{res.stderr}")
        os.replace(tmp, target)
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-v", "--verbose", action="store_true")
    ns = ap.parse_args()
    print(build(force=ns.force or is_stale(), verbose=ns.verbose))
