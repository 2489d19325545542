"""Builds liblce_gfx950.so from csrc/ with hipcc (cross-compiles without a GPU).

Usage: ``python -m linear_cross_entropy_loss_amd.build [--force]``
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_NAME = "liblce_gfx950.so"
LIB_PATH = PKG_DIR / LIB_NAME

SOURCES = ["lce_api.hip", "lce_fwd.hip", "lce_bwd_dz.hip", "lce_bwd_dx.hip", "lce_bwd_dw.hip", "lce_convert.hip", "lce_compact.hip"]
# Measurement probes (`bench.py --probe`): a library of their own, so that the operator's library holds the operator only.
PROBE_LIB_NAME = "liblce_probe_gfx950.so"
PROBE_LIB_PATH = PKG_DIR / PROBE_LIB_NAME
PROBE_SOURCES = ["lce_probe.hip"]

# Packed-fp32 VALU forms are disabled for all device code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str, objdir: Path) -> Path:
    obj = objdir / (src + ".o")
    extra = os.environ.get("LCE_EXTRA_HIPCC_FLAGS", "").split()
    if src in PROBE_SOURCES:
        extra = extra + ["-munsafe-fp-atomics"]  # the flush probe measures hardware fp32 atomic adds
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
    return obj


def build(force: bool = True, verbose: bool = False) -> Path:
    """Compile every kernel translation unit for gfx950 and link the library."""
    if LIB_PATH.exists() and not force:
        return LIB_PATH
    objdir = PKG_DIR / "build"
    objdir.mkdir(exist_ok=True)
    jobs = min(len(SOURCES) + len(PROBE_SOURCES), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        all_objs = list(ex.map(lambda s: _compile(s, objdir), SOURCES + PROBE_SOURCES))
    for path, objs in ((LIB_PATH, all_objs[:len(SOURCES)]), (PROBE_LIB_PATH, all_objs[len(SOURCES):])):
        tmp = path.with_suffix(".so.tmp")
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr}")
        os.replace(tmp, path)
        if verbose:
            print(f"built {path}")
    return LIB_PATH


if __name__ == "__main__":
    build(force=True, verbose=True)
    sys.exit(0)
