"""Builds liblce_gfx950.so from csrc/ with hipcc (cross-compiles without a GPU).

Usage: ``python -m linear_cross_entropy_loss_amd.build [--probes]``  (``--probes``: the measurement probes of
``bench.py --probe`` instead, a library of their own)
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

SOURCES = ["lce_api.hip", "lce_fwd.hip", "lce_bwd_dz.hip", "lce_bwd_dx.hip", "lce_bwd_dw.hip", "lce_convert.hip", "lce_compact.hip", "lce_fuse.hip"]
# Measurement probes (`bench.py --probe`): sources and library of their own, built on demand only.
PROBE_DIR = PKG_DIR / "probes"
PROBE_LIB_NAME = "liblce_probe_gfx950.so"
PROBE_LIB_PATH = PROBE_DIR / PROBE_LIB_NAME
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


def _compile(srcdir: Path, src: str, objdir: Path, extra=()) -> Path:
    obj = objdir / (src + ".o")
    env_extra = os.environ.get("LCE_EXTRA_HIPCC_FLAGS", "").split()
    cmd = [_hipcc(), *HIPCC_FLAGS, *env_extra, *extra, "-c", str(srcdir / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
    return obj


def _link(path: Path, objs) -> None:
    tmp = path.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, path)


def build(force: bool = True, verbose: bool = False) -> Path:
    """Compile every kernel translation unit of the operator for gfx950 and link the library."""
    if LIB_PATH.exists() and not force:
        return LIB_PATH
    objdir = PKG_DIR / "build"
    objdir.mkdir(exist_ok=True)
    jobs = min(len(SOURCES), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(CSRC, s, objdir), SOURCES))
    _link(LIB_PATH, objs)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


def build_probes(verbose: bool = False) -> Path:
    """Compile and link the measurement probes (not part of the operator, nothing else loads them)."""
    objdir = PKG_DIR / "build"
    objdir.mkdir(exist_ok=True)
    # (the flush probe measures hardware fp32 atomic adds)
    objs = [_compile(PROBE_DIR, s, objdir, ["-munsafe-fp-atomics"]) for s in PROBE_SOURCES]
    _link(PROBE_LIB_PATH, objs)
    if verbose:
        print(f"built {PROBE_LIB_PATH}")
    return PROBE_LIB_PATH


if __name__ == "__main__":
    if "--probes" in sys.argv[1:]:
        build_probes(verbose=True)
    else:
        build(force=True, verbose=True)
    sys.exit(0)
