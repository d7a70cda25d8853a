"""Builds libflash_decode_gfx950.so from csrc/*.hip with hipcc (cross-compiles without a GPU).

    python triton-distributed_amd/build.py            # build in tree
    python triton-distributed_amd/build.py --force    # rebuild everything

The library is kept inside the package directory so that it travels with the
source tree; nothing is installed into site-packages.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
BUILD = os.path.join(PKG_DIR, "_build")
LIB_NAME = "libflash_decode_gfx950.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)
SOURCES = ["fd_api.hip", "fd_split_mfma.hip", "fd_split_mfma_fp8.hip", "fd_split_mfma_fp8_d256.hip", "fd_split_mfma_fp8_d64.hip", "fd_split_mfma_d256.hip", "fd_split_mfma_d64.hip", "fd_split_valu.hip", "fd_combine.hip",
           "fd_kv_append.hip"]
HEADERS = [os.path.join(CSRC, "fd_common.h"), os.path.join(CSRC, "fd_mma.h"),
           os.path.join(os.path.dirname(PKG_DIR), "include", "flash_decode.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed-FP32 VALU ops are switched off for every device translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src: str, force: bool, verbose: bool) -> str:
    obj = os.path.join(BUILD, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + HEADERS):
        cmd = [_hipcc()] + HIPCC_FLAGS + ["-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}")
        if verbose:
            noise = "is not a recognized feature for this target"
            out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
            if out.strip():
                print(out, flush=True)
    return obj


def build(force: bool = False, verbose: bool = True) -> str:
    """Compiles every HIP source for gfx950 and links the shared library.  Returns its path."""
    os.makedirs(BUILD, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, verbose), SOURCES))
    if force or _stale(LIB_PATH, objs):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stdout}")
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--quiet", action="store_true")
    ns = ap.parse_args()
    print(build(force=ns.force, verbose=not ns.quiet))
    sys.exit(0)


def ensure_built(verbose: bool = False) -> str:
    """For tests, the smoke check and the bench: the library as it is if it has been built (or FD_LIBRARY_PATH names
    one), else one build.  The package itself never builds behind the caller's back: ``load_library`` raises."""
    override = os.environ.get("FD_LIBRARY_PATH")
    if override:
        return override
    if os.path.exists(LIB_PATH):
        return LIB_PATH
    return build(force=False, verbose=verbose)
