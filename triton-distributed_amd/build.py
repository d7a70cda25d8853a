"""Builds libflash_decode_gfx950.so from csrc/*.hip with hipcc (cross-compiles without a GPU).

    python triton-distributed_amd/build.py            # build in tree
    python triton-distributed_amd/build.py --force    # rebuild everything

The library is kept inside the package directory so that it travels with the
source tree; nothing is installed into site-packages.
"""
from __future__ import annotations

import argparse
import hashlib
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
    # Machine-code sinking off: the split kernels request a sequence's length right behind their argument batch and
    # use it only after the index arithmetic of the work item; the sinking pass moves such a load down to the block of
    # its first use, where the wave then waits a full round trip for it.
    "-mllvm", "-disable-machine-sink",
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


def source_id() -> str:
    """Hash of every source and header the library is built from (and of the compiler flags)."""
    h = hashlib.sha256(" ".join(HIPCC_FLAGS).encode())
    for path in [os.path.join(CSRC, s) for s in SOURCES] + HEADERS:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


_ID_TAG = b"FD_BUILD_ID="


def built_id(path: str = LIB_PATH) -> str:
    """The build id inside a built library (what its ``fd_build_id()`` returns), read from the file without loading
    it -- a stale image, once loaded, would stay this process's image of that path; "" if there is none."""
    try:
        with open(path, "rb") as f:
            blob = f.read()
    except OSError:
        return ""
    at = blob.find(_ID_TAG)
    if at < 0:
        return ""
    end = blob.find(b"\0", at)
    return blob[at + len(_ID_TAG):end].decode("ascii", "replace")


def _compile(src: str, force: bool, verbose: bool, build_id: str) -> str:
    obj = os.path.join(BUILD, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    stamped = src == "fd_api.hip"   # the translation unit that carries the build id: rebuilt whenever the id changes
    if force or _stale(obj, [path] + HEADERS) or stamped:
        cmd = [_hipcc()] + HIPCC_FLAGS + ([f'-DFD_BUILD_ID="{build_id}"'] if stamped else []) + ["-c", path, "-o", obj]
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
    build_id = source_id()
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, verbose, build_id), SOURCES))
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
    """For tests, the smoke check and the bench: the library as it is if it has been built from the sources in this
    tree (or FD_LIBRARY_PATH names one), else one build.  A library whose ``fd_build_id()`` differs from the hash of
    the sources beside it is stale -- it would be tested in place of the code under review -- and is rebuilt (an
    error if that is not possible, never a silent pass).  The package itself never builds behind the caller's
    back: ``load_library`` raises."""
    override = os.environ.get("FD_LIBRARY_PATH")
    if override:
        return override
    if os.path.exists(LIB_PATH):
        want, have = source_id(), built_id()
        if have == want:
            return LIB_PATH
        print(f"{LIB_NAME} is stale (built from {have or 'unknown sources'}, the tree is {want}): rebuilding",
              file=sys.stderr, flush=True)
        build(force=True, verbose=verbose)
        if built_id() != want:
            raise RuntimeError(f"{LIB_PATH} does not match the sources after a rebuild")
        return LIB_PATH
    return build(force=False, verbose=verbose)
