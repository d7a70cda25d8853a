"""Builds the plain-C restatement of the decode oracle (``libref_decode.so``, gcc) and, on request, the C consumer of
the library's ABI that checks itself against it (``tests/c_abi/run_c_abi``).  Test infrastructure only."""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "libref_decode.so")
C_ABI_SRC = os.path.join(ROOT, "tests", "c_abi", "run_c_abi.c")
C_ABI_BIN = os.path.join(ROOT, "tests", "c_abi", "run_c_abi")


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("failed: " + " ".join(cmd) + "\n" + res.stdout)


def build_oracle(force: bool = False) -> str:
    src = os.path.join(HERE, "ref_decode.c")
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(src):
        _run([shutil.which("gcc") or "gcc", "-O2", "-std=c11", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wextra", "-shared",
              "-o", LIB, src, "-lm"])
    return LIB


def build_c_abi_consumer(force: bool = False, rocm: str = "/opt/rocm") -> str:
    """Needs the flash-decode library to be built already (it links against it)."""
    pkg = os.path.join(ROOT, "triton-distributed_amd")
    deps = [C_ABI_SRC, os.path.join(HERE, "ref_decode.c"), os.path.join(ROOT, "include", "flash_decode.h")]
    if force or not os.path.exists(C_ABI_BIN) or any(os.path.getmtime(C_ABI_BIN) < os.path.getmtime(d) for d in deps):
        _run([shutil.which("gcc") or "gcc", "-O2", "-std=c11", "-Wall", "-D__HIP_PLATFORM_AMD__", C_ABI_SRC,
              os.path.join(HERE, "ref_decode.c"), "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(rocm, "include"),
              "-L" + pkg, "-lflash_decode_gfx950", "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-lm",
              "-Wl,-rpath,$ORIGIN/../../triton-distributed_amd", "-Wl,-rpath," + os.path.join(rocm, "lib"), "-o", C_ABI_BIN])
    return C_ABI_BIN


if __name__ == "__main__":
    print(build_oracle(force=True))
    print(build_c_abi_consumer(force=True))
