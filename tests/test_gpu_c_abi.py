"""Runs the C consumer of the ABI (tests/c_abi/run_c_abi.c: no Python between the caller and the library) on the GPU;
it checks fd_decode / fd_decode_planned / fd_schedule / fd_plan_splits / fd_kv_append against the plain-C oracle and exits 0 on success."""
import importlib.util
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu


def test_c_program_through_the_abi(fd):
    fd.load_library()          # the library must exist; the consumer links against it
    spec = importlib.util.spec_from_file_location("oracle_c_build", os.path.join(ROOT, "oracle", "c", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    binary = mod.build_c_abi_consumer()            # compiles only if it is not there (gcc, no GPU needed)
    res = subprocess.run([binary], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(res.stdout)
    assert res.returncode == 0 and "PASSED" in res.stdout, res.stdout
