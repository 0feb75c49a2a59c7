"""The C ABI used from plain C (tests/c_abi/abi_client.c): it must compile and link against the header and the
library without the Python mirror, and -- on a GPU -- run clean."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_abi", "abi_client.c")
LIBDIR = os.path.join(ROOT, "neureka_amd")


def build(tmp_path) -> str:
    exe = str(tmp_path / "abi_client")
    cmd = ["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), SRC, "-o", exe,
           "-L", LIBDIR, "-lneureka_hip", "-lm", f"-Wl,-rpath,{LIBDIR}"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return exe


def test_c_client_compiles_and_links(tmp_path):
    assert os.path.exists(build(tmp_path))


@pytest.mark.gpu
def test_c_client_runs(tmp_path):
    print("[case] C ABI client", flush=True)
    r = subprocess.run([build(tmp_path)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "all checks passed" in r.stdout, r.stdout + r.stderr
