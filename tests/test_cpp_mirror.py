"""Builds the C++ host mirror's restatement of the reference's own unit tests and runs it:
host-only checks here, everything on the GPU box."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "cpp", "test_reference_suite.cpp")
LIBDIR = os.path.join(ROOT, "pmetal_amd")


def _build(tmp_path):
    if not os.path.exists(os.path.join(LIBDIR, "libpmetal_hip.so")):
        from pmetal_amd import build
        build.build()
    exe = str(tmp_path / "test_reference_suite")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"), SRC, "-o", exe,
                    "-L", LIBDIR, "-lpmetal_hip", f"-Wl,-rpath,{LIBDIR}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    return exe


def test_cpp_mirror_host_only(tmp_path):
    r = subprocess.run([_build(tmp_path), "--host-only"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_cpp_mirror_on_gpu(tmp_path):
    r = subprocess.run([_build(tmp_path)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
