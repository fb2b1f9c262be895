"""The C++ header API (include/flashck/fmha/fmha_fwd.h) compiles, links against the library and validates its
arguments before launching; runs without a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_compiles_links_and_validates(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    lib_dir = os.path.join(ROOT, "flashck_amd")
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not installed")
    assert os.path.exists(os.path.join(lib_dir, "libflashck_fmha.so")), "build the library first: python -m flashck_amd.build"
    exe = str(tmp_path / "fmha_header_check")
    cmd = [hipcc, "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cpp", "fmha_header_check.cpp"), "-o", exe,
           "-L", lib_dir, "-lflashck_fmha", f"-Wl,-rpath,{lib_dir}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip().endswith("OK"), r.stdout + r.stderr
