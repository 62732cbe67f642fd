"""The C++ mirror of the operator surface (include/shrike.hpp) on the GPU: the reference's closed-form FFN
case through the decode operators and through the prefill chain, built with g++ against libshrikehip only."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.gpu
def test_cpp_mirror_runs_the_closed_form_case_on_the_gpu(gpu, tmp_path):
    exe = tmp_path / "gpu_harness"
    libdir = os.path.join(ROOT, "shrike_amd")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "gpu_harness.cpp"), "-o", str(exe),
                    "-L", libdir, "-lshrikehip", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=100)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "all gpu checks passed" in out.stdout


def test_cpp_gpu_harness_builds(tmp_path):
    """Compiles and links here, where there is no GPU to run it on."""
    exe = tmp_path / "gpu_harness"
    libdir = os.path.join(ROOT, "shrike_amd")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "gpu_harness.cpp"), "-o", str(exe),
                    "-L", libdir, "-lshrikehip", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
