"""include/shrike.hpp (the C++ host mirror of the reference's operator classes) compiles against the
C ABI, and the reference's host-side unit tests written against it pass. No GPU is touched."""
import os
import subprocess

from shrike_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_harness_builds_and_passes(tmp_path):
    exe = tmp_path / "host_harness"
    libdir = os.path.dirname(capi.LIB_PATH)
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "host_harness.cpp"), "-o", str(exe),
                    "-L", libdir, "-lshrikehip", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "all host checks passed" in out.stdout
