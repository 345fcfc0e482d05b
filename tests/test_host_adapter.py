"""Compiles and runs the host-only C++ check of the reference-shaped adapter
(ml-drift_amd/host/mld_hip_ops.h) against libmldhip.so.  No GPU needed."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_adapter(tmp_path):
    exe = str(tmp_path / "host_adapter_test")
    lib_dir = os.path.join(ROOT, "ml-drift_amd")
    subprocess.check_call(["g++", "-std=c++17", "-O1", os.path.join(ROOT, "tests", "host_adapter_test.cpp"), "-o", exe,
                           "-L" + lib_dir, "-lmldhip", "-Wl,-rpath," + lib_dir])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host adapter ok" in out.stdout
