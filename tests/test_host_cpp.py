"""Runs the C++ unit tests of the host side (kernel registry / selection / emitters / code generator);
the cases and their assertions live in tests/cpp/test_host.cpp."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "nnfusion_amd", "bin", "test_host")


def test_host_cpp_suite(tmp_path):
    assert os.path.exists(BIN), "nnfusion_amd/bin/test_host is not built (make -C nnfusion_amd/csrc/host)"
    proc = subprocess.run([BIN, str(tmp_path), os.path.join(ROOT, "tests", "golden")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    lines = [l for l in proc.stdout.splitlines() if l.startswith(("PASS", "FAIL"))]
    failed = [l for l in lines if l.startswith("FAIL")]
    assert proc.returncode == 0 and not failed, proc.stdout
    assert len(lines) >= 15
