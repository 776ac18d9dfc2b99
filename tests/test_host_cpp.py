"""Runs the C++ unit tests of the host layer (kernelcodegen_amd/host/tests/test_host.cc):
Frontend nests, the schedule primitives against the structural facts of the
reference's README stage dumps, interpreter equivalence of naive and scheduled
modules, the FMHA pattern match, the facade and the backend binding."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "kernelcodegen_amd", "host")


def test_host_unit_tests():
    exe = os.path.join(HOST, "test_host")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", HOST, "-j8", "test_host"], check=True, capture_output=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-4000:] + res.stderr[-2000:]
    assert "0 failed" in res.stdout
    assert res.stdout.count("[PASS]") >= 13 and "[FAIL]" not in res.stdout
