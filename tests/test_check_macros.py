"""TC_CHECK message layout and exception types: a C++ program built against tc/core/check.h
restates the scenarios of the reference's test/test_check.cc and reports mismatches."""
import os
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_check_macros_match_the_reference_messages():
    src = os.path.join(ROOT, "tests", "cpp", "check_messages.cc")
    inc = os.path.join(ROOT, "tensorcomprehensions_amd", "csrc")
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, "check_messages")
        subprocess.run(["g++", "-std=c++17", "-O0", "-I", inc, src, "-o", exe], check=True, capture_output=True, text=True)
        r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout
    assert "0 expectation(s) failed" in r.stdout
