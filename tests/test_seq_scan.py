"""csrc/seq_scan.h turns a left-to-right fp32 summation into an associative scan over integer step
functions.  This compiles the header for the host and fuzzes it against real float additions
(softmax-like terms, exact ties, subnormals, binade jumps, linear and tree-shaped scans).  CPU only."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_seq_scan_equals_sequential_float_sum(tmp_path):
    exe = tmp_path / "seq_scan_check"
    subprocess.check_call(["g++", "-O1", "-ffp-contract=off", "-I", os.path.join(ROOT, "onnxruntime-genai_amd", "csrc"),
                           os.path.join(ROOT, "tests", "seq_scan_check.cpp"), "-o", str(exe)])
    bad, cases = subprocess.check_output([str(exe)], text=True).split()
    assert bad == "0" and int(cases) > 1000
