"""The kernels evaluate exp/log with csrc/exact_math.h so that device results equal the host libm
results the reference CPU path produces (std::exp/std::log on float).  This test compiles the header
for the host and compares it with libm over all 2^32 float bit patterns.  CPU only."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_expf_logf_bit_identical_to_host_libm(tmp_path):
    exe = tmp_path / "exact_math_check"
    flags = ["-O2", "-fopenmp", "-ffp-contract=off"]
    if "fma" in open("/proc/cpuinfo").read():
        flags.append("-mfma")
    subprocess.check_call(["g++", *flags, "-I", os.path.join(ROOT, "onnxruntime-genai_amd", "csrc"),
                           os.path.join(ROOT, "tests", "exact_math_check.cpp"), "-o", str(exe)])
    out = subprocess.check_output([str(exe)], text=True).split()
    assert out == ["0", "0"], f"expf/logf mismatches vs libm: {out}"
