"""The 16-bit float conversions of the kernels' epilogues (iree_amd/csrc/uk_device.h),
compiled for the host and compared with the oracle's restatement of
common.h:665-792 (pinned against the compiled reference in
tests/test_oracle_mmt4d.py): tests/host_checks/rounding_check.hip. The kernels
use a branch-free form of the reference's step-by-step rounding; this is the
check that the two are the same function, quirks included, without a GPU.
"""
import os
import subprocess

from iree_amd import build as hip_build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, "%s\n%s" % (" ".join(cmd), r.stdout[-4000:])
    return r.stdout


def test_epilogue_rounding_equals_the_oracle(tmp_path):
    oracle_obj = str(tmp_path / "uk_oracle.o")
    _run(["gcc", "-std=c11", "-O2", "-c", os.path.join(ROOT, "oracle", "uk_oracle.c"), "-o", oracle_obj])
    check_obj = str(tmp_path / "rounding_check.o")
    _run([hip_build.HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-I" + hip_build.CSRC, "-c",
          os.path.join(ROOT, "tests", "host_checks", "rounding_check.hip"), "-o", check_obj])
    exe = str(tmp_path / "rounding_check")
    # (Objects only on the link line: with a source file on it the driver takes them for sources too.)
    _run([hip_build.HIPCC, "--offload-arch=gfx950", check_obj, oracle_obj, "-o", exe, "-lpthread", "-lm"])
    out = _run([exe])
    assert "rounding check ok" in out, out
    assert "f32->f16: 3145728 inputs, 0 mismatches" in out and "f32->bf16: 393216 inputs, 0 mismatches" in out, out
