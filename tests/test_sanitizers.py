"""AddressSanitizer + UndefinedBehaviorSanitizer runs of the host-side code, on
the CPU (the reference offers the same as build options, CMakeLists.txt:453-456):

* oracle/uk_oracle.c over ragged shapes, gaps and offsets on exact-size heap
  buffers (tests/sanitize/oracle_san_driver.c);
* the host shim of the C ABI, iree_amd/csrc/uk_api.hip (parameter checks, early
  exits, operand extents near the limits the checks admit, staging decisions),
  its host pass compiled with the sanitizers and linked with the library's
  ordinary kernel objects (tests/sanitize/shim_san_driver.cpp). Device code is
  not instrumented.
"""
import os
import subprocess

from iree_amd import build as hip_build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN = os.path.join(ROOT, "tests", "sanitize")
CLANGXX = "/opt/rocm/lib/llvm/bin/clang++"


def _run(cmd, **kw):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    assert r.returncode == 0, "%s\n%s" % (" ".join(cmd), r.stdout[-4000:])
    return r.stdout


def test_oracle_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "oracle_san")
    _run(["gcc", "-std=c11", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
          "-static-libasan", "-static-libubsan", os.path.join(SAN, "oracle_san_driver.c"),
          os.path.join(ROOT, "oracle", "uk_oracle.c"), "-o", exe, "-lpthread", "-lm"])
    out = _run([exe], env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1"))
    assert "oracle sanitizer run ok" in out


def test_host_shim_under_asan_ubsan(tmp_path):
    objs = [os.path.join(hip_build.OBJ_DIR, os.path.splitext(s)[0] + ".o") for s in hip_build.sources()]
    if not all(os.path.exists(o) for o in objs):
        hip_build.build()
    san = ["-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=all"]
    shim = str(tmp_path / "uk_api_san.o")
    host_san = [x for flag in san for x in ("-Xarch_host", flag)]
    _run([hip_build.HIPCC] + [f for f in hip_build.COMMON_FLAGS if f != "-O3"] + ["-O1", "-g"] + host_san +
         ["-c", os.path.join(hip_build.CSRC, "uk_api.hip"), "-o", shim])
    driver = str(tmp_path / "driver.o")
    _run([CLANGXX, "-O1", "-g", "-std=c++17"] + san + ["-c", os.path.join(SAN, "shim_san_driver.cpp"), "-o", driver])
    exe = str(tmp_path / "shim_san")
    _run([hip_build.HIPCC, "--offload-arch=gfx950", "-fno-gpu-sanitize", "-fsanitize=address", "-fsanitize=undefined",
          driver, shim] + [o for o in objs if not o.endswith("/uk_api.o")] + ["-o", exe])
    # (The HIP runtime keeps allocations until the process ends.)
    out = _run([exe], env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
    assert "shim sanitizer run ok" in out
