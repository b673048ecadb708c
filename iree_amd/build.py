"""Builds iree_amd/libiree_uk_mi355x.so from iree_amd/csrc with hipcc for gfx950.

Usage: python -m iree_amd.build [-v]
The library is built in-tree so that it travels with the source tree; nothing
is installed outside it.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build", "obj")
LIB_PATH = os.path.join(HERE, "libiree_uk_mi355x.so")
PLUGIN_PATH = os.path.join(HERE, "libiree_uk_mi355x_plugin.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# Packed-FP32 instruction selection is switched off for every device
# translation unit; the host pass does not know the feature and says so.
COMMON_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # The MFMA main loops are written as fully unrolled loops whose indices must
    # be compile-time constants (register arrays); the f32 kernel's loop body is
    # past the default size limit for `#pragma unroll`.
    "-mllvm", "-pragma-unroll-threshold=1000000",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src, verbose):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + COMMON_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
    if verbose and out.strip():
        print(out)
    return obj


def build(verbose=False, jobs=8):
    """Compiles every source (always, even if the library exists) and links."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    build_plugin()
    return LIB_PATH


def build_plugin():
    """The HAL executable plugin: plain C on top of the library's C ABI, found
    next to it at run time ($ORIGIN)."""
    cmd = ["gcc", "-O2", "-std=c11", "-Wall", "-Wextra", "-fPIC", "-shared", "-fvisibility=hidden",
           "-I", os.path.join(os.path.dirname(HERE), "include"), "-I", os.path.join(CSRC, "plugin"),
           os.path.join(CSRC, "plugin", "uk_plugin.c"), "-o", PLUGIN_PATH,
           "-L", HERE, "-liree_uk_mi355x", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("plugin build failed:\n" + r.stdout)
    return PLUGIN_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
