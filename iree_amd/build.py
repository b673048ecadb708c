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
# Benchmark-only helper (csrc/bench): not part of the microkernel library.
BENCH_PROBE_PATH = os.path.join(HERE, "libuk_bench_probe.so")
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


CLANG = os.environ.get("UK_CLANG", "/opt/rocm/lib/llvm/bin/clang")
DEVICE_DIR = os.path.join(CSRC, "device")
DEVICE_UKERNEL = "iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8"
DEVICE_BITCODE = os.path.join(HERE, DEVICE_UKERNEL + ".gfx950.bc")
# The flags the reference builds its ROCm microkernels with
# (build_tools/cmake/iree_bitcode_library.cmake:273-294): freestanding C23,
# no device library, AMDGPU bitcode as the output.
BITCODE_FLAGS = [
    "-x", "c", "-std=c23", "-nogpulib", "-fno-short-wchar", "-target", "amdgcn-amd-amdhsa", "-march=gfx950",
    "-fgpu-rdc", "-O3", "-fno-ident", "-fvisibility=hidden", "-Wall", "-Werror", "-c", "-emit-llvm",
]


def build_device_bitcode():
    """The in-dispatch microkernel as AMDGPU bitcode, the form a compiler's ROCm
    backend links into its dispatches."""
    cmd = [CLANG] + BITCODE_FLAGS + [os.path.join(DEVICE_DIR, DEVICE_UKERNEL + ".c"), "-o", DEVICE_BITCODE]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("device bitcode build failed:\n" + r.stdout)
    return DEVICE_BITCODE


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src, verbose):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + COMMON_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    if src == "multi_mma.hip":
        # The wrapper's kernels call the microkernel out of its bitcode. (The
        # option reaches the host pass too, which says that the bitcode is not
        # for its target and ignores it.)
        cmd += ["-Xclang", "-mlink-builtin-bitcode", "-Xclang", DEVICE_BITCODE]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l
                    and "Linking two modules of different" not in l and "[-Wlinker-warnings]" not in l
                    and "warnings generated when compiling for host" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
    if verbose and out.strip():
        print(out)
    return obj


def build(verbose=False, jobs=8):
    """Compiles every source (always, even if the library exists) and links."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    build_device_bitcode()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    build_plugin()
    build_bench_probe()
    return LIB_PATH


def build_bench_probe():
    """The matrix-pipe and HBM-stream probes bench.py reports next to its figures."""
    bench_dir = os.path.join(CSRC, "bench")
    cmd = [HIPCC] + COMMON_FLAGS + ["-shared"] + sorted(
        os.path.join(bench_dir, f) for f in os.listdir(bench_dir) if f.endswith(".hip")) + ["-o", BENCH_PROBE_PATH]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("bench probe build failed:\n" + r.stdout)
    return BENCH_PROBE_PATH


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
