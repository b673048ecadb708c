"""Writes tests/golden/reference_outputs.json: outputs of the reference's own
ukernels (compiled from its sources into oracle/_ref by oracle/Makefile) on the
seeded inputs of the benchmark configurations, condensed to what fits a
repository: a BLAKE2b-128 digest of the whole output plus 1024 sampled values.
Run in a container that has the reference tree: python tests/golden/make_golden.py

Integer outputs do not depend on the tile shape, so the 4096-cubed s8s8s32
output is produced with the reference's AVX-512-VNNI tiles (16x16x2, the only
int8 shape its x86-64 code accelerates) from the same logical matrices and
digested in row-major order of the logical result; the GPU test re-tiles its
8x8x4 output the same way. Everything else uses the generic tile functions in
the configuration's own tile shape.
"""
import ctypes as C
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402
from iree_amd import abi, synth  # noqa: E402

THREADS = os.cpu_count() or 1


def digest(a):
    return hashlib.blake2b(np.ascontiguousarray(a).tobytes(), digest_size=16).hexdigest()


def sample_indices(n, count=1024, seed=12345):
    return np.sort(synth.bits64(seed, 99, count) % np.uint64(n)).astype(np.int64)


def tile(x, T0, K0):
    """[rows, depth] -> [rows/T0][depth/K0][T0][K0], flattened."""
    r, d = x.shape
    return np.ascontiguousarray(x.reshape(r // T0, T0, d // K0, K0).transpose(0, 2, 1, 3)).reshape(-1)


def untile_out(flat, M, N, M0, N0):
    return np.ascontiguousarray(flat.reshape(M, N, M0, N0).transpose(0, 2, 1, 3)).reshape(M * M0, N * N0)


def run_ref(ref, cpu, lhs, rhs, out, M, N, K, M0, N0, K0, flags, rhs_stride=None):
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data
    p.lhs_stride0, p.out_stride0 = K * M0 * K0, N * M0 * N0
    p.rhs_stride0 = K * N0 * K0 if rhs_stride is None else rhs_stride
    p.M, p.N, p.K, p.M0, p.N0, p.K0 = M, N, K, M0, N0, K0
    p.flags = flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK
    p.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
    t0 = time.time()
    ref.ref_mmt4d_mt(C.byref(p), THREADS)
    assert ref.ref_fail_count() == 0
    return time.time() - t0


def main():
    ref = oracle.ref_lib()
    assert ref is not None, "needs oracle/_ref (the reference tree must be present to build it)"
    cpu = oracle.host_cpu_data()
    out = {}

    # config 1: s8s8s32, 1024^3, tiles 8x8x4, generic tile function, tiled output as is.
    M = N = 128; K = 256
    lhs = synth.uniform_int8(0, 0, M * K * 32); rhs = synth.uniform_int8(0, 1, N * K * 32)
    res = np.zeros(M * N * 64, dtype=np.int32)
    dt = run_ref(ref, cpu, lhs, rhs, res, M, N, K, 8, 8, 4, abi.MMT4D_TYPE_S8S8S32)
    idx = sample_indices(res.size)
    out["s8s8s32_1024_8x8x4"] = {"seed": [0, 0, 1], "digest_of_tiled_output": digest(res),
                                 "sample_index": idx.tolist(), "sample_value": res[idx].tolist(), "seconds": round(dt, 1)}
    print("config 1:", dt, flush=True)

    # headline: s8s8s32 logical 4096^3. Inputs are the 8x8x4-tiled streams the benchmark uses; re-tiled to 16x16x2.
    M = N = 512; K = 1024
    lhs = synth.uniform_int8(0, 0, M * K * 32); rhs = synth.uniform_int8(0, 1, N * K * 32)
    a = np.ascontiguousarray(lhs.reshape(M, K, 8, 4).transpose(0, 2, 1, 3)).reshape(4096, 4096)
    b = np.ascontiguousarray(rhs.reshape(N, K, 8, 4).transpose(0, 2, 1, 3)).reshape(4096, 4096)
    res = np.zeros(4096 * 4096, dtype=np.int32)
    dt = run_ref(ref, cpu, tile(a, 16, 2), tile(b, 16, 2), res, 256, 256, 2048, 16, 16, 2, abi.MMT4D_TYPE_S8S8S32)
    logical = untile_out(res, 256, 256, 16, 16)
    idx = sample_indices(logical.size)
    out["s8s8s32_4096_logical"] = {"seed": [0, 0, 1], "digest_of_row_major_logical_output": digest(logical),
                                   "sample_index": idx.tolist(), "sample_value": logical.reshape(-1)[idx].tolist(),
                                   "reference_tiles": "16x16x2 (AVX-512 VNNI)", "seconds": round(dt, 1)}
    print("headline:", dt, flush=True)
    del a, b, logical

    # config 5: s8s4s32 512 x 11008 x 4096, tiles 16x16x32: the first 4 of the 32 rows of lhs tiles (64 logical rows).
    Ms, N, K = 4, 688, 128
    lhs = synth.uniform_int8(5, 0, 512 * 4096)[:Ms * K * 16 * 32]
    rhs = synth.uniform_int4_packed(5, 1, 11008 * 4096)
    res = np.zeros(Ms * N * 256, dtype=np.int32)
    dt = run_ref(ref, cpu, lhs, rhs, res, Ms, N, K, 16, 16, 32, abi.MMT4D_TYPE_S8S4S32)
    idx = sample_indices(res.size)
    out["s8s4s32_512x11008x4096_rows_0_63"] = {"seed": [5, 0, 1], "digest_of_tiled_output": digest(res),
                                               "sample_index": idx.tolist(), "sample_value": res[idx].tolist(),
                                               "seconds": round(dt, 1)}
    print("config 5:", dt, flush=True)

    # config 3: f16f16f32 4096^3 tiles 16x16x16 with accumulate: rows of lhs tiles 0 and 131, float values
    # (compared within tolerance on the GPU: no digest).
    M = N = K = 256
    lhs = synth.f16_bits(synth.normal_f32(3, 0, M * K * 256, 1.0 / 64))
    rhs = synth.f16_bits(synth.normal_f32(3, 1, N * K * 256, 1.0 / 64))
    init = synth.normal_f32(3, 2, M * N * 256, 1.0)
    entry = {"seed": [3, 0, 1, 2], "rows_of_tiles": [0, 131], "sample_index": [], "sample_value": []}
    for row in (0, 131):
        res = init[row * N * 256:(row + 1) * N * 256].copy()
        dt = run_ref(ref, cpu, lhs[row * K * 256:(row + 1) * K * 256], rhs, res, 1, N, K, 16, 16, 16,
                     abi.MMT4D_TYPE_F16F16F32 | abi.MMT4D_ACCUMULATE)
        idx = sample_indices(res.size, count=512, seed=777 + row)
        entry["sample_index"].append(idx.tolist())
        entry["sample_value"].append([float(v) for v in res[idx]])
        print("config 3 row", row, dt, flush=True)
    out["f16f16f32_4096_16x16x16_accumulate"] = entry

    # config 2: pack f32 [8191, 8190] with 16x1 tiles, the three variants of the benchmark, and unpack of the first.
    R, Cc = 8191, 8190
    src = synth.normal_f32(2, 0, R * Cc)
    entry = {"seed": [2, 0]}
    for name, flags, o0, o1 in (("tiles16x1", 0, 512, Cc), ("transpose_inner", abi.PACK_TRANSPOSE_INNER, R, 512),
                                ("rhs_form", abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER, 512, R)):
        packed = np.full(o0 * o1 * 16, np.nan, dtype=np.float32)
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src.ctypes.data, packed.ctypes.data
        p.in_stride0, p.in_stride1, p.out_stride0, p.out_stride1 = Cc, 1, o1 * 16, 16
        p.in_size0, p.in_size1 = R, Cc
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = o0, o1, 16, 1
        p.padding_value, p.flags = 0, abi.PACK_TYPE_F32F32 | flags
        p.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
        if ref.ref_pack_mt(C.byref(p), THREADS) != 0:   # the threaded driver splits rows of tiles of untransposed outputs only
            ref.ref_pack(C.byref(p))
        entry["pack_" + name] = digest(packed)
        if name == "tiles16x1":
            back = np.full(R * Cc, -1.0, dtype=np.float32)
            u = abi.UnpackParams()
            u.in_buffer, u.out_buffer = packed.ctypes.data, back.ctypes.data
            u.in_stride0, u.in_stride1, u.out_stride0, u.out_stride1 = Cc * 16, 16, Cc, 1
            u.in_size0, u.in_size1, u.in_size2, u.in_size3 = 512, Cc, 16, 1
            u.out_size0, u.out_size1, u.flags = R, Cc, abi.UNPACK_TYPE_F32F32
            u.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
            if ref.ref_unpack_mt(C.byref(u), THREADS) != 0:
                ref.ref_unpack(C.byref(u))
            entry["unpack_tiles16x1"] = digest(back)
            entry["source"] = digest(src)
        print("config 2", name, flush=True)
    out["pack_unpack_f32_8191x8190"] = entry

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_outputs.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
