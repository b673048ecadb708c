"""Benchmark of the data-tiled matmul microkernels on one MI355X.

Headline workload (one "step" = one launch): iree_uk_mmt4d, s8s8s32, logical
4096x4096x4096 with the 8x8x4 tiles of the reference's int8 configuration
(lhs [512,1024,8,4], rhs [512,1024,8,4], out [512,512,8,8] int32), inputs
resident in HBM. Prints ONE JSON line; besides the headline it carries the
MFMA roofline of that kernel, the reference CPU ukernels timed on this host,
and one-launch figures for the other configurations (pack/unpack GB/s, f16,
skinny bf16, int4) under "also".

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-also]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Published MI355X peaks used for the roofline fractions.
PEAK_INT8_TOPS = 5033.0     # dense int8 MFMA
PEAK_F16_TFLOPS = 2516.0    # dense f16 / bf16 MFMA
PEAK_F32_TFLOPS = 157.3     # dense f32 MFMA
PEAK_HBM_GBS = 8000.0       # HBM3E

# HBM traffic of ONE launch of the headline kernel, measured with the
# profiler's FETCH_SIZE and WRITE_SIZE counters (two separate counter runs of
# this script, each reading scaled by what the same counter reports for a plain
# device-to-device copy of known size: x2.00 for FETCH_SIZE, x1.00 for
# WRITE_SIZE on this part). The algorithmic minimum is 32 MiB read + 64 MiB
# written = 100.7 MB; reads above it are lhs/rhs panels fetched by more than
# one of the 8 L2s. profiles/ holds the counter summaries.
HEADLINE_TRAFFIC_BYTES = 167_835_648   # 49,175.5 KiB x 2.00 fetched + 65,551 KiB written


def _mmt4d_params(abi, lhs, rhs, out, M, N, K, M0, N0, K0, flags):
    lb, rb, ob = abi.MMT4D_BITS[flags & 0xFF]
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs, rhs, out
    p.lhs_stride0, p.rhs_stride0, p.out_stride0 = K * M0 * K0, K * N0 * K0, N * M0 * N0
    p.M, p.N, p.K, p.M0, p.N0, p.K0, p.flags = M, N, K, M0, N0, K0, flags
    return p


def _time_launches(torch, fn, steps, warmup):
    """Average ms per call of fn() over `steps` calls, by HIP events on the
    stream the kernels are launched on, bracketed by device synchronisation."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1) / steps, wall_ms / steps


def _per_launch_ms(torch, fn, launches):
    """Duration of each of `launches` calls of fn(), every one bracketed by its
    own pair of HIP events: (median, min) in ms."""
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
             for _ in range(launches)]
    torch.cuda.synchronize()
    for e0, e1 in pairs:
        e0.record()
        fn()
        e1.record()
    torch.cuda.synchronize()
    ms = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    return ms[len(ms) // 2], ms[0]


def _headline(torch, lib, abi, synth, steps, warmup):
    import numpy as np
    M = N = 512
    K = 1024
    M0 = N0 = 8
    K0 = 4
    flags = abi.MMT4D_TYPE_S8S8S32
    lhs = torch.from_numpy(synth.uniform_int8(0, 0, M * K * M0 * K0)).cuda()
    rhs = torch.from_numpy(synth.uniform_int8(0, 1, N * K * N0 * K0)).cuda()
    out = torch.empty(M * N * M0 * N0, dtype=torch.int32, device="cuda")
    p = _mmt4d_params(abi, lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0, flags)
    ev_ms, wall_ms = _time_launches(torch, lambda: lib.iree_uk_mmt4d_p(C.byref(p)), steps, warmup)
    med_ms, min_ms = _per_launch_ms(torch, lambda: lib.iree_uk_mmt4d_p(C.byref(p)), max(steps, 20))
    kernel = lib.iree_uk_mi355x_last_kernel().decode()
    # Checksum of checksums, independent of any CPU code: the sum of all
    # outputs equals (column sums of A) . (column sums of B), with k running
    # over (k, k0) pairs.
    a_cols = lhs.view(M, K, M0, K0).to(torch.int64).sum(dim=(0, 2)).reshape(-1)
    b_cols = rhs.view(N, K, N0, K0).to(torch.int64).sum(dim=(0, 2)).reshape(-1)
    verified = bool((a_cols * b_cols).sum().item() == out.to(torch.int64).sum().item())
    ops = 2.0 * M * N * K * M0 * N0 * K0
    return dict(ops=ops, ev_ms=ev_ms, wall_ms=wall_ms, med_ms=med_ms, min_ms=min_ms, kernel=kernel,
                verified=verified, params=p, keep=(lhs, rhs, out),
                workload="iree_uk_mmt4d s8s8s32 logical 4096x4096x4096, tiles M0=N0=8 K0=4 "
                         "(lhs [512,1024,8,4], rhs [512,1024,8,4], out i32 [512,512,8,8]), "
                         "accumulate off, operands resident in HBM")


def _sustained_ceiling(torch, abi, synth):
    """What the matrix pipe sustains on the headline's data with the headline kernel's inner-loop instruction
    mix (32 MFMAs, 16 LDS reads, 8 loads to LDS, one barrier per step) and no HBM traffic, prologue or
    epilogue: the benchmark's probe on uniformly random int8. The published peak assumes 2.4 GHz; the part
    clocks lower on data that toggles."""
    from iree_amd import library
    rnd = torch.from_numpy(synth.uniform_int8(0, 0, 2 << 20)).cuda()
    tops, mhz = C.c_double(), C.c_double()
    rc = library.load_bench_probe().uk_bench_probe_matrix_pipe(abi.MMT4D_TYPE_S8S8S32, rnd.data_ptr(), rnd.numel(), 1, 4096,
                                                               C.byref(tops), C.byref(mhz))
    if rc != 0:
        raise RuntimeError("matrix pipe probe failed: HIP error %d" % rc)
    return {"value": round(tops.value, 1), "unit": "TOP/s", "shader_mhz": round(mhz.value),
            "frac_of_peak": round(tops.value / PEAK_INT8_TOPS, 4),
            "what": "probe: the kernel's MFMA + LDS instruction mix on uniformly random int8, L1-resident operands, "
                    "no prologue, no store"}


def _in_kernel_timeline(torch, synth):
    """Where the time of one headline launch goes, from readings of the 100 MHz counter inside the kernel (the
    benchmark's probe: the library's kernel source compiled once more with its timeline readings on). Medians over
    the 256 workgroups, in microseconds, for the kernel as launched (staggered tail: the last three chunks are
    multiplied fragment by fragment and stored as they finish) and for the variant that stores everything
    after the loop."""
    import numpy as np
    from iree_amd import library
    probe = library.load_bench_probe()
    lhs = torch.from_numpy(synth.uniform_int8(0, 0, 4096 * 4096)).cuda()
    rhs = torch.from_numpy(synth.uniform_int8(0, 1, 4096 * 4096)).cuda()
    out = torch.empty(4096 * 4096, dtype=torch.int32, device="cuda")
    res = {}
    for name, staggered in (("staggered_tail", 1), ("all_stores_after_the_loop", 0)):
        readings = (C.c_double * (256 * 5))()
        tiles = C.c_int()
        rc = probe.uk_bench_probe_mmt4d_timeline(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), 512, 512, 1024, 8, 8, 4,
                                                 staggered, 400, 10, readings, C.byref(tiles))
        if rc != 0:
            raise RuntimeError("timeline probe failed: HIP error %d" % rc)
        t = np.array(readings[:5 * tiles.value]).reshape(tiles.value, 5) / 1e3
        med = lambda x: round(float(np.median(x)), 2)
        res[name] = {"prologue_us": med(t[:, 1] - t[:, 0]), "main_loop_us": med(t[:, 2] - t[:, 1]),
                     "tail_until_last_mfma_us": med(t[:, 3] - t[:, 2]),
                     "stores_after_last_mfma_until_acknowledged_us": med(t[:, 4] - t[:, 3]),
                     "first_start_to_last_end_us": round(float(t[:, 4].max()), 2),
                     "workgroup_starts_spread_us": round(float(t[:, 0].max()), 2)}
    # The two variants timed from outside, alternating, 4 x 50 launches each.
    stream = torch.cuda.current_stream().cuda_stream
    totals = {1: 0.0, 0: 0.0}
    for _ in range(4):
        for staggered in (1, 0):
            def launch():
                rc = probe.uk_bench_probe_mmt4d_launch(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), 512, 512, 1024,
                                                       8, 8, 4, staggered, stream)
                if rc != 0:
                    raise RuntimeError("timeline probe failed: HIP error %d" % rc)
            ms, _ = _time_launches(torch, launch, 50, 5)
            totals[staggered] += ms / 4
    res["staggered_tail"]["launch_us_back_to_back"] = round(totals[1] * 1e3, 2)
    res["all_stores_after_the_loop"]["launch_us_back_to_back"] = round(totals[0] * 1e3, 2)
    res["what"] = ("s8s8s32 4096^3 tiles 8x8x4; 100 MHz counter read by wavefront 0 of each of the 256 workgroups, last of "
                   "five back-to-back launches, averaged over ten such groups after 400 warm-up launches; medians over the "
                   "workgroups. launch_us_back_to_back: the same two kernels timed by events, alternating, 4 x 50 launches")
    return res


def _e2e_chain(torch, lib, abi, synth, steps, warmup):
    """The chain the reference's matmul benchmark runs (tools/e2e_matmul_benchmark.c:173-186):
    pack lhs, pack rhs (given as [K, N], both transposes), mmt4d, unpack, on row-major int8
    4096x4096 operands, with the tile sizes iree_uk_query_tile_sizes_2d hands out. One step =
    the four calls; checked against the sum of the row-major product (column sums of A times
    row sums of B)."""
    def tiles(role):
        q, o = abi.QueryTileSizes2dParams(), abi.QueryTileSizes2dOutParams()
        q.flags = abi.QTS_OP_MATMUL_I8I8I32 | role
        lib.iree_uk_query_tile_sizes_2d(C.byref(q), C.byref(o))
        return o.tile_size0, o.tile_size1
    (m0, k0), (n0, _) = tiles(abi.QTS_ROLE_LHS), tiles(abi.QTS_ROLE_RHS)
    S = 4096
    a = torch.from_numpy(synth.uniform_int8(21, 0, S * S)).cuda()      # A [M, K]
    b = torch.from_numpy(synth.uniform_int8(21, 1, S * S)).cuda()      # B [K, N]
    M1, N1, K1 = S // m0, S // n0, S // k0
    a4, b4 = torch.empty_like(a), torch.empty_like(b)
    c4 = torch.empty(S * S, dtype=torch.int32, device="cuda")
    c = torch.empty(S * S, dtype=torch.int32, device="cuda")

    def pack(src, dst, rows, cols, o0, o1, t0, t1, flags):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src.data_ptr(), dst.data_ptr()
        p.in_stride0, p.in_stride1, p.in_size0, p.in_size1 = cols, 1, rows, cols
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = o0, o1, t0, t1
        p.out_stride0, p.out_stride1 = o1 * t0 * t1, t0 * t1
        p.flags = abi.PACK_TYPE_I8I8 | flags
        return p
    p_lhs = pack(a, a4, S, S, M1, K1, m0, k0, 0)
    p_rhs = pack(b, b4, S, S, N1, K1, n0, k0, abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER)
    p_mm = _mmt4d_params(abi, a4.data_ptr(), b4.data_ptr(), c4.data_ptr(), M1, N1, K1, m0, n0, k0,
                         abi.MMT4D_TYPE_S8S8S32)
    u = abi.UnpackParams()
    u.in_buffer, u.out_buffer = c4.data_ptr(), c.data_ptr()
    u.in_size0, u.in_size1, u.in_size2, u.in_size3 = M1, N1, m0, n0
    u.in_stride0, u.in_stride1 = N1 * m0 * n0, m0 * n0
    u.out_size0, u.out_size1, u.out_stride0, u.out_stride1 = S, S, S, 1
    u.flags = abi.UNPACK_TYPE_I32I32
    parts = {}

    def timed(name, fn):
        ms, _ = _time_launches(torch, fn, steps, warmup)
        parts[name] = {"ms": round(ms, 5), "kernel": lib.iree_uk_mi355x_last_kernel().decode()}
    timed("pack_lhs", lambda: lib.iree_uk_pack_p(C.byref(p_lhs)))
    timed("pack_rhs_transposed", lambda: lib.iree_uk_pack_p(C.byref(p_rhs)))
    timed("mmt4d", lambda: lib.iree_uk_mmt4d_p(C.byref(p_mm)))
    timed("unpack", lambda: lib.iree_uk_unpack_p(C.byref(u)))

    def chain():
        lib.iree_uk_pack_p(C.byref(p_lhs))
        lib.iree_uk_pack_p(C.byref(p_rhs))
        lib.iree_uk_mmt4d_p(C.byref(p_mm))
        lib.iree_uk_unpack_p(C.byref(u))
    ms, _ = _time_launches(torch, chain, steps, warmup)
    want = (a.view(S, S).to(torch.int64).sum(dim=0) * b.view(S, S).to(torch.int64).sum(dim=1)).sum().item()
    rows = [0, 1777, 4095]
    ref_rows = (a.view(S, S)[rows].double() @ b.view(S, S).double()).long()
    ok = bool(c.to(torch.int64).sum().item() == want) and bool(torch.equal(c.view(S, S)[rows].long(), ref_rows))

    # The fused form: a row-major [M, K] matrix is the mmt4d lhs [M][K1][1][K0] as it stands, and the
    # result [M][N1][1][N0] is the row-major [M, N] matrix, so with tiles one row tall only the rhs
    # is packed: two launches instead of four, no packed copy of the lhs or of the result.
    c_fused = torch.empty(S * S, dtype=torch.int32, device="cuda")
    p_rm = _mmt4d_params(abi, a.data_ptr(), b4.data_ptr(), c_fused.data_ptr(), S, N1, K1, 1, n0, k0,
                         abi.MMT4D_TYPE_S8S8S32)
    timed("mmt4d_row_major_lhs_and_result", lambda: lib.iree_uk_mmt4d_p(C.byref(p_rm)))

    def fused():
        lib.iree_uk_pack_p(C.byref(p_rhs))
        lib.iree_uk_mmt4d_p(C.byref(p_rm))
    fused_ms, _ = _time_launches(torch, fused, steps, warmup)
    fused_ok = bool(torch.equal(c_fused, c))
    return {"tiles": "%dx%dx%d" % (m0, n0, k0), "ms": round(ms, 5), "value": round(2.0 * S ** 3 / ms / 1e9, 1),
            "unit": "TOP/s", "frac_of_peak": round(2.0 * S ** 3 / ms / 1e9 / PEAK_INT8_TOPS, 4),
            "equals_row_major_product": ok, "parts": parts,
            "fused_row_major_lhs_and_result": {
                "what": "pack rhs, then mmt4d with tiles 1x%dx%d reading the row-major lhs and writing the "
                        "row-major result (no pack of the lhs, no unpack)" % (n0, k0),
                "ms": round(fused_ms, 5), "value": round(2.0 * S ** 3 / fused_ms / 1e9, 1), "unit": "TOP/s",
                "frac_of_peak": round(2.0 * S ** 3 / fused_ms / 1e9 / PEAK_INT8_TOPS, 4),
                "equals_unfused_result": fused_ok}}


def _also(torch, lib, abi, synth, steps, warmup):
    """One-launch figures for the other configurations."""
    import numpy as np
    from iree_amd import library
    res = {}

    def mm(name, flags, M, N, K, M0, N0, K0, lhs, rhs, out_dtype, peak, unit, acc=False, bytes_model=None):
        out = torch.zeros(M * N * M0 * N0, dtype=out_dtype, device="cuda")
        p = _mmt4d_params(abi, lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0,
                          flags | (abi.MMT4D_ACCUMULATE if acc else 0))
        ms, _ = _time_launches(torch, lambda: lib.iree_uk_mmt4d_p(C.byref(p)), steps, warmup)
        ops = 2.0 * M * N * K * M0 * N0 * K0
        entry = {"kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5)}
        if bytes_model is None:
            entry.update({"value": round(ops / ms / 1e9, 1), "unit": unit,
                          "frac_of_peak": round(ops / ms / 1e9 / peak, 4)})
        else:
            entry.update({"value": round(bytes_model / ms / 1e6, 1), "unit": "GB/s",
                          "frac_of_peak": round(bytes_model / ms / 1e6 / PEAK_HBM_GBS, 4),
                          "gflops": round(ops / ms / 1e6, 1)})
        res[name] = entry

    def f16_operand(seed, stream, n, sigma, bf16=False):
        x = synth.normal_f32(seed, stream, n, sigma)
        bits = synth.bf16_bits(x) if bf16 else synth.f16_bits(x)
        return torch.from_numpy(bits.view(np.int16)).cuda()

    # f16f16f32 4096^3, tiles 16x16x16, accumulate on.
    n = 4096 * 4096
    mm("mmt4d_f16f16f32_4096_16x16x16_acc", abi.MMT4D_TYPE_F16F16F32, 256, 256, 256, 16, 16, 16,
       f16_operand(3, 0, n, 1.0 / 64), f16_operand(3, 1, n, 1.0 / 64), torch.float32,
       PEAK_F16_TFLOPS, "TFLOP/s", acc=True)
    # 4096^3 in the tile shapes an x86-64 caller passes (mmt4d_x86_64_tiles.inl): 2-byte row pieces for int8 with
    # VNNI and for f16, 4-byte for bf16; operands of the same distributions as above.
    xl, xr = torch.from_numpy(synth.uniform_int8(0, 0, n)).cuda(), torch.from_numpy(synth.uniform_int8(0, 1, n)).cuda()
    mm("mmt4d_s8s8s32_4096_x86_tile_16x16x2", abi.MMT4D_TYPE_S8S8S32, 256, 256, 2048, 16, 16, 2, xl, xr, torch.int32,
       PEAK_INT8_TOPS, "TOP/s")
    del xl, xr
    mm("mmt4d_f16f16f32_4096_x86_tile_16x16x1", abi.MMT4D_TYPE_F16F16F32, 256, 256, 4096, 16, 16, 1,
       f16_operand(3, 0, n, 1.0 / 64), f16_operand(3, 1, n, 1.0 / 64), torch.float32, PEAK_F16_TFLOPS, "TFLOP/s")
    mm("mmt4d_bf16bf16f32_4096_x86_tile_16x16x2", abi.MMT4D_TYPE_BF16BF16F32, 256, 256, 2048, 16, 16, 2,
       f16_operand(4, 0, n, 1.0, bf16=True), f16_operand(4, 10, n, 0.02, bf16=True), torch.float32, PEAK_F16_TFLOPS,
       "TFLOP/s")
    # The headline problem once more with all-zero operands: same kernel, same
    # instruction stream, same memory traffic. The part sustains a higher clock
    # when the data does not toggle, which is what the difference to the headline
    # (uniformly random int8) shows; it is not a result.
    zl = torch.zeros(n, dtype=torch.int8, device="cuda")
    mm("mmt4d_s8s8s32_4096_8x8x4_all_zero_operands_clock_check", abi.MMT4D_TYPE_S8S8S32, 512, 512, 1024, 8, 8, 4,
       zl, zl, torch.int32, PEAK_INT8_TOPS, "TOP/s")
    del zl
    # A second opinion on what this part does on this problem: the vendor's own
    # int8 GEMM (torch._int_mm -> hipBLASLt) on the same logical 4096^3 with
    # uniformly random int8, row-major operands. Not a result of this library.
    try:
        va = torch.from_numpy(synth.uniform_int8(0, 0, n)).cuda().view(4096, 4096)
        vb = torch.from_numpy(synth.uniform_int8(0, 1, n)).cuda().view(4096, 4096)
        best = None
        for operand in (vb, vb.t()):
            ms, _ = _time_launches(torch, lambda: torch._int_mm(va, operand), steps, warmup)
            best = ms if best is None else min(best, ms)
        res["vendor_library_int8_gemm_4096_for_comparison"] = {
            "what": "torch._int_mm (hipBLASLt), best of B and B^T layouts", "ms": round(best, 5),
            "value": round(2.0 * 4096 ** 3 / best / 1e9, 1), "unit": "TOP/s",
            "frac_of_peak": round(2.0 * 4096 ** 3 / best / 1e9 / PEAK_INT8_TOPS, 4)}
        del va, vb
    except Exception as exc:  # not every torch build has it
        res["vendor_library_int8_gemm_4096_for_comparison"] = {"unavailable": str(exc)[:200]}
    # The same for the f16 configuration's operands (f16 output there, f32 here).
    try:
        ha = f16_operand(3, 0, n, 1.0 / 64).view(torch.float16).view(4096, 4096)
        hb = f16_operand(3, 1, n, 1.0 / 64).view(torch.float16).view(4096, 4096)
        best = None
        for operand in (hb, hb.t()):
            ms, _ = _time_launches(torch, lambda: torch.matmul(ha, operand), steps, warmup)
            best = ms if best is None else min(best, ms)
        res["vendor_library_f16_gemm_4096_for_comparison"] = {
            "what": "torch.matmul on f16 (f16 result, no accumulate input), best of B and B^T layouts",
            "ms": round(best, 5), "value": round(2.0 * 4096 ** 3 / best / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_peak": round(2.0 * 4096 ** 3 / best / 1e9 / PEAK_F16_TFLOPS, 4)}
        # The like-for-like figure: the same product with an f32 result, which is what mmt4d writes (64 MiB
        # instead of 32).
        try:
            best = None
            for operand in (hb, hb.t()):
                ms, _ = _time_launches(torch, lambda: torch.mm(ha, operand, out_dtype=torch.float32), steps, warmup)
                best = ms if best is None else min(best, ms)
            res["vendor_library_f16_gemm_f32_result_4096_for_comparison"] = {
                "what": "torch.mm on f16 with out_dtype=float32 (no accumulate input), best of B and B^T layouts",
                "ms": round(best, 5), "value": round(2.0 * 4096 ** 3 / best / 1e9, 1), "unit": "TFLOP/s",
                "frac_of_peak": round(2.0 * 4096 ** 3 / best / 1e9 / PEAK_F16_TFLOPS, 4)}
        except Exception as exc:
            res["vendor_library_f16_gemm_f32_result_4096_for_comparison"] = {"unavailable": str(exc)[:200]}
        del ha, hb
    except Exception as exc:
        res["vendor_library_f16_gemm_4096_for_comparison"] = {"unavailable": str(exc)[:200]}
    res["e2e_pack_mmt4d_unpack_s8s8s32_4096"] = _e2e_chain(torch, lib, abi, synth, steps, warmup)
    res["mmt4d_s8s8s32_4096_in_kernel_timeline"] = _in_kernel_timeline(torch, synth)
    # What the matrix pipe sustains on this device, measured by the
    # benchmark's probe (a helper library of its own): the 256x256 kernel's inner-loop instruction mix with no
    # HBM traffic, no prologue and no epilogue, on all-zero bytes, on the
    # headline's uniformly random int8 and on the f16 / bf16 configurations'
    # operands, without and with the loop's LDS reads, loads to LDS and barrier.
    # A ceiling to read the mmt4d figures against, not a result: the cycle count
    # per step is the same in all of them, the clock is not.
    probe = {}
    rnd = torch.from_numpy(synth.uniform_int8(0, 0, 2 << 20)).cuda()
    zer = torch.zeros(2 << 20, dtype=torch.int8, device="cuda")
    f16 = f16_operand(3, 0, 1 << 20, 1.0 / 64)              # the f16 configuration's operand distribution
    bf16 = f16_operand(4, 10, 1 << 20, 0.02, bf16=True)     # the bf16 configuration's weights
    for type_flag, peak, unit, data_name, buf in (
            (abi.MMT4D_TYPE_S8S8S32, PEAK_INT8_TOPS, "TOP/s", "int8_zero_bytes", zer),
            (abi.MMT4D_TYPE_S8S8S32, PEAK_INT8_TOPS, "TOP/s", "int8_uniform_random", rnd),
            (abi.MMT4D_TYPE_F16F16F32, PEAK_F16_TFLOPS, "TFLOP/s", "f16_normal_over_64", f16),
            (abi.MMT4D_TYPE_BF16BF16F32, PEAK_F16_TFLOPS, "TFLOP/s", "bf16_normal_sigma_0.02", bf16)):
        for traffic in (0, 1):
            tops, mhz = C.c_double(), C.c_double()
            rc = library.load_bench_probe().uk_bench_probe_matrix_pipe(type_flag, buf.data_ptr(), buf.numel() * buf.element_size(),
                                                      traffic, 4096, C.byref(tops), C.byref(mhz))
            if rc != 0:
                raise RuntimeError("matrix pipe probe failed: HIP error %d" % rc)
            probe["%s_%s" % (data_name, "with_lds_traffic" if traffic else "mfma_only")] = {
                "value": round(tops.value, 1), "unit": unit, "frac_of_peak": round(tops.value / peak, 4),
                "shader_mhz": round(mhz.value)}
    res["matrix_pipe_sustained_rate_probe"] = probe
    del rnd, zer, f16, bf16
    # f32f32f32 4096^3 with the tile shape query_tile_sizes hands out for f32 (16x16x4).
    mm("mmt4d_f32f32f32_4096_16x16x4", abi.MMT4D_TYPE_F32F32F32, 256, 256, 1024, 16, 16, 4,
       torch.from_numpy(synth.normal_f32(6, 0, n, 1.0)).cuda(), torch.from_numpy(synth.normal_f32(6, 1, n, 1.0)).cuda(),
       torch.float32, PEAK_F32_TFLOPS, "TFLOP/s")
    # The in-dispatch int8 microkernel (16x16x64 MFMA, data-tiled operands of the
    # GPU backend's layout) over a 16 x 16 grid of 256x256 tiles, K = 4096; it
    # accumulates into C, which is therefore read and written.
    ta = torch.from_numpy(synth.uniform_int8(7, 0, n)).cuda()
    tb = torch.from_numpy(synth.uniform_int8(7, 1, n)).cuda()
    tc = torch.zeros(n, dtype=torch.int32, device="cuda")
    ms, _ = _time_launches(torch, lambda: lib.iree_uk_mi355x_multi_mma_i32_16x16x64_i8(
        ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), 16, 16, 64, 8, 2, 8, 2, 1), steps, warmup)
    res["multi_mma_i32_16x16x64_i8_4096_device_ukernel"] = {
        "kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
        "value": round(2.0 * 4096 ** 3 / ms / 1e9, 1), "unit": "TOP/s",
        "frac_of_peak": round(2.0 * 4096 ** 3 / ms / 1e9 / PEAK_INT8_TOPS, 4)}
    # The same product as a 32 x 32 grid of 128x128 tiles (4 x 4 intrinsics per subgroup, 2 x 2 subgroups): several
    # workgroups per compute unit.
    ms, _ = _time_launches(torch, lambda: lib.iree_uk_mi355x_multi_mma_i32_16x16x64_i8(
        ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), 32, 32, 64, 4, 2, 4, 2, 1), steps, warmup)
    res["multi_mma_i32_16x16x64_i8_4096_device_ukernel_128x128_tiles"] = {
        "kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
        "value": round(2.0 * 4096 ** 3 / ms / 1e9, 1), "unit": "TOP/s",
        "frac_of_peak": round(2.0 * 4096 ** 3 / ms / 1e9 / PEAK_INT8_TOPS, 4)}
    del ta, tb, tc
    # s8s4s32 512 x 11008 x 4096, tiles 16x16x32.
    lhs = torch.from_numpy(synth.uniform_int8(5, 0, 512 * 4096)).cuda()
    rhs = torch.from_numpy(synth.uniform_int4_packed(5, 1, 11008 * 4096).view(np.int8)).cuda()
    mm("mmt4d_s8s4s32_512x11008x4096_16x16x32", abi.MMT4D_TYPE_S8S4S32, 32, 688, 128, 16, 16, 32,
       lhs, rhs, torch.int32, PEAK_INT8_TOPS, "TOP/s")
    # bf16 skinny shapes: M0 in {1, 4, 16}, N = 14336, K = 4096; HBM-bound on the
    # rhs. Three rhs copies are rotated so the 256 MB last-level cache cannot
    # serve them. (The HBM-bound rows are timed over at least 30 launches: theirs
    # take 20 to 100 us each, and the mean of a handful moves by 2-3 %.)
    nk = 14336 * 4096
    rhs_set = [f16_operand(4, 10 + i, nk, 0.02, bf16=True) for i in range(3)]
    for m0 in (1, 4, 16):
        lhs = f16_operand(4, m0, m0 * 4096, 1.0, bf16=True)
        outs = torch.zeros(896 * m0 * 16, dtype=torch.float32, device="cuda")
        ps = [_mmt4d_params(abi, lhs.data_ptr(), r.data_ptr(), outs.data_ptr(), 1, 896, 512, m0, 16, 8,
                            abi.MMT4D_TYPE_BF16BF16F32) for r in rhs_set]
        state = {"i": 0}

        def step():
            lib.iree_uk_mmt4d_p(C.byref(ps[state["i"] % 3]))
            state["i"] += 1
        ms, _ = _time_launches(torch, step, max(steps, 30), warmup)
        nbytes = nk * 2 + m0 * 4096 * 2 + 896 * 16 * m0 * 4
        res["mmt4d_bf16_skinny_M%d_N14336_K4096" % m0] = {
            "kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
            "value": round(nbytes / ms / 1e6, 1), "unit": "GB/s",
            "frac_of_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
    # The same rhs bytes read as the narrow tiles an x86-64 target picks for a
    # matrix-vector product (bf16 1x16x2, mmt4d_x86_64_tiles.inl): 4-byte row
    # pieces, which no MFMA operand can be loaded from directly.
    lhs = f16_operand(4, 1, 4096, 1.0, bf16=True)
    outs = torch.zeros(896 * 16, dtype=torch.float32, device="cuda")
    ps = [_mmt4d_params(abi, lhs.data_ptr(), r.data_ptr(), outs.data_ptr(), 1, 896, 2048, 1, 16, 2,
                        abi.MMT4D_TYPE_BF16BF16F32) for r in rhs_set]
    state = {"i": 0}

    def step_narrow():
        lib.iree_uk_mmt4d_p(C.byref(ps[state["i"] % 3]))
        state["i"] += 1
    ms, _ = _time_launches(torch, step_narrow, max(steps, 30), warmup)
    nbytes = nk * 2 + 4096 * 2 + 896 * 16 * 4
    res["mmt4d_bf16_skinny_x86_tile_1x16x2_N14336_K4096"] = {
        "kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
        "value": round(nbytes / ms / 1e6, 1), "unit": "GB/s", "frac_of_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
    del rhs_set

    # The same with int4 weights (s8s4s32, tiles M0 x 16 x 32): N = 28672,
    # K = 8192, 117 MB of nibbles per rhs copy, three copies rotated. The
    # checksum of the M0 = 16 result is compared with torch's on the widened
    # weights.
    n_i4, k_i4 = 28672, 8192
    rhs_i4 = [torch.from_numpy(synth.uniform_int4_packed(12, i, n_i4 * k_i4).view(np.int8)).cuda() for i in range(3)]
    for m0 in (1, 16):
        lhs = torch.from_numpy(synth.uniform_int8(12, 10 + m0, m0 * k_i4)).cuda()
        outs = torch.zeros((n_i4 // 16) * m0 * 16, dtype=torch.int32, device="cuda")
        ps = [_mmt4d_params(abi, lhs.data_ptr(), r.data_ptr(), outs.data_ptr(), 1, n_i4 // 16, k_i4 // 32, m0, 16, 32,
                            abi.MMT4D_TYPE_S8S4S32) for r in rhs_i4]
        state = {"i": 0}

        def step_i4():
            lib.iree_uk_mmt4d_p(C.byref(ps[state["i"] % 3]))
            state["i"] += 1
        ms, _ = _time_launches(torch, step_i4, max(steps, 30), warmup)
        nbytes = n_i4 * k_i4 // 2 + m0 * k_i4 + n_i4 * m0 * 4
        entry = {"kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
                 "value": round(nbytes / ms / 1e6, 1), "unit": "GB/s",
                 "frac_of_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
        if m0 == 16:
            lib.iree_uk_mmt4d_p(C.byref(ps[0]))
            torch.cuda.synchronize()
            r = rhs_i4[0].to(torch.int16)
            w = torch.stack([r & 0xF, (r >> 4) & 0xF], dim=1).reshape(-1)
            w = ((w ^ 8) - 8).to(torch.float64).view(n_i4 // 16, k_i4 // 32, 16, 32)
            a = lhs.view(k_i4 // 32, 16, 32).to(torch.float64)
            # sum over all outputs = sum_k (column sums of a) * (column sums of w), exact in float64
            want = (a.sum(dim=1) * w.sum(dim=(0, 2))).sum().item()
            entry["checksum_verified"] = bool(outs.to(torch.float64).sum().item() == want)
            del r, w, a
        res["mmt4d_s8s4s32_skinny_M%d_N28672_K8192" % m0] = entry
    # The same 117 MB per copy read as int8 weights in the x86-64 VNNI matrix-vector tiles (s8s8s32 1x16x2):
    # N = 28672, K = 4096. Checked through the sum of all outputs, as above.
    lhs = torch.from_numpy(synth.uniform_int8(12, 30, 4096)).cuda()
    outs = torch.zeros(n_i4, dtype=torch.int32, device="cuda")
    ps = [_mmt4d_params(abi, lhs.data_ptr(), r.data_ptr(), outs.data_ptr(), 1, n_i4 // 16, 2048, 1, 16, 2,
                        abi.MMT4D_TYPE_S8S8S32) for r in rhs_i4]
    state = {"i": 0}

    def step_vnni():
        lib.iree_uk_mmt4d_p(C.byref(ps[state["i"] % 3]))
        state["i"] += 1
    ms, _ = _time_launches(torch, step_vnni, max(steps, 30), warmup)
    nbytes = n_i4 * 4096 + 4096 + n_i4 * 4
    entry = {"kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
             "value": round(nbytes / ms / 1e6, 1), "unit": "GB/s", "frac_of_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
    lib.iree_uk_mmt4d_p(C.byref(ps[0]))
    torch.cuda.synchronize()
    w = rhs_i4[0].view(n_i4 // 16, 2048, 16, 2).to(torch.float64)
    want = (lhs.view(2048, 2).to(torch.float64) * w.sum(dim=(0, 2))).sum().item()
    entry["checksum_verified"] = bool(outs.to(torch.float64).sum().item() == want)
    del w
    res["mmt4d_s8s8s32_skinny_x86_tile_1x16x2_N28672_K4096"] = entry
    del rhs_i4

    # pack / unpack f32 [8191, 8190] <-> [512, 8190, 16, 1]; two buffer sets rotated
    # (each set is 537 MB, beyond the last-level cache).
    R, Cc = 8191, 8190
    src = [torch.from_numpy(synth.normal_f32(2, i, R * Cc)).cuda() for i in range(2)]
    packed = [torch.empty(512 * Cc * 16, dtype=torch.float32, device="cuda") for _ in range(2)]
    back = [torch.empty(R * Cc, dtype=torch.float32, device="cuda") for _ in range(2)]

    def pack_params(i, flags, o0, o1, t0, t1):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src[i].data_ptr(), packed[i].data_ptr()
        p.in_stride0, p.in_stride1 = Cc, 1
        p.out_stride0, p.out_stride1 = o1 * t0 * t1, t0 * t1
        p.in_size0, p.in_size1 = R, Cc
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = o0, o1, t0, t1
        p.padding_value = 0
        p.flags = abi.PACK_TYPE_F32F32 | flags
        return p

    def timed_pair(name, make, nbytes):
        ps = [make(0), make(1)]
        state = {"i": 0}

        def step():
            fn, p = ps[state["i"] & 1]
            fn(C.byref(p))
            state["i"] += 1
        ms, _ = _time_launches(torch, step, max(steps, 30), warmup)
        res[name] = {"kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
                     "value": round(nbytes / ms / 1e6, 1), "unit": "GB/s",
                     "frac_of_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}

    timed_pair("pack_f32_8191x8190_to_512x8190x16x1",
               lambda i: (lib.iree_uk_pack_p, pack_params(i, 0, 512, Cc, 16, 1)),
               (R * Cc + 512 * Cc * 16) * 4)
    # "Transposed-inner" variant: same out sizes (.., 16, 1) with TRANSPOSE_INNER,
    # i.e. 1x16 tiles along dim 1: out [8191, 512, 16, 1].
    packed2 = [torch.empty(R * 512 * 16, dtype=torch.float32, device="cuda") for _ in range(2)]

    def pack_tr(i):
        p = pack_params(i, abi.PACK_TRANSPOSE_INNER, R, 512, 16, 1)
        p.out_buffer = packed2[i].data_ptr()
        return (lib.iree_uk_pack_p, p)
    timed_pair("pack_f32_8191x8190_transpose_inner_to_8191x512x16x1", pack_tr,
               (R * Cc + R * 512 * 16) * 4)
    del packed2
    # The form the rhs of a matmul is packed in: both transposes, out [512, 8191, 16, 1]
    # from the [8191, 8190] source read as its transpose.
    packed3 = [torch.empty(512 * R * 16, dtype=torch.float32, device="cuda") for _ in range(2)]

    def pack_rhs(i):
        p = pack_params(i, abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER, 512, R, 16, 1)
        p.out_buffer = packed3[i].data_ptr()
        return (lib.iree_uk_pack_p, p)
    timed_pair("pack_f32_8191x8190_transpose_both_to_512x8191x16x1", pack_rhs, (R * Cc + 512 * R * 16) * 4)
    del packed3

    # Every second element of each row (in_stride1 = 2, as the reference's tests draw it,
    # tools/pack_test.c:80-93): [8191, 4095] out of the same buffers into [512, 4095, 16, 1]. Counted are the
    # elements read and written; the lines fetched hold twice the elements read.
    def pack_strided(i):
        p = pack_params(i, 0, 512, Cc // 2, 16, 1)
        p.in_stride1, p.in_size1 = 2, Cc // 2
        return (lib.iree_uk_pack_p, p)
    timed_pair("pack_f32_8191x4095_element_stride_2_to_512x4095x16x1", pack_strided,
               (R * (Cc // 2) + 512 * (Cc // 2) * 16) * 4)

    def unpack_params(i):
        p = abi.UnpackParams()
        p.in_buffer, p.out_buffer = packed[i].data_ptr(), back[i].data_ptr()
        p.in_stride0, p.in_stride1 = Cc * 16, 16
        p.out_stride0, p.out_stride1 = Cc, 1
        p.in_size0, p.in_size1, p.in_size2, p.in_size3 = 512, Cc, 16, 1
        p.out_size0, p.out_size1 = R, Cc
        p.flags = abi.UNPACK_TYPE_F32F32
        return (lib.iree_uk_unpack_p, p)
    # Make sure `packed` holds packed data for both sets, then time unpack.
    for i in range(2):
        lib.iree_uk_pack_p(C.byref(pack_params(i, 0, 512, Cc, 16, 1)))
    timed_pair("unpack_f32_512x8190x16x1_to_8191x8190", unpack_params, 2 * R * Cc * 4)
    torch.cuda.synchronize()
    res["pack_unpack_round_trip_bit_exact"] = bool(all(torch.equal(src[i], back[i]) for i in range(2)))
    # What this device does on the same bytes with no rearrangement at all: the
    # framework's device-to-device copy of the [8191, 8190] f32 matrix, same two
    # buffer sets rotated. A ceiling to read the pack / unpack rows against, not a
    # result of this library.
    copy_state = {"i": 0}

    def copy_step():
        i = copy_state["i"] & 1
        back[i].copy_(src[i])
        copy_state["i"] += 1
    ms, _ = _time_launches(torch, copy_step, max(steps, 30), warmup)
    res["plain_device_copy_f32_8191x8190_for_comparison"] = {
        "what": "torch.Tensor.copy_ of the same matrix (read + write counted)", "ms": round(ms, 5),
        "value": round(2 * R * Cc * 4 / ms / 1e6, 1), "unit": "GB/s",
        "frac_of_peak": round(2 * R * Cc * 4 / ms / 1e6 / PEAK_HBM_GBS, 4)}
    # What the device streams with plain kernels and nothing else to do (the
    # benchmark's own probe, csrc/bench/probe_hbm_stream.hip: 16 bytes per lane, read
    # only / write only / copy, best of a few launch shapes), over the same two
    # buffer sets. The GB/s rows of this library are reported against these as well
    # (`of_stream_ceiling`): against the copy for pack and unpack, against the
    # read-only stream for the matrix-vector kernels.
    probe_lib = library.load_bench_probe()
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    stream_bytes = R * Cc * 4 // 16 * 16
    # (vectors in flight per thread, workgroups (0: one pass), blocks an XCD takes at a time, workgroups resident
    # per compute unit (0: as many as fit))
    STREAM_SHAPES = ((4, 0, 1, 0), (8, 0, 1, 0), (4, 4096, 1, 0), (8, 2048, 1, 0), (4, 0, 64, 0), (4, 0, 16, 0),
                     (8, 0, 32, 0), (4, 0, 64, 5), (4, 0, 1, 5), (4, 0, 64, 4), (8, 0, 32, 3), (1, 0, 1, 0), (1, 0, 64, 0),
                     (1, 0, 1, 5), (2, 0, 1, 6), (2, 0, 64, 5), (2, 0, 1, 3))
    ceilings = {}
    for mode, mode_name in ((0, "read_only"), (1, "write_only"), (2, "copy")):
        best = None
        for unroll, grid, xcd_group, resident in STREAM_SHAPES:
            st = {"i": 0}

            def stream_step():
                i = st["i"] & 1
                rc = probe_lib.uk_bench_probe_hbm_stream(mode, back[i].data_ptr(), src[i].data_ptr(), stream_bytes, grid,
                                                         unroll, 1, xcd_group, resident, sink.data_ptr(),
                                                         torch.cuda.current_stream().cuda_stream)
                if rc != 0:
                    raise RuntimeError("hbm stream probe failed: HIP error %d" % rc)
                st["i"] += 1
            ms, _ = _time_launches(torch, stream_step, max(steps, 30), warmup)
            best = ms if best is None else min(best, ms)
        moved = stream_bytes * (2 if mode == 2 else 1)
        ceilings[mode_name] = {"ms": round(best, 5), "value": round(moved / best / 1e6, 1), "unit": "GB/s",
                               "frac_of_peak": round(moved / best / 1e6 / PEAK_HBM_GBS, 4)}
    # The matrix-vector kernels stream 117 MB per launch (a launch of 19 us, of which start and end weigh more):
    # the read-only stream over that many bytes, same rotation.
    decode_bytes = 14336 * 4096 * 2
    best = None
    for unroll, grid, xcd_group, resident in STREAM_SHAPES:
        st = {"i": 0}

        def decode_stream_step():
            i = st["i"] & 1
            rc = probe_lib.uk_bench_probe_hbm_stream(0, back[i].data_ptr(), src[i].data_ptr(), decode_bytes, grid, unroll, 1,
                                                     xcd_group, resident, sink.data_ptr(),
                                                     torch.cuda.current_stream().cuda_stream)
            if rc != 0:
                raise RuntimeError("hbm stream probe failed: HIP error %d" % rc)
            st["i"] += 1
        ms, _ = _time_launches(torch, decode_stream_step, max(steps, 30), warmup)
        best = ms if best is None else min(best, ms)
    ceilings["read_only_117MB"] = {"ms": round(best, 5), "value": round(decode_bytes / best / 1e6, 1), "unit": "GB/s",
                                   "frac_of_peak": round(decode_bytes / best / 1e6 / PEAK_HBM_GBS, 4)}
    res["hbm_stream_ceiling"] = dict(
        ceilings, what="plain read / fill / copy kernels over %d bytes, non-temporal 16-byte accesses, "
                       "two buffer sets rotated; best of seventeen launch shapes each (4 to 32 KiB per workgroup, with and without blocks dealt to the XCDs in groups, with and without a limit on the workgroups resident per compute unit); read_only_117MB: the read-only stream over the %d "
                       "bytes of rhs a matrix-vector launch reads" % (stream_bytes, decode_bytes))
    del src, packed, back

    # int8 operands of a 16384^3 matmul into the layouts of the 16x16x64 tile:
    # lhs [16384, 16384] -> [1024, 256, 16, 64]; rhs [K=16384, N=16384] ->
    # [1024, 256, 16, 64] with both transposes (n-tile outermost, k innermost).
    # Three buffer sets (each 537 MB) rotated.
    n16 = 16384
    isrc = [torch.from_numpy(synth.uniform_int8(8, i, n16 * n16)).cuda() for i in range(3)]
    idst = [torch.empty(n16 * n16, dtype=torch.int8, device="cuda") for _ in range(3)]

    def pack_i8(i, flags, s2, s3):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = isrc[i].data_ptr(), idst[i].data_ptr()
        p.in_stride0, p.in_stride1 = n16, 1
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = 1024, 256, s2, s3
        p.out_stride0, p.out_stride1 = 256 * s2 * s3, s2 * s3
        p.in_size0, p.in_size1 = n16, n16
        p.padding_value = 0
        p.flags = abi.PACK_TYPE_I8I8 | flags
        return p

    def timed_three(name, flags):
        ps = [pack_i8(i, flags, 16, 64) for i in range(3)]
        state = {"i": 0}

        def step():
            lib.iree_uk_pack_p(C.byref(ps[state["i"] % 3]))
            state["i"] += 1
        ms, _ = _time_launches(torch, step, max(steps, 30), warmup)
        res[name] = {"kernel": lib.iree_uk_mi355x_last_kernel().decode(), "ms": round(ms, 5),
                     "value": round(2.0 * n16 * n16 / ms / 1e6, 1), "unit": "GB/s",
                     "frac_of_peak": round(2.0 * n16 * n16 / ms / 1e6 / PEAK_HBM_GBS, 4)}
    timed_three("pack_i8_16384x16384_lhs_to_1024x256x16x64", 0)
    timed_three("pack_i8_16384x16384_rhs_transpose_both_to_1024x256x16x64",
                abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER)
    # The rhs result against the same permutation done by torch.
    want = isrc[0].view(256, 64, 1024, 16).permute(2, 0, 3, 1).contiguous().view(-1)
    lib.iree_uk_pack_p(C.byref(pack_i8(0, abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER, 16, 64)))
    torch.cuda.synchronize()
    res["pack_i8_rhs_layout_bit_exact"] = bool(torch.equal(want, idst[0]))
    for name, entry in res.items():
        if isinstance(entry, dict) and entry.get("unit") == "GB/s" and "kernel" in entry:
            against = "copy" if name.startswith(("pack_", "unpack_")) else "read_only_117MB"
            entry["of_stream_ceiling"] = round(entry["value"] / ceilings[against]["value"], 4)
            entry["stream_ceiling"] = against
    return res


def _power_clock_samples(torch, lib, abi, synth, seconds):
    """Socket power and shader clocks (amd-smi, polled from a thread) while the headline
    kernel runs back to back for `seconds`: on its uniformly random int8, on all-zero
    operands (same instruction stream and traffic), and the vendor's int8 GEMM on the same
    logical problem. Shows what the part sustains on this data; not a result."""
    import subprocess
    import threading
    import numpy as np

    def poll(stop, out):
        while not stop.is_set():
            try:
                r = subprocess.run(["amd-smi", "metric", "-p", "-c", "--json"], stdout=subprocess.PIPE,
                                   stderr=subprocess.DEVNULL, text=True, timeout=10)
                d = json.loads(r.stdout)
                g = d[0] if isinstance(d, list) else d.get("gpu_data", [d])[0]
                value = lambda x: float(x["value"] if isinstance(x, dict) else x)
                clocks = [value(v["clk"]) for k, v in g["clock"].items() if k.startswith("gfx_")]
                out.append((value(g["power"]["socket_power"]), clocks))
            except Exception:  # tool missing or another output format: no samples
                time.sleep(0.5)

    def loop(name, fn, ops):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        stop, samples = threading.Event(), []
        th = threading.Thread(target=poll, args=(stop, samples))
        th.start()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0, launches = time.time(), 0
        e0.record()
        while time.time() - t0 < seconds:
            for _ in range(200):
                fn()
            launches += 200
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        stop.set()
        th.join()
        ms = e0.elapsed_time(e1) / launches
        samples = samples[1:] if len(samples) > 2 else samples   # the first may predate the loop
        power = [s[0] for s in samples]
        clock = [float(np.mean(s[1])) for s in samples if s[1]]
        return {"loop": name, "launches": launches, "ms_per_launch": round(ms, 5),
                "value": round(ops / ms / 1e9, 1), "unit": "TOP/s", "frac_of_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4),
                "samples": len(samples),
                "socket_power_W_mean": round(float(np.mean(power)), 1) if power else None,
                "socket_power_W_max": round(float(np.max(power)), 1) if power else None,
                "shader_clock_MHz_mean_over_xcds": round(float(np.mean(clock))) if clock else None,
                "shader_clock_MHz_min": round(float(np.min(clock))) if clock else None}

    n = 4096 * 4096
    ops = 2.0 * 4096 ** 3
    out = torch.empty(n, dtype=torch.int32, device="cuda")

    def headline_on(l, r):
        p = _mmt4d_params(abi, l.data_ptr(), r.data_ptr(), out.data_ptr(), 512, 512, 1024, 8, 8, 4, abi.MMT4D_TYPE_S8S8S32)
        return lambda: lib.iree_uk_mmt4d_p(C.byref(p))
    rl = torch.from_numpy(synth.uniform_int8(0, 0, n)).cuda()
    rr = torch.from_numpy(synth.uniform_int8(0, 1, n)).cuda()
    zeros = torch.zeros(n, dtype=torch.int8, device="cuda")
    rows = [loop("mmt4d s8s8s32 4096^3 8x8x4, uniform random int8 (the headline)", headline_on(rl, rr), ops),
            loop("the same launch on all-zero operands", headline_on(zeros, zeros), ops)]
    try:
        a2, b2 = rl.view(4096, 4096), rr.view(4096, 4096).t()
        rows.append(loop("torch._int_mm 4096^3 (hipBLASLt), uniform random int8", lambda: torch._int_mm(a2, b2), ops))
    except Exception:
        pass
    return rows


def _cpu_baseline(abi, synth, threads):
    """The reference CPU ukernels (compiled from the reference's own sources into
    oracle/_ref) on this host; falls back to this repository's scalar port."""
    import numpy as np
    import oracle
    ref = oracle.ref_lib()
    # Bounded sample of the headline workload: the first 64 of its 512 rows of
    # 8x8 tiles against all 512 rhs panels, full K (1/8 of the work).
    Ms, N, K, M0, N0, K0 = 64, 512, 1024, 8, 8, 4
    lhs = synth.uniform_int8(0, 0, 512 * K * M0 * K0)[:Ms * K * M0 * K0]
    rhs = synth.uniform_int8(0, 1, N * K * N0 * K0)
    out = np.zeros(Ms * N * M0 * N0, dtype=np.int32)
    cpu = oracle.host_cpu_data()
    p = _mmt4d_params(abi, lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data, Ms, N, K, M0, N0, K0,
                      abi.MMT4D_TYPE_S8S8S32 | abi.MMT4D_ALLOW_GENERIC_FALLBACK)
    p.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
    if ref is not None:
        run, kind = (lambda: ref.ref_mmt4d_mt(C.byref(p), threads)), "reference"
    else:
        run, kind = (lambda: oracle.lib().oracle_mmt4d_mt(C.byref(p), threads)), "port"
    best = None
    for _ in range(2):
        t0 = time.perf_counter()
        run()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    ops = 2.0 * Ms * N * K * M0 * N0 * K0
    base = {"value": round(ops / best / 1e12, 5), "unit": "TOP/s", "cores": threads, "kind": kind,
            "sample": "rows 0..63 of the 512 rows of 8x8 lhs tiles x all 512 rhs panels x full K "
                      "(1/8 of the headline workload), generic tile function (the reference has no "
                      "x86-64 tile for 8x8x4), best of 2"}
    extra = None
    if ref is not None:
        # The reference's architecture-specific tiles need its own tile shape:
        # s8s8s32 16x16x2 (AVX-512 VNNI where the host has it), same logical size.
        M, N, K, M0, N0, K0 = 256, 256, 2048, 16, 16, 2
        lhs = synth.uniform_int8(0, 0, M * K * M0 * K0)
        rhs = synth.uniform_int8(0, 1, N * K * N0 * K0)
        out = np.zeros(M * N * M0 * N0, dtype=np.int32)
        q = _mmt4d_params(abi, lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data, M, N, K, M0, N0, K0,
                          abi.MMT4D_TYPE_S8S8S32 | abi.MMT4D_ALLOW_GENERIC_FALLBACK)
        q.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
        has_arch = bool(ref.ref_mmt4d_info(C.byref(q)) & 1)
        best = None
        for _ in range(2):
            t0 = time.perf_counter()
            ref.ref_mmt4d_mt(C.byref(q), threads)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        extra = {"value": round(2.0 * 4096 ** 3 / best / 1e12, 5), "unit": "TOP/s", "cores": threads,
                 "kind": "reference",
                 "sample": "full 4096^3 in the reference's own x86-64 tile shape 16x16x2, "
                           "architecture-specific tile function %s, best of 2"
                           % ("selected" if has_arch else "NOT available on this host (generic used)")}
    return base, extra


def _cpu_baseline_other_configs(abi, synth, threads):
    """The compiled reference on this host for the other configurations, in the tile shapes of
    the configurations themselves (no x86-64 tile exists for any of them: generic tile
    functions, mmt4d_tile_generic.c) and in the reference's own x86-64 tile shapes
    (arch/x86_64/mmt4d_x86_64_tiles.inl). Each entry says whether the reference selected an
    architecture-specific tile function on this host. Bounded samples where the generic
    functions would take minutes."""
    import numpy as np
    import oracle
    ref = oracle.ref_lib()
    if ref is None:
        return None
    cpu = oracle.host_cpu_data()
    rows = {}

    def run(name, flags, M, N, K, M0, N0, K0, lhs, rhs, out, sample, unit="TFLOP/s", nbytes=None, reps=2):
        p = _mmt4d_params(abi, lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data, M, N, K, M0, N0, K0,
                          flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK)
        p.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
        arch = bool(ref.ref_mmt4d_info(C.byref(p)) & 1)
        best = None
        for _ in range(reps):
            t0 = time.perf_counter()
            ref.ref_mmt4d_mt(C.byref(p), threads)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        ops = 2.0 * M * N * K * M0 * N0 * K0
        entry = {"value": round(ops / best / 1e12, 5), "unit": unit, "cores": threads, "kind": "reference",
                 "arch_tile_selected": arch, "seconds": round(best, 4), "sample": sample}
        if nbytes is not None:
            entry.update({"value": round(nbytes / best / 1e9, 2), "unit": "GB/s", "gflops": round(ops / best / 1e9, 2)})
        rows[name] = entry

    def f16(seed, stream, n, sigma, bf16=False):
        x = synth.normal_f32(seed, stream, n, sigma)
        return synth.bf16_bits(x) if bf16 else synth.f16_bits(x)

    n = 4096 * 4096
    h_l, h_r = f16(3, 0, n, 1.0 / 64), f16(3, 1, n, 1.0 / 64)
    acc = synth.normal_f32(3, 2, n)
    # f16f16f32 4096^3 with accumulate: the reference's x86-64 shape 16x16x1 (whole problem) and the
    # configuration's own 16x16x16 (generic; 16 of its 256 rows of tiles).
    run("mmt4d_f16f16f32_4096_x86_tile_16x16x1_acc", abi.MMT4D_TYPE_F16F16F32 | abi.MMT4D_ACCUMULATE, 256, 256, 4096,
        16, 16, 1, h_l, h_r, acc.copy(), "whole 4096^3, best of 2")
    run("mmt4d_f16f16f32_4096_16x16x16_acc", abi.MMT4D_TYPE_F16F16F32 | abi.MMT4D_ACCUMULATE, 16, 256, 256, 16, 16, 16,
        h_l, h_r, acc.copy(), "rows 0..15 of the 256 rows of lhs tiles (1/16 of the workload), best of 1", reps=1)
    del h_l, h_r, acc
    b_l, b_r = f16(4, 0, n, 1.0, bf16=True), f16(4, 10, n, 0.02, bf16=True)
    run("mmt4d_bf16bf16f32_4096_x86_tile_16x16x2", abi.MMT4D_TYPE_BF16BF16F32, 256, 256, 2048, 16, 16, 2, b_l, b_r,
        np.zeros(n, np.float32), "whole 4096^3, best of 2")
    del b_l, b_r
    # bf16 matrix-vector shapes, N = 14336, K = 4096 (rhs panels split over the threads).
    nk = 14336 * 4096
    w = f16(4, 10, nk, 0.02, bf16=True)
    x1 = f16(4, 1, 4096, 1.0, bf16=True)
    run("mmt4d_bf16_skinny_x86_tile_1x16x2_N14336_K4096", abi.MMT4D_TYPE_BF16BF16F32, 1, 896, 2048, 1, 16, 2, x1, w,
        np.zeros(14336, np.float32), "whole workload, best of 3", nbytes=nk * 2 + 4096 * 2 + 14336 * 4, reps=3)
    for m0 in (1, 16):
        xm = f16(4, m0, m0 * 4096, 1.0, bf16=True)
        run("mmt4d_bf16_skinny_M%d_N14336_K4096_%dx16x8" % (m0, m0), abi.MMT4D_TYPE_BF16BF16F32, 1, 896 // 4, 512, m0, 16,
            8, xm, w, np.zeros(14336 * m0 // 4, np.float32),
            "the first 224 of the 896 rhs panels (1/4 of the workload), best of 1",
            nbytes=(nk * 2) // 4 + m0 * 4096 * 2 + 14336 * m0, reps=1)
    del w
    # s8s4s32 512 x 11008 x 4096, tiles 16x16x32: no architecture-specific tile in the reference.
    lhs = synth.uniform_int8(5, 0, 512 * 4096)
    rhs = synth.uniform_int4_packed(5, 1, 11008 * 4096)
    run("mmt4d_s8s4s32_512x11008x4096_16x16x32", abi.MMT4D_TYPE_S8S4S32, 32, 688 // 4, 128, 16, 16, 32, lhs,
        rhs.view(np.int8), np.zeros(512 * 11008 // 4, np.int32),
        "the first 172 of the 688 rhs panels (1/4 of the workload), best of 1", unit="TOP/s", reps=1)
    return rows


def _cpu_pack_unpack(abi, synth, threads):
    """The reference's pack and unpack on this host (f32 [8191, 8190] <-> [512, 8190, 16, 1],
    rows of tiles split over `threads`), GB/s counted like the GPU figures (read + written)."""
    import numpy as np
    import oracle
    ref = oracle.ref_lib()
    if ref is None:
        return None
    R, Cc = 8191, 8190
    src = synth.normal_f32(2, 0, R * Cc)
    packed = np.empty(512 * Cc * 16, dtype=np.float32)
    back = np.empty(R * Cc, dtype=np.float32)
    cpu = oracle.host_cpu_data()
    p = abi.PackParams()
    p.in_buffer, p.out_buffer = src.ctypes.data, packed.ctypes.data
    p.in_stride0, p.in_stride1, p.out_stride0, p.out_stride1 = Cc, 1, Cc * 16, 16
    p.in_size0, p.in_size1 = R, Cc
    p.out_size0, p.out_size1, p.out_size2, p.out_size3 = 512, Cc, 16, 1
    p.padding_value, p.flags = 0, abi.PACK_TYPE_F32F32
    p.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
    u = abi.UnpackParams()
    u.in_buffer, u.out_buffer = packed.ctypes.data, back.ctypes.data
    u.in_stride0, u.in_stride1, u.out_stride0, u.out_stride1 = Cc * 16, 16, Cc, 1
    u.in_size0, u.in_size1, u.in_size2, u.in_size3 = 512, Cc, 16, 1
    u.out_size0, u.out_size1, u.flags = R, Cc, abi.UNPACK_TYPE_F32F32
    u.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))

    def best_of(fn, n=3):
        best = None
        for _ in range(n):
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best
    t_pack = best_of(lambda: ref.ref_pack_mt(C.byref(p), threads))
    t_unpack = best_of(lambda: ref.ref_unpack_mt(C.byref(u), threads))
    return {"pack_f32_8191x8190_to_512x8190x16x1": {"value": round((R * Cc + 512 * Cc * 16) * 4 / t_pack / 1e9, 2),
                                                   "unit": "GB/s", "cores": threads, "kind": "reference"},
            "unpack_f32_512x8190x16x1_to_8191x8190": {"value": round(2 * R * Cc * 4 / t_unpack / 1e9, 2),
                                                      "unit": "GB/s", "cores": threads, "kind": "reference"},
            "round_trip_bit_exact": bool(np.array_equal(src, back)),
            "sample": "the whole workload, best of 3"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-also", action="store_true", help="headline workload only")
    ap.add_argument("--sample-power", type=float, default=0.0, metavar="SECONDS",
                    help="also loop the headline kernel for SECONDS per data set while polling amd-smi for "
                         "socket power and shader clocks (adds `power_clock_samples` to the line)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device-to-device copy three times (a kernel of "
                         "known traffic, to scale the profiler's FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this library runs on ONE GPU (a ukernel call has no cross-device "
                 "part); --gpus %d is not supported, use --gpus 1" % args.gpus)

    import torch
    from iree_amd import abi, library, synth
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    lib = library.load()  # raises if the HIP library is missing: no fallback
    rc = lib.iree_uk_mi355x_init(0)
    if rc != 0:
        sys.exit("bench.py: device 0 is not usable as a gfx950 part (code %d)" % rc)
    torch.cuda.set_device(0)
    lib.iree_uk_mi355x_set_stream(torch.cuda.current_stream().cuda_stream, 1)

    head = _headline(torch, lib, abi, synth, args.steps, args.warmup)
    sustained = _sustained_ceiling(torch, abi, synth)
    also = None if args.no_also else _also(torch, lib, abi, synth, max(6, args.steps // 5), 5)
    lib.iree_uk_mi355x_set_stream(None, 0)
    if also is not None:
        # The same call the way the reference's callers make it: host pointers,
        # synchronous (staged through device memory, PCIe-bound). Never `value`.
        import numpy as np
        lhs_h, rhs_h, out_d = (t.cpu().numpy() for t in head["keep"])
        out_h = np.empty_like(out_d)
        hp = _mmt4d_params(abi, lhs_h.ctypes.data, rhs_h.ctypes.data, out_h.ctypes.data, 512, 512, 1024, 8, 8, 4,
                           abi.MMT4D_TYPE_S8S8S32)
        lib.iree_uk_mmt4d_p(C.byref(hp))
        t0 = time.perf_counter()
        lib.iree_uk_mmt4d_p(C.byref(hp))
        also["mmt4d_s8s8s32_4096_host_pointers_synchronous"] = {
            "ms": round((time.perf_counter() - t0) * 1e3, 3), "bit_exact_vs_device_run": bool((out_h == out_d).all())}
    if args.calibrate_copy:
        a = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda").fill_(1)
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b

    threads = min(16, os.cpu_count() or 1)
    cpu, cpu_arch = (None, None) if args.no_cpu else _cpu_baseline(abi, synth, threads)

    tops = head["ops"] / head["ev_ms"] / 1e9
    line = {
        "metric": "mmt4d s8s8s32 throughput at logical 4096^3 on 1 MI355X",
        "value": round(head["ops"] / head["wall_ms"] / 1e9, 2),
        "unit": "TOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["wall_ms"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": head["workload"], "kernel": head["kernel"],
                   "checksum_verified": head["verified"]},
        "roofline": {"bound": "mfma", "achieved": round(tops, 2), "peak": PEAK_INT8_TOPS,
                     "unit": "TOP/s", "frac": round(tops / PEAK_INT8_TOPS, 4),
                     "traffic": HEADLINE_TRAFFIC_BYTES,
                     "traffic_source": "profiles/bench_all_workloads_hbm_traffic.txt (rocprofv3 FETCH_SIZE, "
                                       "WRITE_SIZE of this command, scaled by a plain copy; not measured in this run)",
                     # `achieved` = ops / this: the mean over the timed steps, launched back to back,
                     # between two HIP events on the launch stream.
                     "kernel_ms_mean_back_to_back": round(head["ev_ms"], 5),
                     # Each launch between its own pair of events (includes the events' own gaps).
                     "kernel_ms_single_launch_median": round(head["med_ms"], 5),
                     "kernel_ms_single_launch_min": round(head["min_ms"], 5),
                     # Not the roofline: what the instruction mix sustains on this data at the clock the
                     # part grants it, and `achieved` as a fraction of that.
                     "sustained_ceiling": dict(sustained, achieved_of_it=round(tops / sustained["value"], 4))},
        "cpu_baseline": cpu,
    }
    if cpu_arch is not None:
        line["cpu_baseline_arch_tiles"] = cpu_arch
    if not args.no_cpu and not args.no_also:
        cpu_pack = _cpu_pack_unpack(abi, synth, threads)
        if cpu_pack is not None:
            line["cpu_baseline_pack_unpack"] = cpu_pack
        cpu_other = _cpu_baseline_other_configs(abi, synth, threads)
        if cpu_other is not None:
            line["cpu_baseline_other_configs"] = cpu_other
    if also is not None:
        line["also"] = also
    if args.sample_power > 0:
        lib.iree_uk_mi355x_set_stream(torch.cuda.current_stream().cuda_stream, 1)
        line["power_clock_samples"] = _power_clock_samples(torch, lib, abi, synth, args.sample_power)
        lib.iree_uk_mi355x_set_stream(None, 0)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
