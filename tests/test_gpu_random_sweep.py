"""Seeded random sweeps through the C ABI against the oracle: shapes, tile
sizes, flags, strides with gaps and offsets drawn at random (fixed seeds), each
case compared over the WHOLE destination buffer (pre-filled, so stray writes
show). Complements the reference's own grids (tests/test_gpu_grid.py), which
only reach small tiles and dense layouts. Integer results and pack/unpack
bit-exact; f16/bf16 within |got - ref| <= 1e-3 * max(|ref|, rms(ref)).
"""
import ctypes as C
import random

import numpy as np
import pytest
import torch

from iree_amd import abi, synth
from test_gpu_configs import gpu_lib  # noqa: F401

pytestmark = pytest.mark.gpu

TI, TO = abi.PACK_TRANSPOSE_INNER, abi.PACK_TRANSPOSE_OUTER
PACK_TYPES = [abi.PACK_TYPE_I8I8, abi.PACK_TYPE_F16F16, abi.PACK_TYPE_BF16BF16, abi.PACK_TYPE_F32F32, abi.PACK_TYPE_I32I32]
UNPACK_OF = {abi.PACK_TYPE_F16F16: abi.UNPACK_TYPE_F16F16, abi.PACK_TYPE_BF16BF16: abi.UNPACK_TYPE_BF16BF16,
             abi.PACK_TYPE_F32F32: abi.UNPACK_TYPE_F32F32, abi.PACK_TYPE_I32I32: abi.UNPACK_TYPE_I32I32}


@pytest.mark.parametrize("seed,small_elements_transposed", [(1, False), (7, True)])
def test_pack_unpack_random_cases(gpu_lib, oracle_lib, seed, small_elements_transposed):
    rnd = random.Random(seed)
    kernels = set()
    for case in range(150):
        typ = rnd.choice(PACK_TYPES[:3] if small_elements_transposed else PACK_TYPES)
        e = abi.PACK_ELEM_BYTES[typ]
        t0, t1 = 1 << rnd.randint(0, 6), 1 << rnd.randint(0, 6)
        if t0 * t1 * e > 4096:
            t1 = max(1, 4096 // (t0 * e))
        flags = rnd.choice([0, TI, TO, TI | TO])
        rows, cols = rnd.randint(1, 900), rnd.randint(1, 1500)
        in_stride = cols + rnd.choice([0, 0, 3, 4, 16])
        in_off = rnd.choice([0, 0, 1, 4, 16])
        if small_elements_transposed:
            # Where the register-transposing kernels apply: inner transpose, dword-aligned rows.
            flags |= TI
            rows = rnd.randint(1, 2500)
            in_stride = (in_stride + 3) // 4 * 4
            in_off = rnd.choice([0, 4, 16])
        o0 = -(-rows // t0) + rnd.choice([0, 0, 1])
        o1 = -(-cols // t1) + rnd.choice([0, 0, 2])
        s0, s1 = (o1, o0) if flags & TO else (o0, o1)
        s2, s3 = (t1, t0) if flags & TI else (t0, t1)
        out_stride = s1 * s2 * s3 + rnd.choice([0, 0, 16 // e, 64])
        out_off = rnd.choice([0, 0, 16 // e])
        src = np.frombuffer(np.random.default_rng(1000 * seed + case).bytes((in_off + rows * in_stride) * e), dtype=np.int8).copy()
        n_out = out_off + s0 * out_stride

        def pack_params(src_ptr, dst_ptr):
            p = abi.PackParams()
            p.in_buffer, p.out_buffer = src_ptr, dst_ptr
            p.in_offset, p.out_offset = in_off, out_off
            p.in_stride0, p.in_stride1 = in_stride, 1
            p.out_stride0, p.out_stride1 = out_stride, s2 * s3
            p.in_size0, p.in_size1 = rows, cols
            p.out_size0, p.out_size1, p.out_size2, p.out_size3 = s0, s1, s2, s3
            p.padding_value = 0x5AA55AA5
            p.flags = typ | flags
            return p

        what = "case %d type %#x tile %dx%d flags %#x %dx%d outer %dx%d strides %d/%d offsets %d/%d" % (
            case, typ, t0, t1, flags, rows, cols, o0, o1, in_stride, out_stride, in_off, out_off)
        want = np.full(n_out * e, 0x77, dtype=np.int8)
        oracle_lib.oracle_pack(C.byref(pack_params(src.ctypes.data, want.ctypes.data)))
        d_src = torch.from_numpy(src).cuda()
        d_out = torch.full((n_out * e,), 0x77, dtype=torch.int8, device="cuda")
        gpu_lib.iree_uk_pack_p(C.byref(pack_params(d_src.data_ptr(), d_out.data_ptr())))
        kernels.add(gpu_lib.iree_uk_mi355x_last_kernel())
        assert np.array_equal(d_out.cpu().numpy(), want), "pack " + what
        if typ not in UNPACK_OF:
            continue
        back_stride = cols + rnd.choice([0, 1, 4])

        def unpack_params(src_ptr, dst_ptr):
            p = abi.UnpackParams()
            p.in_buffer, p.out_buffer = src_ptr, dst_ptr
            p.in_offset, p.out_offset = out_off, in_off
            p.in_stride0, p.in_stride1 = out_stride, s2 * s3
            p.out_stride0, p.out_stride1 = back_stride, 1
            p.in_size0, p.in_size1, p.in_size2, p.in_size3 = s0, s1, s2, s3
            p.out_size0, p.out_size1 = rows, cols
            p.flags = UNPACK_OF[typ] | flags
            return p

        n_back = (in_off + rows * back_stride) * e
        want_back = np.full(n_back, 0x33, dtype=np.int8)
        oracle_lib.oracle_unpack(C.byref(unpack_params(want.ctypes.data, want_back.ctypes.data)))
        d_in = torch.from_numpy(want).cuda()
        d_back = torch.full((n_back,), 0x33, dtype=torch.int8, device="cuda")
        gpu_lib.iree_uk_unpack_p(C.byref(unpack_params(d_in.data_ptr(), d_back.data_ptr())))
        kernels.add(gpu_lib.iree_uk_mi355x_last_kernel())
        assert np.array_equal(d_back.cpu().numpy(), want_back), "unpack " + what
    # The sweep is only worth its time if it reaches the specialised kernels.
    assert b"pack_tiled" in kernels and b"pack_transposing" in kernels
    assert small_elements_transposed or b"unpack_tiled" in kernels


def _mmt4d_sweep(gpu_lib, oracle_lib, seed, cases, types, n0_choices, long_k):
    """Random problems of the given type flags against the oracle; returns the kernels that ran."""
    rnd = random.Random(seed)
    kernels = set()
    for case in range(cases):
        typ = rnd.choice(types)
        lb, rb, ob = abi.MMT4D_BITS[typ & abi.MMT4D_TYPE_MASK]
        M0, N0 = rnd.choice([1, 2, 4, 8, 16]), rnd.choice(n0_choices)
        K0 = rnd.choice([1, 2, 4, 8, 16, 32, 64] if lb < 32 else [1, 2, 4, 8, 16])
        if typ == abi.MMT4D_TYPE_S8S4S32 and K0 < 2:
            K0 = 2
        kind = rnd.random()
        if kind < 0.35:      # a skinny lhs against many rhs tiles
            M, N, K = rnd.choice([1, 1, 2, 4]), rnd.randint(16, 200), rnd.randint(1, 40)
            if long_k and rnd.random() < 0.5:
                K = rnd.randint(40, 700)
            if rnd.random() < 0.6:
                N0 = 16
        elif kind < 0.7:
            M, N, K = rnd.randint(1, 12), rnd.randint(1, 30), rnd.randint(1, 24)
        else:
            M, N, K = rnd.randint(8, 40), rnd.randint(8, 60), rnd.randint(1, 12)
        row_bytes = K0 * lb // 8
        if rnd.random() < 0.5 and 0 < row_bytes <= 64 and 64 % row_bytes == 0:
            per = 64 // row_bytes     # K that ends on a 64-byte chunk: the direct-to-LDS kernels
            K = max(per, K // per * per)
        flags = typ | rnd.choice([0, abi.MMT4D_ACCUMULATE])
        ls = K * M0 * K0 + rnd.choice([0, 0, 16, 64])
        rs = K * N0 * K0 + rnd.choice([0, 0, 32, 128])
        os_ = N * M0 * N0 + rnd.choice([0, 0, 4, 16])
        lo, ro, oo = rnd.choice([0, 0, 16, 64]), rnd.choice([0, 0, 32, 128]), rnd.choice([0, 0, 4, 8])
        rng = np.random.default_rng(case)
        is_f16 = False
        if lb == 8:
            lhs = rng.integers(-128, 128, lo + M * ls, dtype=np.int8)
            rhs = rng.integers(-128, 128, (ro + N * rs) * rb // 8, dtype=np.int8)
            init = rng.integers(-10000, 10000, oo + M * os_, dtype=np.int32)
        elif lb == 32:
            lhs = rng.standard_normal(lo + M * ls).astype(np.float32)
            rhs = (rng.standard_normal(ro + N * rs) / 8).astype(np.float32)
            init = rng.standard_normal(oo + M * os_).astype(np.float32)
        else:
            is_f16 = (typ & abi.MMT4D_TYPE_MASK) in (abi.MMT4D_TYPE_F16F16F32, abi.MMT4D_TYPE_F16F16F16)
            to_bits = synth.f16_bits if is_f16 else synth.bf16_bits
            lhs = to_bits(rng.standard_normal(lo + M * ls).astype(np.float32))
            rhs = to_bits((rng.standard_normal(ro + N * rs) / 8).astype(np.float32))
            init = rng.standard_normal(oo + M * os_).astype(np.float32)
            if ob == 16:
                init = to_bits(init)

        def params(l, r, o):
            p = abi.Mmt4dParams()
            p.lhs_buffer, p.rhs_buffer, p.out_buffer = l, r, o
            p.lhs_offset, p.rhs_offset, p.out_offset = lo, ro, oo
            p.lhs_stride0, p.rhs_stride0, p.out_stride0 = ls, rs, os_
            p.M, p.N, p.K, p.M0, p.N0, p.K0 = M, N, K, M0, N0, K0
            p.flags = flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK
            return p

        want = init.copy()
        oracle_lib.oracle_mmt4d_mt(C.byref(params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data)), 8)
        dev = lambda x: torch.from_numpy(x.view(np.int16) if x.dtype == np.uint16 else x).cuda()  # noqa: E731
        d_l, d_r, d_o = dev(lhs), dev(rhs), dev(init.copy())
        gpu_lib.iree_uk_mmt4d_p(C.byref(params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr())))
        kernel = gpu_lib.iree_uk_mi355x_last_kernel()
        kernels.add(kernel)
        got = d_o.cpu().numpy()
        what = "case %d type %#x %dx%dx%d tile %dx%dx%d flags %#x strides %d/%d/%d offsets %d/%d/%d %s" % (
            case, typ, M, N, K, M0, N0, K0, flags, ls, rs, os_, lo, ro, oo, kernel.decode())
        if want.dtype == np.int32:
            assert np.array_equal(got, want), what
            continue
        ulp = 0.0
        if ob == 16:   # one rounding to the 16-bit output at the end: within one unit in the last place on top
            got = got.view(np.uint16)
            if is_f16:
                got, want, ulp = got.view(np.float16).astype(np.float32), want.view(np.float16).astype(np.float32), 2.0 ** -10
            else:
                got, want = (got.astype(np.uint32) << 16).view(np.float32), (want.astype(np.uint32) << 16).view(np.float32)
                ulp = 2.0 ** -7
        rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        assert np.all(np.abs(got - want) <= (1e-3 + ulp) * np.maximum(np.abs(want), rms)), what
    return kernels


def test_mmt4d_random_cases(gpu_lib, oracle_lib):
    types = [abi.MMT4D_TYPE_S8S8S32, abi.MMT4D_TYPE_S8S4S32, abi.MMT4D_TYPE_F16F16F32, abi.MMT4D_TYPE_BF16BF16F32]
    kernels = _mmt4d_sweep(gpu_lib, oracle_lib, 1, 300, types, [4, 8, 16, 16], long_k=False)
    assert {b"mmt4d_generic", b"mmt4d_mfma_64x64", b"mmt4d_gemv"} <= kernels


def test_mmt4d_random_cases_more_types_and_shapes(gpu_lib, oracle_lib):
    # f32 and the 16-bit outputs (roundings between k steps skipped) as well, rhs tiles down to 2 rows, and skinny
    # problems with a K long enough for every wavefront of the narrow-tile kernel to get several rounds.
    skip = abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
    types = [abi.MMT4D_TYPE_S8S8S32, abi.MMT4D_TYPE_S8S8S32, abi.MMT4D_TYPE_F16F16F32, abi.MMT4D_TYPE_BF16BF16F32,
             abi.MMT4D_TYPE_F32F32F32, abi.MMT4D_TYPE_F16F16F16 | skip, abi.MMT4D_TYPE_BF16BF16BF16 | skip]
    kernels = _mmt4d_sweep(gpu_lib, oracle_lib, 21, 300, types, [2, 4, 8, 16, 16], long_k=True)
    assert {b"mmt4d_generic", b"mmt4d_mfma_64x64", b"mmt4d_skinny"} <= kernels


# The tile shapes for which the reference's x86-64 and Arm targets have their own pack / unpack tile functions
# (arch/x86_64/pack_x86_64_entry_point.c:99-113, arch/arm_64/pack_arm_64_entry_point.c:16-31; unpack:
# arch/x86_64/unpack_x86_64_entry_point.c:18-30, arch/arm_64/unpack_arm_64_entry_point.c:13-19), as (element bytes,
# out_size2, out_size3): what a caller compiled for those CPUs passes. Each with every transpose combination, on a
# ragged matrix, bit for bit against the oracle, and none of them on a one-thread-per-element kernel.
CPU_PACK_TILES = [(4, 8, 8), (4, 16, 16), (4, 8, 1), (4, 16, 1), (2, 16, 2), (1, 8, 2), (1, 16, 2), (1, 8, 1), (1, 8, 4),
                  (1, 8, 8)]
CPU_UNPACK_TILES = [(4, 8, 8), (4, 16, 16)]


@pytest.mark.parametrize("e,s2,s3", CPU_PACK_TILES)
@pytest.mark.parametrize("flags", [0, TI, TO, TI | TO])
def test_pack_tile_shapes_of_the_reference_cpu_targets(gpu_lib, oracle_lib, e, s2, s3, flags):
    typ = {4: abi.PACK_TYPE_F32F32, 2: abi.PACK_TYPE_BF16BF16, 1: abi.PACK_TYPE_I8I8}[e]
    t0, t1 = (s3, s2) if flags & TI else (s2, s3)      # tile extents along dims 0 and 1 of the source
    rows, cols = 1276, 2044     # (8-byte tiles are taken in pairs: an even number of them whichever way they run)
    o0, o1 = -(-rows // t0), -(-cols // t1)
    s0, s1 = (o1, o0) if flags & TO else (o0, o1)
    out_stride = s1 * s2 * s3
    src = np.frombuffer(np.random.default_rng(e * 100 + s2 + s3 + flags).bytes(rows * cols * e), dtype=np.int8).copy()

    def pack_params(src_ptr, dst_ptr):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_stride0, p.in_stride1 = cols, 1
        p.out_stride0, p.out_stride1 = out_stride, s2 * s3
        p.in_size0, p.in_size1 = rows, cols
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = s0, s1, s2, s3
        p.padding_value = 0x5AA55AA5
        p.flags = typ | flags
        return p

    want = np.full(s0 * out_stride * e, 0x77, dtype=np.int8)
    oracle_lib.oracle_pack(C.byref(pack_params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_out = torch.full((want.size,), 0x77, dtype=torch.int8, device="cuda")
    gpu_lib.iree_uk_pack_p(C.byref(pack_params(d_src.data_ptr(), d_out.data_ptr())))
    kernel = gpu_lib.iree_uk_mi355x_last_kernel()
    assert np.array_equal(d_out.cpu().numpy(), want)
    assert kernel and b"generic" not in kernel, kernel
    if (e, s2, s3) not in CPU_UNPACK_TILES or flags:
        return
    back = np.full(rows * cols * e, 0x33, dtype=np.int8)

    def unpack_params(src_ptr, dst_ptr):
        p = abi.UnpackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_stride0, p.in_stride1 = out_stride, s2 * s3
        p.out_stride0, p.out_stride1 = cols, 1
        p.in_size0, p.in_size1, p.in_size2, p.in_size3 = s0, s1, s2, s3
        p.out_size0, p.out_size1 = rows, cols
        p.flags = abi.UNPACK_TYPE_F32F32
        return p

    d_back = torch.full((back.size,), 0x33, dtype=torch.int8, device="cuda")
    gpu_lib.iree_uk_unpack_p(C.byref(unpack_params(d_out.data_ptr(), d_back.data_ptr())))
    kernel = gpu_lib.iree_uk_mi355x_last_kernel()
    assert np.array_equal(d_back.cpu().numpy(), src)
    assert kernel and b"generic" not in kernel, kernel


@pytest.mark.parametrize("flags", [0, TI, TO, TI | TO])
def test_eight_byte_tiles_with_an_odd_tile_count(gpu_lib, oracle_lib, flags):
    # int8 8x1 tiles are taken two at a time; with an odd number of them along out dimension 1 the last column of
    # tiles is written by a second launch. Rows of the tiled buffer padded to 16-byte multiples; the whole
    # destination (pre-filled) is compared, padding tiles beyond the source included.
    s2, s3 = 8, 1
    t0, t1 = (s3, s2) if flags & TI else (s2, s3)
    rows, cols = 1237, 2041
    o0, o1 = -(-rows // t0) + 2, -(-cols // t1)       # two rows of tiles that are nothing but padding
    if ((o0 if flags & TO else o1) & 1) == 0:
        o0, o1 = (o0 + 1, o1) if flags & TO else (o0, o1 + 1)
    s0, s1 = (o1, o0) if flags & TO else (o0, o1)
    assert s1 & 1
    out_stride = s1 * 8 + 8
    src = np.frombuffer(np.random.default_rng(flags + 5).bytes(rows * cols), dtype=np.int8).copy()

    def pack_params(src_ptr, dst_ptr):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_stride0, p.in_stride1 = cols, 1
        p.out_stride0, p.out_stride1 = out_stride, 8
        p.in_size0, p.in_size1 = rows, cols
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = s0, s1, s2, s3
        p.padding_value = 0x5A
        p.flags = abi.PACK_TYPE_I8I8 | flags
        return p

    want = np.full(s0 * out_stride, 0x77, dtype=np.int8)
    oracle_lib.oracle_pack(C.byref(pack_params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_out = torch.full((want.size,), 0x77, dtype=torch.int8, device="cuda")
    gpu_lib.iree_uk_pack_p(C.byref(pack_params(d_src.data_ptr(), d_out.data_ptr())))
    assert gpu_lib.iree_uk_mi355x_last_kernel() in (b"pack_tiled", b"pack_transposing")
    assert np.array_equal(d_out.cpu().numpy(), want)
