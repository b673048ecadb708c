"""GPU parity for the skinny-lhs kernel (mmt4d_gemv.hip) on one 16-row lhs tile,
against the oracle restatement of the generic tile functions
(mmt4d_tile_generic.c:54-78 int8, :199-225 f16, :289-315 bf16): every row-piece
size it takes, odd rhs tile counts, K shares that are not a multiple of the
unrolling, K that does not end on a 64-byte step, accumulate, strided rhs.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, synth
from test_gpu_configs import assert_float_close, gpu_lib, mm_params  # noqa: F401

pytestmark = pytest.mark.gpu

CASES = [
    # flags, N, K, K0, expected kernel
    (abi.MMT4D_TYPE_BF16BF16F32, 37, 512, 8, b"mmt4d_gemv"),     # rb 16, N % 4 != 0
    (abi.MMT4D_TYPE_BF16BF16F32, 64, 4 * 17, 8, b"mmt4d_gemv"),  # 17 K-steps: shares of 5, 5, 5, 2
    (abi.MMT4D_TYPE_F16F16F32, 50, 256, 16, b"mmt4d_gemv"),      # rb 32
    (abi.MMT4D_TYPE_S8S8S32, 41, 64, 64, b"mmt4d_gemv"),         # rb 64
    (abi.MMT4D_TYPE_S8S8S32, 29, 128, 32, b"mmt4d_gemv"),        # rb 32, int8
    (abi.MMT4D_TYPE_S8S8S32, 33, 260, 16, b"mmt4d_gemv"),        # rb 16, 65 K-steps
    (abi.MMT4D_TYPE_BF16BF16F32, 20, 1026, 8, b"mmt4d_gemv"),        # K does not end on a K-step
    (abi.MMT4D_TYPE_BF16BF16F32, 24, 8200, 8, b"mmt4d_gemv"),        # long K
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "t%x_N%d_K%d_K0%d" % (c[0], c[1], c[2], c[3]))
@pytest.mark.parametrize("acc", [0, abi.MMT4D_ACCUMULATE])
def test_sixteen_row_lhs(gpu_lib, oracle_lib, case, acc):
    flags, N, K, K0, kernel = case
    M0 = N0 = 16
    flags |= acc
    rhs_stride = K * N0 * K0 + 64  # elements; a gap between rhs panels
    if (flags & 0xFF) == abi.MMT4D_TYPE_S8S8S32:
        lhs = synth.uniform_int8(41, 0, K * M0 * K0)
        rhs = synth.uniform_int8(41, 1, N * rhs_stride)
        init = (synth.uniform_int8(41, 2, N * M0 * N0).astype(np.int32)) * 1000
    else:
        to_bits = synth.f16_bits if (flags & 0xFF) == abi.MMT4D_TYPE_F16F16F32 else synth.bf16_bits
        lhs = to_bits(synth.normal_f32(41, 0, K * M0 * K0, 1.0))
        rhs = to_bits(synth.normal_f32(41, 1, N * rhs_stride, 0.05))
        init = synth.normal_f32(41, 2, N * M0 * N0, 1.0)
    want = init.copy()
    p = mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, 1, N, K, M0, N0, K0,
                  flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK)
    p.rhs_stride0 = rhs_stride
    oracle_lib.oracle_mmt4d_mt(C.byref(p), 8)
    as_dev = lambda x: torch.from_numpy(x.view(np.int16) if x.dtype == np.uint16 else x).cuda()
    d_l, d_r, d_o = as_dev(lhs), as_dev(rhs), as_dev(init.copy())
    q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), 1, N, K, M0, N0, K0, flags)
    q.rhs_stride0 = rhs_stride
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == kernel
    got = d_o.cpu().numpy()
    if want.dtype == np.int32:
        assert np.array_equal(got, want)
    else:
        assert_float_close(got, want, "16-row lhs N=%d K=%d K0=%d" % (N, K, K0))


# Tile counts around the number of compute units (one workgroup per rhs tile: fewer workgroups than units, exactly
# one or more per unit, the decode shape's 896), bit for bit on int8, with guard words either side of the output.
@pytest.mark.parametrize("N", [256, 200, 128, 300, 896])
@pytest.mark.parametrize("M0", [1, 4, 16])
def test_tile_counts_around_the_number_of_compute_units(gpu_lib, oracle_lib, N, M0):
    N0, K0, K = 16, 16, 24
    flags = abi.MMT4D_TYPE_S8S8S32 | abi.MMT4D_ACCUMULATE
    lhs = synth.uniform_int8(43, 0, K * M0 * K0)
    rhs = synth.uniform_int8(43, 1, N * K * N0 * K0)
    init = synth.uniform_int8(43, 2, N * M0 * N0).astype(np.int32) * 77
    want = init.copy()
    oracle_lib.oracle_mmt4d_mt(C.byref(mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, 1, N, K, M0, N0, K0,
                                                 flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK)), 8)
    d_l, d_r, d_o = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), torch.from_numpy(init.copy()).cuda()
    guard = torch.full((64,), 123456, dtype=torch.int32, device="cuda")
    d_all = torch.cat([guard, d_o, guard])
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_all.data_ptr() + 256, 1, N, K, M0, N0, K0,
                                              flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_gemv"
    got = d_all.cpu().numpy()
    assert np.array_equal(got[64:-64], want)
    assert (got[:64] == 123456).all() and (got[-64:] == 123456).all()


# The resident-lhs kernel (one workgroup per compute unit, the lhs operands of each wavefront's K share copied to
# LDS once, rhs dealt out in half tiles): at least one rhs tile per compute unit, more than 4 lhs rows, K of
# 64 or 128 steps of 64 bytes. Tile counts that give the units whole tiles, half tiles at either end of their
# ranges, ranges of unequal length, and equally many whole tiles per unit (dealt out in rounds instead of ranges); lhs rows from one, two and four lhs tiles, fewer than 16 rows; a gap
# between rhs panels, strided lhs and out rows; with guard words around the output. int8 bit for bit.
RESIDENT = [
    # flags, M, M0, N, K, K0
    (abi.MMT4D_TYPE_S8S8S32, 1, 16, 896, 64, 64),     # 64 steps; 3.5 tiles per unit
    (abi.MMT4D_TYPE_S8S8S32, 1, 16, 256, 128, 64),    # 128 steps; exactly one tile per unit
    (abi.MMT4D_TYPE_S8S8S32, 1, 16, 768, 64, 64),     # three whole tiles per unit: one of every round of 256 tiles
    (abi.MMT4D_TYPE_BF16BF16F32, 1, 16, 512, 512, 8),   # two whole tiles per unit, 128 steps
    (abi.MMT4D_TYPE_S8S8S32, 2, 8, 257, 256, 16),     # 64 steps; two lhs tiles of 8 rows
    (abi.MMT4D_TYPE_S8S8S32, 4, 4, 1000, 128, 32),    # 64 steps; four lhs tiles of 4 rows
    (abi.MMT4D_TYPE_S8S8S32, 3, 4, 511, 512, 16),     # 128 steps; 12 lhs rows
    (abi.MMT4D_TYPE_S8S8S32, 1, 8, 1791, 64, 64),     # 8 lhs rows; 7 tiles per unit at most
    (abi.MMT4D_TYPE_BF16BF16F32, 1, 16, 897, 512, 8),   # the decode shape plus one tile
    (abi.MMT4D_TYPE_F16F16F32, 1, 16, 300, 128, 16),    # rb 32, 64 steps
    (abi.MMT4D_TYPE_BF16BF16F32, 2, 8, 384, 256, 16),   # rb 32, 128 steps
]


@pytest.mark.parametrize("case", RESIDENT, ids=lambda c: "t%x_M%dx%d_N%d_K%d_K0%d" % c)
@pytest.mark.parametrize("acc", [0, abi.MMT4D_ACCUMULATE])
def test_resident_lhs_kernel(gpu_lib, oracle_lib, case, acc):
    flags, M, M0, N, K, K0 = case
    N0 = 16
    flags |= acc
    lhs_stride, rhs_stride, out_stride = K * M0 * K0 + 32, K * N0 * K0 + 64, N * M0 * N0 + 8
    if (flags & 0xFF) == abi.MMT4D_TYPE_S8S8S32:
        lhs = synth.uniform_int8(47, 0, M * lhs_stride)
        rhs = synth.uniform_int8(47, 1, N * rhs_stride)
        init = (synth.uniform_int8(47, 2, M * out_stride).astype(np.int32)) * 1000
    else:
        to_bits = synth.f16_bits if (flags & 0xFF) == abi.MMT4D_TYPE_F16F16F32 else synth.bf16_bits
        lhs = to_bits(synth.normal_f32(47, 0, M * lhs_stride, 1.0))
        rhs = to_bits(synth.normal_f32(47, 1, N * rhs_stride, 0.05))
        init = synth.normal_f32(47, 2, M * out_stride, 1.0)

    def strided(p):
        p.lhs_stride0, p.rhs_stride0, p.out_stride0 = lhs_stride, rhs_stride, out_stride
        return p
    want = init.copy()
    oracle_lib.oracle_mmt4d_mt(C.byref(strided(mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, M, N, K,
                                                         M0, N0, K0, flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK))), 8)
    as_dev = lambda x: torch.from_numpy(x.view(np.int16) if x.dtype == np.uint16 else x).cuda()
    d_l, d_r = as_dev(lhs), as_dev(rhs)
    guard = torch.full((64,), 7, dtype=torch.from_numpy(init).dtype, device="cuda")
    d_all = torch.cat([guard, torch.from_numpy(init.copy()).cuda(), guard])
    gpu_lib.iree_uk_mmt4d_p(C.byref(strided(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_all.data_ptr() + 256, M, N, K,
                                                      M0, N0, K0, flags))))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_gemv_resident_lhs"
    got_all = d_all.cpu().numpy()
    got = got_all[64:-64]
    assert (got_all[:64] == 7).all() and (got_all[-64:] == 7).all()
    if want.dtype == np.int32:
        assert np.array_equal(got, want)       # the gaps between out rows included
    else:
        rows = np.arange(M * out_stride).reshape(M, out_stride)
        inside = rows[:, :N * M0 * N0].reshape(-1)
        assert_float_close(got[inside], want[inside], "resident lhs %r" % (case,))
        gaps = rows[:, N * M0 * N0:].reshape(-1)
        assert np.array_equal(got[gaps], init[gaps])
