"""GPU parity for the skinny-lhs kernel with int4 weights (s8s4s32,
mmt4d_gemv.hip) against the oracle restatement of
mmt4d_tile_generic.c:11-51 (low nibble = even element, sign-extended): the
decode shapes M0 in {1, 4, 16}, K0 = 32 and 64, lhs rows from several tiles,
odd rhs tile counts, K shares that are not a multiple of the unrolling,
accumulate, strided rhs and offsets; and the shapes it must leave to the other
kernels. Bit-exact.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, synth
from test_gpu_configs import gpu_lib, mm_params  # noqa: F401

pytestmark = pytest.mark.gpu

CASES = [
    # M, M0, N, K, K0, expected kernel
    (1, 1, 33, 8, 32, b"mmt4d_gemv"),
    (1, 4, 40, 12, 32, b"mmt4d_gemv"),
    (1, 16, 37, 128, 32, b"mmt4d_gemv"),      # K = 4096
    (1, 16, 21, 68, 32, b"mmt4d_gemv"),       # 17 steps: shares of 5, 5, 5, 2
    (4, 4, 25, 16, 32, b"mmt4d_gemv"),        # 16 lhs rows from 4 tiles
    (2, 8, 19, 6, 64, b"mmt4d_gemv"),         # K0 = 64
    (1, 16, 50, 20, 64, b"mmt4d_gemv"),
    (1, 16, 18, 3, 32, None),                 # K * K0 = 96: not a whole step
    (1, 16, 18, 8, 16, None),                 # 8-byte rhs row pieces
    (1, 2, 18, 2048, 64, b"mmt4d_gemv"),      # K * K0 = 131072: 16x-scaled sums could overflow; chained over two slices of K
    # The resident-lhs kernel: more than 4 lhs rows, a tile or more per compute unit, 64 or 32 steps of 128 values.
    # (Its lhs operands sit in LDS with the bytes of every dword pair reordered to match nibbles that are widened
    # without interleaving: any lhs value pattern must still come out bit for bit.)
    (1, 16, 897, 256, 32, b"mmt4d_gemv_resident_lhs"),    # K = 8192: half tiles at both ends of the units' ranges
    (1, 16, 256, 128, 64, b"mmt4d_gemv_resident_lhs"),    # one tile per unit, K0 = 64
    (2, 8, 1791, 128, 32, b"mmt4d_gemv_resident_lhs"),    # K = 4096 (32 steps), two lhs tiles, up to 7 tiles per unit
    (3, 4, 300, 256, 32, b"mmt4d_gemv_resident_lhs"),     # 12 lhs rows
    (1, 16, 2000, 256, 32, b"mmt4d_gemv"),                # more tiles per unit than it keeps accumulators for
    # Six tiles or more per compute unit: the resident-lhs kernel with any number of lhs rows.
    (1, 1, 1600, 128, 32, b"mmt4d_gemv_resident_lhs"),    # one lhs row, 32 steps
    (1, 4, 1537, 128, 64, b"mmt4d_gemv_resident_lhs"),    # four lhs rows, 64 steps, half tiles in play
    (1, 2, 1535, 128, 32, b"mmt4d_gemv"),                 # just under six tiles per unit
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "M%dx%d_N%d_K%d_K0%d" % c[:5])
@pytest.mark.parametrize("acc", [0, abi.MMT4D_ACCUMULATE])
def test_int4_weights_skinny_lhs(gpu_lib, oracle_lib, case, acc):
    M, M0, N, K, K0, kernel = case
    N0 = 16
    flags = abi.MMT4D_TYPE_S8S4S32 | acc
    lhs_off, rhs_off, out_off = 16, 64, 4          # elements (rhs: 4-bit elements)
    lhs_stride = K * M0 * K0 + 32
    rhs_stride = K * N0 * K0 + 128                 # 4-bit elements: a 64-byte gap between panels
    out_stride = N * M0 * N0 + 8
    lhs = synth.uniform_int8(51, 0, lhs_off + M * lhs_stride)
    rhs = synth.uniform_int4_packed(51, 1, rhs_off + N * rhs_stride)
    init = synth.uniform_int8(51, 2, out_off + M * out_stride).astype(np.int32) * 100000
    want = init.copy()
    p = mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, M, N, K, M0, N0, K0,
                  flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK, lhs_off, rhs_off, out_off,
                  lhs_stride, rhs_stride, out_stride)
    oracle_lib.oracle_mmt4d_mt(C.byref(p), 8)
    d_l, d_r, d_o = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), torch.from_numpy(init.copy()).cuda()
    q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags,
                  lhs_off, rhs_off, out_off, lhs_stride, rhs_stride, out_stride)
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    name = gpu_lib.iree_uk_mi355x_last_kernel()
    if kernel is None:
        assert name != b"mmt4d_gemv"
    else:
        assert name == kernel
    assert np.array_equal(d_o.cpu().numpy(), want)


def test_int4_weights_extreme_values(gpu_lib, oracle_lib):
    # All weights -8 against all activations -128 over K * K0 = 65536: the largest
    # magnitude the 16x-scaled accumulators reach, 2^30 * 16 / 16 ... must stay exact.
    M0, N0, K0, N, K = 16, 16, 32, 16, 2048
    lhs = np.full(K * M0 * K0, -128, dtype=np.int8)
    rhs = np.full(N * K * N0 * K0 // 2, 0x88, dtype=np.uint8)
    want = np.zeros(N * M0 * N0, dtype=np.int32)
    flags = abi.MMT4D_TYPE_S8S4S32
    oracle_lib.oracle_mmt4d_mt(C.byref(mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, 1, N, K, M0, N0, K0,
                                                 flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK)), 8)
    assert int(want[0]) == 128 * 8 * K * K0
    d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs.view(np.int8)).cuda()
    d_o = torch.zeros(N * M0 * N0, dtype=torch.int32, device="cuda")
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), 1, N, K, M0, N0, K0, flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_gemv"
    assert np.array_equal(d_o.cpu().numpy(), want)
