"""GPU parity for the skinny-lhs kernel of the narrow tile shapes (mmt4d_skinny.hip): at most 8 lhs rows in total
and row pieces (K0 elements) of 2, 4 or 8 bytes, i.e. what the reference's CPU targets pick for matrix-vector and
few-row products (mmt4d_x86_64_tiles.inl: 1x16x2 int8/bf16, 1x16x1 f16/f32 and their 2-, 4- and 8-row siblings;
mmt4d_arm_64_tiles.inl: 1x8x4 and 1x8x8 int8, 1x8x1 f32, ...).

Integer results are compared bit for bit with a float64 matrix product of the same operands, float results within
|got - ref| <= 1e-3 * max(|ref|, rms(ref)) of it (test_gpu_big_tiles.run_case).
"""
import ctypes as C

import pytest
import torch

from iree_amd import abi
from test_gpu_big_tiles import run_case
from test_gpu_configs import gpu_lib, mm_params  # noqa: F401

pytestmark = pytest.mark.gpu

S8, F16, BF16, F32 = abi.MMT4D_TYPE_S8S8S32, abi.MMT4D_TYPE_F16F16F32, abi.MMT4D_TYPE_BF16BF16F32, abi.MMT4D_TYPE_F32F32F32
F16_OUT16, BF16_OUT16 = abi.MMT4D_TYPE_F16F16F16, abi.MMT4D_TYPE_BF16BF16BF16  # run with the roundings between k steps skipped


# (type, M, M0, N0, K0): every piece size of every type, every row count, both rhs tile heights, several lhs tiles.
SHAPES = [
    (S8, 1, 1, 16, 2), (S8, 1, 2, 16, 2), (S8, 1, 4, 16, 2), (S8, 2, 4, 16, 2), (S8, 3, 1, 16, 2), (S8, 2, 2, 8, 2),
    (S8, 1, 1, 8, 4), (S8, 1, 2, 8, 4), (S8, 1, 4, 16, 4), (S8, 5, 1, 4, 4), (S8, 1, 1, 8, 8), (S8, 1, 4, 8, 8),
    (S8, 2, 4, 2, 8), (F16, 1, 1, 16, 1), (F16, 1, 4, 16, 1), (F16, 7, 1, 8, 1), (F16, 1, 2, 8, 2), (F16, 1, 1, 16, 4),
    (BF16, 1, 1, 16, 2), (BF16, 1, 2, 16, 2), (BF16, 8, 1, 16, 1), (BF16, 3, 1, 8, 4), (F32, 1, 1, 16, 1),
    (F32, 1, 4, 8, 1), (F32, 2, 2, 4, 1), (F32, 1, 1, 8, 2), (F32, 6, 1, 2, 2), (F16_OUT16, 1, 1, 16, 1),
    (F16_OUT16, 1, 4, 8, 1), (F16_OUT16, 3, 2, 8, 2), (BF16_OUT16, 1, 1, 16, 2), (BF16_OUT16, 1, 2, 8, 4),
    (BF16_OUT16, 5, 1, 8, 4)]


@pytest.mark.parametrize("flags,M,M0,N0,K0", SHAPES)
def test_narrow_tiles_few_rows(gpu_lib, flags, M, M0, N0, K0):
    # K: less than one 1 KiB block of the stream, a stream that ends inside a block and inside a wavefront's share,
    # and one long enough for several rounds of every wavefront.
    for n, K in enumerate((3, 77, 1500)):
        run_case(gpu_lib, flags, M, 37 + n, K, M0, N0, K0, "mmt4d_skinny", accumulate=bool(n & 1), seed=K + M0)
    # strided operands with offsets (rhs tile rows stay 16-byte aligned, lhs rows 8-byte), padded output
    e = 1 if flags == S8 else (4 if flags == F32 else 2)
    run_case(gpu_lib, flags, M, 21, 130, M0, N0, K0, "mmt4d_skinny", lhs_pad=8, rhs_pad=16 // e, out_pad=5,
             offsets=(8, 32 // e, 3), accumulate=True, seed=9)


def test_non_finite_lhs_values_do_not_leak_into_other_k_steps(gpu_lib):
    # The rhs stream of a tile row ends inside a block of 64 lanes x 16 bytes; the idle lanes must add nothing, also
    # when the lhs holds an infinity at the k step they would read.
    M0, N0, K0, K, N = 1, 16, 2, 5, 3
    lhs = torch.ones(K * M0 * K0, device="cuda", dtype=torch.bfloat16)
    lhs[0] = float("inf")
    rhs = torch.ones(N * K * N0 * K0, device="cuda", dtype=torch.bfloat16)
    rhs.view(N, K, N0, K0)[:, 0, :, 0] = 0.25
    rhs.view(N, K, N0, K0)[:, 0, 5, 0] = 0.0  # inf * 0 = nan in exactly these outputs
    out = torch.zeros(N * M0 * N0, device="cuda")
    p = mm_params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), 1, N, K, M0, N0, K0, BF16)
    gpu_lib.iree_uk_mmt4d_p(C.byref(p))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_skinny"
    got = out.view(N, N0)
    assert bool(torch.isnan(got[:, 5]).all())
    rest = torch.cat([got[:, :5], got[:, 6:]], dim=1)
    assert bool(torch.isinf(rest).all()) and bool((rest > 0).all())


def test_eight_row_tiles_a_matrix_kernel_can_load_go_there(gpu_lib):
    # More than 4 rows make this kernel VALU bound; 8x16x2 int8 tiles are 16 bytes per k step, which the matrix
    # kernels load directly.
    run_case(gpu_lib, S8, 1, 40, 64, 8, 16, 2, "mmt4d_mfma_64x64", accumulate=True)
    run_case(gpu_lib, BF16, 1, 40, 64, 8, 16, 1, "mmt4d_mfma_64x64")
    # ... unless it cannot (lhs rows only 8-byte aligned)
    run_case(gpu_lib, S8, 1, 40, 64, 8, 16, 2, "mmt4d_skinny", offsets=(8, 0, 0))


def run_s16_case(gpu_lib, u4, M, N, K, M0, N0, K0, accumulate, expect_kernel, seed=0):
    """s16s16s32, s16u4s32 (u4 True) or s16s8s32 (u4 "s8") against an exact float64 product (values small enough
    that no int32 sum wraps)."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    lhs = torch.randint(-300, 301, (M * K * M0 * K0,), dtype=torch.int16, device="cuda", generator=g)
    if u4 == "s8":
        rhs = torch.randint(-128, 128, (N * K * N0 * K0,), dtype=torch.int8, device="cuda", generator=g)
        b = rhs.view(N, K, N0, K0)
    elif u4:
        packed = torch.randint(0, 256, (N * K * N0 * K0 // 2,), dtype=torch.uint8, device="cuda", generator=g)
        b = torch.stack([packed & 0xF, packed >> 4], dim=-1).reshape(N, K, N0, K0)  # element 2j in the low nibble of byte j
        rhs = packed
    else:
        rhs = torch.randint(-300, 301, (N * K * N0 * K0,), dtype=torch.int16, device="cuda", generator=g)
        b = rhs.view(N, K, N0, K0)
    out = torch.randint(-1000, 1000, (M * N * M0 * N0,), dtype=torch.int32, device="cuda", generator=g)
    before = out.clone()
    kind = abi.MMT4D_TYPE_S16S8S32 if u4 == "s8" else (abi.MMT4D_TYPE_S16U4S32 if u4 else abi.MMT4D_TYPE_S16S16S32)
    flags = kind | (abi.MMT4D_ACCUMULATE if accumulate else 0)
    p = mm_params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0, flags)
    gpu_lib.iree_uk_mmt4d_p(C.byref(p))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == expect_kernel.encode()
    a2 = lhs.view(M, K, M0, K0).permute(0, 2, 1, 3).reshape(M * M0, K * K0).double()
    b2 = b.permute(0, 2, 1, 3).reshape(N * N0, K * K0).double()
    ref = a2 @ b2.t()
    if accumulate:
        ref = ref + before.view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0).double()
    got = out.view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0)
    assert torch.equal(got.long(), ref.long())


# The x86-64 VNNI tiles for 16-bit activations: s16s16s32 Mx16x2 / Mx8x2 and s16u4s32 1x32x8 (mmt4d_x86_64_tiles.inl).
@pytest.mark.parametrize("u4,M,M0,N0,K0", [(False, 1, 1, 16, 2), (False, 1, 4, 16, 2), (False, 3, 2, 8, 2), (False, 1, 8, 16, 2),
                                           (False, 1, 1, 8, 1), (False, 1, 2, 4, 4), (True, 1, 1, 32, 8), (True, 1, 4, 32, 8),
                                           (True, 5, 1, 16, 8), (True, 1, 2, 4, 8)])
def test_sixteen_bit_integer_types(gpu_lib, u4, M, M0, N0, K0):
    for n, K in enumerate((1, 50, 1100)):
        run_s16_case(gpu_lib, u4, M, 23 + n, K, M0, N0, K0, bool(n & 1), "mmt4d_skinny", seed=K + M0)


# s16s8s32: the reference has the generic tile function only (mmt4d_tile_generic.c:145-176, tested on 7x5x6 tiles,
# tools/mmt4d_test.c:550); power-of-two tiles with 2, 4 or 8 rhs bytes per k step run here, any number of rows.
@pytest.mark.parametrize("M,M0,N0,K0", [(1, 1, 16, 2), (1, 4, 8, 2), (3, 2, 16, 2), (1, 1, 8, 4), (1, 8, 4, 4), (2, 4, 16, 4),
                                        (1, 1, 2, 8), (1, 2, 8, 8), (5, 4, 4, 8), (2, 16, 16, 2)])
def test_sixteen_bit_lhs_eight_bit_rhs(gpu_lib, M, M0, N0, K0):
    for n, K in enumerate((1, 50, 1100)):
        run_s16_case(gpu_lib, "s8", M, 23 + n, K, M0, N0, K0, bool(n & 1), "mmt4d_skinny", seed=K + M0 + K0)


def test_sixteen_bit_lhs_eight_bit_rhs_extreme_values(gpu_lib, oracle_lib):
    # -32768 x -128 and 32767 x -128 in every position: the widening of the rhs bytes must keep their sign, the sums
    # wrap in int32 exactly as the reference's (mmt4d_tile_generic.c:145-176 accumulates in int32).
    import numpy as np
    M0, N0, K0, N, K = 4, 8, 4, 3, 600
    lhs = np.full(K * M0 * K0, -32768, np.int16)
    lhs[1::2] = 32767
    rhs = np.full(N * K * N0 * K0, -128, np.int8)
    rhs[::3] = 127
    rhs[1::7] = -1
    want = np.zeros(N * M0 * N0, np.int32)
    flags = abi.MMT4D_TYPE_S16S8S32
    oracle_lib.oracle_mmt4d(C.byref(mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, 1, N, K, M0, N0, K0,
                                              flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK)))
    d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
    d_o = torch.zeros(want.size, dtype=torch.int32, device="cuda")
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), 1, N, K, M0, N0, K0, flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_skinny"
    assert np.array_equal(d_o.cpu().numpy(), want)


# int4 weights in the Arm tiles (s8s4s32 Mx16x2 baseline, Mx8x8 with dot products, Mx8x16 with i8mm;
# mmt4d_arm_64_tiles.inl:50-59).
@pytest.mark.parametrize("M,M0,N0,K0", [(1, 1, 8, 8), (1, 2, 8, 8), (1, 4, 8, 8), (1, 8, 8, 8), (1, 1, 8, 16), (1, 4, 8, 16),
                                        (3, 1, 16, 16), (2, 2, 4, 8), (1, 1, 16, 2), (1, 2, 16, 2), (1, 4, 16, 2),
                                        (3, 4, 16, 2), (1, 1, 32, 2), (3, 8, 8, 8)])
def test_int4_weights_in_narrow_tiles(gpu_lib, M, M0, N0, K0):
    S8S4 = abi.MMT4D_TYPE_S8S4S32
    for n, K in enumerate((1, 33, 700)):
        run_case(gpu_lib, S8S4, M, 29 + n, K, M0, N0, K0, "mmt4d_skinny", accumulate=bool(n & 1), seed=K + K0)
    # strided with offsets (in 4-bit elements on the rhs side)
    run_case(gpu_lib, S8S4, M, 21, 40, M0, N0, K0, "mmt4d_skinny", lhs_pad=16, rhs_pad=64, out_pad=4, offsets=(16, 96, 4),
             accumulate=True, seed=3)


# int8 Mx8x1, the Arm tiles without dot products (mmt4d_arm_64_tiles.inl:38-40): a k step of the rhs is 8 bytes, two
# per lane. Even K, odd K (the stream ends inside a lane's 16 bytes; rhs tile rows padded to 16-byte multiples), more
# rows than one slab, strides and offsets, accumulate.
@pytest.mark.parametrize("M,M0", [(1, 1), (1, 2), (1, 4), (3, 1), (5, 4)])
def test_int8_one_byte_pieces_in_tiles_of_up_to_four_rows(gpu_lib, M, M0):
    for n, K in enumerate((2, 64, 130, 2000)):
        run_case(gpu_lib, S8, M, 33 + n, K, M0, 8, 1, "mmt4d_skinny", accumulate=bool(n & 1), seed=K + M0)
    for n, K in enumerate((1, 77, 1501)):
        run_case(gpu_lib, S8, M, 21 + n, K, M0, 8, 1, "mmt4d_skinny", rhs_pad=8, accumulate=not (n & 1), seed=K)
    run_case(gpu_lib, S8, M, 19, 131, M0, 8, 1, "mmt4d_skinny", lhs_pad=3, rhs_pad=24, out_pad=5, offsets=(5, 48, 3),
             accumulate=True, seed=11)
    # rhs tile rows that are not 16-byte multiples apart: the generic kernel
    run_case(gpu_lib, S8, M, 7, 77, M0, 8, 1, "mmt4d_generic")


def test_sixteen_bit_integer_types_with_more_rows_are_worked_off_in_slabs(gpu_lib):
    # No matrix kernel exists for them: any number of rows goes through this kernel eight rows at a time, also the
    # 16-row tiles of the x86-64 VNNI target (s16s16s32 16x16x2, mmt4d_x86_64_tiles.inl:69,74).
    run_s16_case(gpu_lib, False, 2, 9, 20, 8, 16, 2, True, "mmt4d_skinny")
    run_s16_case(gpu_lib, False, 5, 33, 300, 16, 16, 2, False, "mmt4d_skinny", seed=4)      # 80 rows
    run_s16_case(gpu_lib, False, 3, 7, 64, 16, 8, 2, True, "mmt4d_skinny", seed=5)          # 48 rows, 8-row rhs tiles
    run_s16_case(gpu_lib, False, 13, 5, 64, 1, 16, 2, True, "mmt4d_skinny", seed=6)         # 13 rows: slabs of 8 + 5
    run_s16_case(gpu_lib, True, 1, 9, 20, 16, 32, 8, False, "mmt4d_skinny", seed=7)
    run_s16_case(gpu_lib, True, 21, 9, 40, 1, 32, 8, True, "mmt4d_skinny", seed=8)


def test_more_rows_than_one_slab_and_what_falls_through(gpu_lib):
    # 9 rows of 1x16x2 int8 tiles: no matrix kernel loads such an lhs; two slabs (8 + 1 rows) here.
    run_case(gpu_lib, S8, 9, 20, 40, 1, 16, 2, "mmt4d_skinny", accumulate=True)
    run_case(gpu_lib, F32, 19, 20, 40, 1, 8, 1, "mmt4d_skinny")
    # rhs tile rows that are not 16-byte aligned: the generic kernel, still exact
    run_case(gpu_lib, S8, 1, 20, 40, 1, 16, 2, "mmt4d_generic", rhs_pad=2)
