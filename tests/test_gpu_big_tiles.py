"""The large block tiles of the MFMA kernels (256x256 and 128x128 per
workgroup) on shapes that do not divide into them: ragged last block rows and
columns, K that ends inside a 64-byte chunk, strided operands with offsets,
accumulation. The reference's own test grid only reaches the smallest block
tile; the benchmark configurations only exact multiples.

Integer results are compared bit for bit with a float64 matrix product of the
same operands (every value is far below 2^53, so that product is exact); float
results within |got - ref| <= 1e-3 * max(|ref|, rms(ref)) of it.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi
from test_gpu_configs import REL_TOL, gpu_lib, mm_params  # noqa: F401

pytestmark = pytest.mark.gpu


def logical(t, outer, K, T0, K0):
    """[outer][K][T0][K0] tiled operand -> [outer*T0, K*K0] float64."""
    return t.view(outer, K, T0, K0).permute(0, 2, 1, 3).reshape(outer * T0, K * K0).double()


def run_case(gpu_lib, flags, M, N, K, M0, N0, K0, expect_kernel, lhs_pad=0, rhs_pad=0, out_pad=0, offsets=(0, 0, 0),
             accumulate=False, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    kind = flags & 0xFF
    lhs_stride, rhs_stride, out_stride = K * M0 * K0 + lhs_pad, K * N0 * K0 + rhs_pad, N * M0 * N0 + out_pad
    lo, ro, oo = offsets

    def operand(n_tiles, stride, off, T0):
        if kind in (abi.MMT4D_TYPE_S8S8S32, abi.MMT4D_TYPE_S8S4S32):
            return torch.randint(-128, 128, (off + n_tiles * stride,), dtype=torch.int8, device="cuda", generator=g)
        dt = {abi.MMT4D_TYPE_F16F16F32: torch.float16, abi.MMT4D_TYPE_BF16BF16F32: torch.bfloat16,
              abi.MMT4D_TYPE_F32F32F32: torch.float32, abi.MMT4D_TYPE_F16F16F16: torch.float16,
              abi.MMT4D_TYPE_BF16BF16BF16: torch.bfloat16}[kind]
        return (torch.randn(off + n_tiles * stride, device="cuda", generator=g) / 8).to(dt)

    lhs = operand(M, lhs_stride, lo, M0)
    if kind == abi.MMT4D_TYPE_S8S4S32:
        # packed nibbles: strides and offsets are in 4-bit elements
        rhs_bytes = torch.randint(-128, 128, ((ro + N * rhs_stride) // 2,), dtype=torch.int8, device="cuda", generator=g)
        rhs = rhs_bytes
    else:
        rhs = operand(N, rhs_stride, ro, N0)
    is_int = kind in (abi.MMT4D_TYPE_S8S8S32, abi.MMT4D_TYPE_S8S4S32)
    # 16-bit outputs reach the matrix pipe only with the roundings between k steps skipped; one final rounding then.
    narrow = {abi.MMT4D_TYPE_F16F16F16: (torch.float16, 2.0 ** -10), abi.MMT4D_TYPE_BF16BF16BF16: (torch.bfloat16, 2.0 ** -7)}
    out_ulp = narrow[kind][1] if kind in narrow else 0.0
    if kind in narrow:
        flags |= abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
    if is_int:
        out = torch.randint(-1000, 1000, (oo + M * out_stride,), dtype=torch.int32, device="cuda", generator=g)
    else:
        out = torch.randn(oo + M * out_stride, device="cuda", generator=g)
        if kind in narrow:
            out = out.to(narrow[kind][0])
    before = out.clone()
    p = mm_params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0,
                  flags | (abi.MMT4D_ACCUMULATE if accumulate else 0), lhs_off=lo, rhs_off=ro, out_off=oo,
                  lhs_stride=lhs_stride, rhs_stride=rhs_stride, out_stride=out_stride)
    gpu_lib.iree_uk_mmt4d_p(C.byref(p))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == expect_kernel.encode()

    def rows_of(buf, off, n_tiles, stride, width):
        return buf[off:off + n_tiles * stride].view(n_tiles, stride)[:, :width]

    a = logical(rows_of(lhs, lo, M, lhs_stride, K * M0 * K0).contiguous(), M, K, M0, K0)
    if kind == abi.MMT4D_TYPE_S8S4S32:
        nib = rhs_bytes[ro // 2:(ro + N * rhs_stride) // 2].view(N, rhs_stride // 2)[:, :K * N0 * K0 // 2].contiguous()
        u = nib.view(torch.uint8).to(torch.int16)
        low = ((u & 0xF) ^ 8) - 8
        high = ((u >> 4) ^ 8) - 8
        vals = torch.stack([low, high], dim=-1).reshape(N, K * N0 * K0)
        b = logical(vals, N, K, N0, K0)
    else:
        b = logical(rows_of(rhs, ro, N, rhs_stride, K * N0 * K0).contiguous(), N, K, N0, K0)
    ref = a @ b.t()
    if accumulate:
        c0 = rows_of(before, oo, M, out_stride, N * M0 * N0).reshape(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0)
        ref = ref + c0.double()
    got = rows_of(out, oo, M, out_stride, N * M0 * N0).reshape(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0)
    if is_int:
        assert torch.equal(got.long(), ref.long())
    else:
        rms = ref.pow(2).mean().sqrt()
        assert bool(((got.double() - ref).abs() <= (REL_TOL + out_ulp) * torch.maximum(ref.abs(), rms)).all())
    # Nothing outside the output tiles was written: the gaps between tile rows and the prefix.
    if out_pad:
        gaps = out[oo:oo + M * out_stride].view(M, out_stride)[:, N * M0 * N0:]
        assert torch.equal(gaps, before[oo:oo + M * out_stride].view(M, out_stride)[:, N * M0 * N0:])
    assert torch.equal(out[:oo], before[:oo])


# (M, N) in tiles chosen so that 256x256 blocks give >= 200 workgroups with a ragged last row and column.
@pytest.mark.parametrize("K,accumulate", [(48, False), (40, True), (16, True)])
def test_s8s8s32_8x8x4_ragged_256(gpu_lib, K, accumulate):
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 451, 463, K, 8, 8, 4, "mmt4d_mfma_256x256", accumulate=accumulate, seed=K)


def test_s8s8s32_8x8x4_ragged_256_strided_with_offsets(gpu_lib):
    # pads keep every tile row 16-byte aligned (the direct kernel), offsets are multiples of 16 elements
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 451, 463, 48, 8, 8, 4, "mmt4d_mfma_256x256", lhs_pad=64, rhs_pad=32,
             out_pad=12, offsets=(32, 48, 8), accumulate=True, seed=3)
    # 4-byte aligned only: the register-staged kernel
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 451, 463, 48, 8, 8, 4, "mmt4d_mfma_256x256", lhs_pad=4, rhs_pad=12,
             out_pad=4, offsets=(4, 20, 4), seed=4)


@pytest.mark.parametrize("M0,N0,K0,K", [(16, 16, 64, 3), (16, 8, 16, 9), (4, 16, 32, 5)])
def test_s8s8s32_wide_pieces_ragged_256(gpu_lib, M0, N0, K0, K):
    M, N = 3608 // M0 + 1, 3704 // N0 + 1
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, M, N, K, M0, N0, K0, "mmt4d_mfma_256x256", accumulate=True, seed=K0)


@pytest.mark.parametrize("M,N", [(100, 119), (131, 67)])
def test_s8s8s32_ragged_128(gpu_lib, M, N):
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, M, N, 32, 16, 16, 16, "mmt4d_mfma_128x128", out_pad=20, accumulate=True, seed=M)
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 2 * M, 2 * N, 19, 8, 8, 4, "mmt4d_mfma_128x128", seed=N)


@pytest.mark.parametrize("flags,M0,N0,K0,K", [(abi.MMT4D_TYPE_F16F16F32, 16, 16, 16, 10), (abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 8, 13),
                                              (abi.MMT4D_TYPE_F16F16F32, 8, 8, 2, 48), (abi.MMT4D_TYPE_F32F32F32, 16, 16, 4, 11),
                                              (abi.MMT4D_TYPE_F32F32F32, 8, 8, 1, 33), (abi.MMT4D_TYPE_F16F16F16, 16, 16, 16, 6),
                                              (abi.MMT4D_TYPE_BF16BF16BF16, 8, 16, 2, 40)])
def test_float_types_ragged_256(gpu_lib, flags, M0, N0, K0, K):
    M, N = 3608 // M0 + 1, 3704 // N0 + 1
    run_case(gpu_lib, flags, M, N, K, M0, N0, K0, "mmt4d_mfma_256x256", accumulate=True, out_pad=16, seed=K)


@pytest.mark.parametrize("M,N,expect,expect_staged", [(226, 232, "mmt4d_mfma_256x256", "mmt4d_mfma_256x256"),
                                                      (100, 119, "mmt4d_mfma_128x128", "mmt4d_mfma_128x128"),
                                                      (9, 11, "mmt4d_mfma_64x128", "mmt4d_mfma_64x64")])
def test_s8s4s32_ragged(gpu_lib, M, N, expect, expect_staged):
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S4S32, M, N, 6, 16, 16, 32, expect, accumulate=True, rhs_pad=64, offsets=(16, 64, 4), seed=M)
    # 8-byte rhs pieces: the register-staged kernel, which has a 64x64 tile.
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S4S32, M, N, 5, 16, 16, 16, expect_staged, seed=N)


# The two oblong block tiles, picked for tall-and-narrow problems (few lhs rows against many rhs rows).
@pytest.mark.parametrize("flags,M0,N0,K0,K", [(abi.MMT4D_TYPE_S8S8S32, 4, 8, 4, 32), (abi.MMT4D_TYPE_S8S8S32, 4, 16, 16, 12),
                                              (abi.MMT4D_TYPE_F16F16F32, 4, 16, 16, 6), (abi.MMT4D_TYPE_BF16BF16F32, 4, 16, 8, 12),
                                              (abi.MMT4D_TYPE_F32F32F32, 4, 16, 4, 8)])
def test_oblong_tiles_ragged(gpu_lib, flags, M0, N0, K0, K):
    n_cols = 14300 // N0 * N0
    run_case(gpu_lib, flags, 500 // M0, n_cols // N0, K, M0, N0, K0, "mmt4d_mfma_256x128", accumulate=True, out_pad=8, seed=K)
    run_case(gpu_lib, flags, 120 // M0, n_cols // N0, K, M0, N0, K0, "mmt4d_mfma_128x64", seed=K + 1)


# Row pieces of 2 and 8 bytes: the tile shapes the reference's CPU targets use (x86-64 int8 16x16x2 and 8x8x2,
# f16 16x16x1; Arm int8 8x8x8, bf16 8x8x4; mmt4d_x86_64_tiles.inl, mmt4d_arm_64_tiles.inl), i.e. what a module
# compiled for such a CPU passes in. K is a multiple of the 64-byte chunk, as the direct-to-LDS kernel needs.
@pytest.mark.parametrize("flags,M0,N0,K0,K", [
    (abi.MMT4D_TYPE_S8S8S32, 16, 16, 2, 96), (abi.MMT4D_TYPE_S8S8S32, 8, 8, 2, 64), (abi.MMT4D_TYPE_S8S8S32, 8, 8, 8, 24),
    (abi.MMT4D_TYPE_S8S8S32, 2, 8, 8, 8), (abi.MMT4D_TYPE_F16F16F32, 16, 16, 1, 64), (abi.MMT4D_TYPE_F16F16F32, 8, 8, 4, 16),
    (abi.MMT4D_TYPE_BF16BF16F32, 8, 8, 4, 24), (abi.MMT4D_TYPE_BF16BF16F32, 16, 8, 1, 96), (abi.MMT4D_TYPE_F32F32F32, 8, 8, 2, 24),
    (abi.MMT4D_TYPE_BF16BF16BF16, 8, 8, 4, 24), (abi.MMT4D_TYPE_F16F16F16, 8, 8, 1, 32)])
def test_narrow_and_8_byte_row_pieces(gpu_lib, flags, M0, N0, K0, K):
    # 256x256 blocks, ragged in both directions, accumulating, padded output rows
    M, N = 3608 // M0 + 1, 3704 // N0 + 1
    run_case(gpu_lib, flags, M, N, K, M0, N0, K0, "mmt4d_mfma_256x256", accumulate=True, out_pad=16, seed=K0 + K)
    # the smallest block tile, strided operands with offsets (all multiples of 16 bytes)
    run_case(gpu_lib, flags, 72 // M0, 88 // N0, K, M0, N0, K0, "mmt4d_mfma_64x64", lhs_pad=32, rhs_pad=16,
             offsets=(16, 32, 4), seed=K0)


# 2-byte row pieces feed the matrix pipe in interleaved pairs of fragments wherever a wavefront owns an even number of
# fragments of an operand (rows 2r / 2r+1 of 64 from one dword), which the epilogue has to undo: every block tile, with
# the lhs paired and the rhs not (128x64), ragged edges that cut pairs apart, accumulation and padded output rows.
@pytest.mark.parametrize("flags,M0,N0,K0,K", [(abi.MMT4D_TYPE_S8S8S32, 16, 16, 2, 64), (abi.MMT4D_TYPE_S8S8S32, 8, 8, 2, 32),
                                              (abi.MMT4D_TYPE_F16F16F32, 16, 16, 1, 96), (abi.MMT4D_TYPE_BF16BF16F32, 8, 16, 1, 32),
                                              (abi.MMT4D_TYPE_F16F16F16, 16, 16, 1, 32), (abi.MMT4D_TYPE_BF16BF16BF16, 16, 8, 1, 64)])
def test_two_byte_row_pieces_on_every_block_tile(gpu_lib, flags, M0, N0, K0, K):
    n_cols = 14300 // N0 * N0
    run_case(gpu_lib, flags, 504 // M0, n_cols // N0, K, M0, N0, K0, "mmt4d_mfma_256x128", accumulate=True, out_pad=8, seed=K)
    run_case(gpu_lib, flags, 120 // M0, n_cols // N0, K, M0, N0, K0, "mmt4d_mfma_128x64", seed=K + 1)
    run_case(gpu_lib, flags, 1608 // M0, 1912 // N0, K, M0, N0, K0, "mmt4d_mfma_128x128", accumulate=True, seed=K + 2)
    run_case(gpu_lib, flags, 3608 // M0 + 1, 3704 // N0 + 1, K, M0, N0, K0, "mmt4d_mfma_256x256", lhs_pad=32, rhs_pad=16,
             out_pad=12, offsets=(16, 32, 4), seed=K + 3)


def test_narrow_row_pieces_fall_back_when_the_direct_kernel_cannot_run(gpu_lib):
    # Less than one 64-byte chunk of K, or rows not 16-byte aligned: the skinny kernel's 8-row slabs, still exact.
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 9, 11, 31, 16, 16, 2, "mmt4d_skinny", accumulate=True)
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 9, 11, 32, 16, 16, 2, "mmt4d_skinny", lhs_pad=4)
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 9, 11, 33, 16, 16, 2, "mmt4d_mfma_64x64", accumulate=True)


# K ending inside a 64-byte chunk on the direct-to-LDS kernel: the last chunk overlaps the one before it and the
# overlap is zeroed in the fragments. Every row piece size, cuts at every granularity (an odd number of k steps,
# cuts inside a lane's 16 bytes and at 16- and 32-byte boundaries), one chunk plus a bit, every block tile.
@pytest.mark.parametrize("flags,M0,N0,K0,Ks", [
    (abi.MMT4D_TYPE_S8S8S32, 8, 8, 4, (17, 21, 24, 27, 31, 45)), (abi.MMT4D_TYPE_S8S8S32, 16, 16, 2, (33, 40, 47, 49, 63, 95)),
    (abi.MMT4D_TYPE_S8S8S32, 8, 8, 8, (9, 11, 13, 22)), (abi.MMT4D_TYPE_S8S8S32, 16, 16, 16, (5, 6, 7, 9)),
    (abi.MMT4D_TYPE_S8S8S32, 16, 8, 32, (3, 5)), (abi.MMT4D_TYPE_F16F16F32, 16, 16, 1, (33, 50, 77)),
    (abi.MMT4D_TYPE_F16F16F32, 16, 16, 16, (3, 5)), (abi.MMT4D_TYPE_BF16BF16F32, 8, 8, 4, (9, 15, 20)),
    (abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 2, (17, 30)), (abi.MMT4D_TYPE_F32F32F32, 16, 16, 4, (5, 6, 7)),
    (abi.MMT4D_TYPE_F32F32F32, 8, 8, 1, (17, 33)), (abi.MMT4D_TYPE_F32F32F32, 8, 16, 2, (9, 13))])
def test_direct_kernel_with_K_ending_inside_a_chunk(gpu_lib, flags, M0, N0, K0, Ks):
    n_cols = 14300 // N0 * N0
    for n, K in enumerate(Ks):
        tile = n % 4
        if tile == 0:
            run_case(gpu_lib, flags, 3608 // M0 + 1, 3704 // N0 + 1, K, M0, N0, K0, "mmt4d_mfma_256x256", accumulate=True,
                     out_pad=16, seed=K)
        elif tile == 1:
            run_case(gpu_lib, flags, 504 // M0, n_cols // N0, K, M0, N0, K0, "mmt4d_mfma_256x128", lhs_pad=32, rhs_pad=16,
                     offsets=(16, 32, 4), seed=K)
        elif tile == 2:
            run_case(gpu_lib, flags, 120 // M0, n_cols // N0, K, M0, N0, K0, "mmt4d_mfma_128x64", accumulate=True, seed=K)
        else:
            run_case(gpu_lib, flags, 1608 // M0, 1912 // N0, K, M0, N0, K0, "mmt4d_mfma_128x128", seed=K)
        run_case(gpu_lib, flags, 72 // M0, 88 // N0, K, M0, N0, K0, "mmt4d_mfma_64x64", accumulate=True, seed=K + 100)


def test_K_tail_overlap_is_zeroed_in_both_operands(gpu_lib):
    # The chunk that K ends in is loaded overlapping the one before it. An infinity inside the overlap must count
    # once: were only one operand zeroed there, inf * 0 would turn the outputs into NaN.
    M, N, K, M0, N0, K0 = 5, 6, 5, 16, 16, 16      # 32-byte row pieces: chunks [k0,k1], [k2,k3], tail k4 -> the last chunk is [k3,k4]
    g = torch.Generator(device="cuda").manual_seed(1)
    lhs = (torch.rand(M * K * M0 * K0, device="cuda", generator=g) + 0.5).to(torch.float16)
    rhs = (torch.rand(N * K * N0 * K0, device="cuda", generator=g) + 0.5).to(torch.float16)
    lhs.view(M, K, M0, K0)[0, 3, 0, 7] = float("inf")      # logical row 0, k step 3
    rhs.view(N, K, N0, K0)[1, 3, 5, 2] = float("inf")      # logical column 21, k step 3
    out = torch.zeros(M * N * M0 * N0, device="cuda")
    p = mm_params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0, abi.MMT4D_TYPE_F16F16F32)
    gpu_lib.iree_uk_mmt4d_p(C.byref(p))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_mfma_64x64"
    got = out.view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0)
    assert not bool(torch.isnan(got).any())
    inf = torch.isinf(got)
    want = torch.zeros_like(inf)
    want[0, :] = True
    want[:, 21] = True
    assert torch.equal(inf, want)
    finite = got[1:, :21]
    ref = logical(lhs, M, K, M0, K0)[1:] @ logical(rhs, N, K, N0, K0)[:21].t()
    assert bool(((finite.double() - ref).abs() <= REL_TOL * ref.abs()).all())


# Few block tiles against a long K: the 64x64 tile whose wavefronts split K (256 bytes of K per row and step) and sum
# their partial tiles at the end. Even and odd numbers of steps, ragged tiles, one tile only, accumulation, strides.
@pytest.mark.parametrize("flags,M0,N0,K0", [(abi.MMT4D_TYPE_S8S8S32, 16, 16, 64), (abi.MMT4D_TYPE_S8S8S32, 8, 8, 16),
                                            (abi.MMT4D_TYPE_S8S8S32, 4, 16, 32), (abi.MMT4D_TYPE_F16F16F32, 16, 16, 16),
                                            (abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 8), (abi.MMT4D_TYPE_BF16BF16F32, 1, 16, 8),
                                            (abi.MMT4D_TYPE_F16F16F16, 16, 16, 8), (abi.MMT4D_TYPE_BF16BF16BF16, 8, 16, 16)])
def test_split_k_tile(gpu_lib, flags, M0, N0, K0):
    e = 1 if flags == abi.MMT4D_TYPE_S8S8S32 else 2
    per_step = 256 // (K0 * e)                      # k steps per 256 bytes of a row
    name = "mmt4d_mfma_64x64_split_k"
    run_case(gpu_lib, flags, 72 // M0 + 1, 88 // N0, 16 * per_step, M0, N0, K0, name, accumulate=True, out_pad=8, seed=1)
    run_case(gpu_lib, flags, 200 // M0, 300 // N0, 17 * per_step, M0, N0, K0, name, lhs_pad=64 // e, rhs_pad=32 // e,
             offsets=(16 // e, 48 // e, 4), seed=2)
    run_case(gpu_lib, flags, max(1, 16 // M0), 48 // N0, 41 * per_step, M0, N0, K0, name, accumulate=True, seed=3)
    # K not whole steps of 256 bytes, or too short to matter: the ordinary 64x64 tile
    run_case(gpu_lib, flags, 72 // M0 + 1, 88 // N0, 16 * per_step + 64 // (K0 * e), M0, N0, K0, "mmt4d_mfma_64x64", seed=4)
    run_case(gpu_lib, flags, max(1, 48 // M0), 88 // N0, 8 * per_step, M0, N0, K0, "mmt4d_mfma_64x64", seed=5)


# The same with one row of 128x64 tiles (65 .. 128 lhs rows against many rhs rows, f16 / bf16): 128 bytes of K per row
# and step.
@pytest.mark.parametrize("flags,M0,N0,K0", [(abi.MMT4D_TYPE_F16F16F32, 16, 16, 16), (abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 8),
                                            (abi.MMT4D_TYPE_BF16BF16F32, 4, 16, 8), (abi.MMT4D_TYPE_F16F16F16, 16, 16, 8),
                                            (abi.MMT4D_TYPE_BF16BF16BF16, 8, 8, 32), (abi.MMT4D_TYPE_F16F16F32, 2, 4, 16)])
def test_split_k_tile_128_rows(gpu_lib, flags, M0, N0, K0):
    e = 2
    per_step = max(1, 128 // (K0 * e))              # k steps per 128 bytes of a row
    name = "mmt4d_mfma_128x64_split_k"
    cols = 9000 // N0
    run_case(gpu_lib, flags, 128 // M0, cols, 64 * per_step, M0, N0, K0, name, accumulate=True, out_pad=8, seed=1)
    run_case(gpu_lib, flags, 100 // M0, cols + 3, 65 * per_step, M0, N0, K0, name, lhs_pad=64 // e, rhs_pad=32 // e,
             offsets=(16 // e, 48 // e, 4), seed=2)
    run_case(gpu_lib, flags, 80 // M0, cols, 97 * per_step, M0, N0, K0, name, accumulate=True, seed=3)
    # 64 rows or fewer, or a K too short to pay for summing the partial tiles: the ordinary tiles
    run_case(gpu_lib, flags, 64 // M0, cols, 64 * per_step, M0, N0, K0, "mmt4d_mfma_64x64", seed=4)
    run_case(gpu_lib, flags, 128 // M0, cols, 32 * per_step, M0, N0, K0, "mmt4d_mfma_128x64", seed=5)


def test_ragged_K_on_the_register_staged_kernel(gpu_lib):
    # 4-byte aligned rows (not 16): the register-staged kernel with its zero-filling tail step.
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S8S32, 451, 463, 37, 8, 8, 4, "mmt4d_mfma_256x256", lhs_pad=4, rhs_pad=12,
             out_pad=4, offsets=(4, 20, 4), accumulate=True, seed=5)
    run_case(gpu_lib, abi.MMT4D_TYPE_BF16BF16F32, 100, 119, 19, 16, 16, 2, "mmt4d_mfma_128x128", lhs_pad=2, rhs_pad=6, seed=6)


# The 64x128 block tile of the int4 rhs, picked for a few dozen lhs rows against many rhs rows.
@pytest.mark.parametrize("M0,rows,K0,K", [(16, 64, 32, 16), (16, 48, 64, 7), (8, 40, 32, 10), (4, 36, 32, 6)])
def test_s8s4s32_64x128_tile_ragged(gpu_lib, M0, rows, K0, K):
    n_tiles = 28600 // 16
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S4S32, rows // M0, n_tiles, K, M0, 16, K0, "mmt4d_mfma_64x128", accumulate=True,
             rhs_pad=64, out_pad=8, offsets=(16, 64, 4), seed=rows)
    run_case(gpu_lib, abi.MMT4D_TYPE_S8S4S32, rows // M0, n_tiles - 3, K, M0, 16, K0, "mmt4d_mfma_64x128", seed=K)
