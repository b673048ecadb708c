"""GPU parity for the 256x256 block tile's staggered tail (mmt4d_mfma_kernels.h: the last three chunks of K are
multiplied fragment by fragment out of the LDS ring and each pair of fragments is stored while the next is
multiplied), which takes every problem on that tile whose K is whole 64-byte chunks, eight or more. The cases
walk what the tail depends on: the number of chunks (the steps before the tail are odd or even in number),
every row-piece layout it is instantiated for (64-, 16-, 8-, 4- and 1-byte pieces, tiles one row tall),
rows and columns that end inside a block tile, accumulate (a variant of its own), strided output rows and
16-bit outputs. Problems are large enough for the cost model to pick the 256x256 tile, so the whole output is
compared with the row-major product computed by torch in float64 (exact for these integers; semantics
mmt4d_tile_generic.c:54-78, 199-225, 289-315) and sampled rows of lhs tiles with the oracle; integer results
bit for bit, floats on small-integer data bit for bit as well (tools/util.c:133-146).
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi
from test_gpu_configs import gpu_lib, mm_params, oracle_tile_rows  # noqa: F401

pytestmark = pytest.mark.gpu

S8, F16, BF16 = abi.MMT4D_TYPE_S8S8S32, abi.MMT4D_TYPE_F16F16F32, abi.MMT4D_TYPE_BF16BF16F32
F16F16, SKIP = abi.MMT4D_TYPE_F16F16F16, abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS

CASES = [
    # flags, rows, cols, M0, N0, K0, K (tiles)      rows x cols large enough for the 256x256 tile
    (S8, 3584, 3584, 8, 8, 4, 128),       # 8 chunks: five steps, then the tail
    (S8, 3584, 3584, 8, 8, 4, 144),       # 9 chunks: six steps
    (S8, 3500, 3600, 8, 8, 4, 176),       # rows and columns end inside a block tile
    (S8, 3584, 3584, 16, 16, 64, 10),     # 64-byte row pieces
    (S8, 3504, 3632, 16, 16, 16, 44),     # 16-byte row pieces, 11 chunks, ragged
    (S8, 3584, 3584, 8, 8, 8, 72),        # 8-byte row pieces
    (S8, 3584, 3584, 8, 8, 1, 512),       # 1-byte row pieces (k-major tiles)
    (S8, 3501, 3584, 1, 16, 64, 9),       # tiles one row tall: row-major lhs and result
    (F16, 3584, 3584, 16, 16, 16, 18),    # 9 chunks of 32 halves
    (BF16, 3520, 3616, 16, 16, 8, 40),    # 10 chunks
    (F16F16 | SKIP, 3584, 3584, 16, 16, 16, 16),   # 16-bit output, one rounding at the end
    # 36 chunks and more: an accumulating call reads the destination during the main loop, a pair of fragments per
    # phase, instead of in the tail.
    (S8, 3584, 3584, 8, 8, 4, 576),       # 36 chunks: the fewest (an odd number of main steps, four per phase)
    (S8, 3500, 3600, 8, 8, 4, 592),       # 37 chunks, rows and columns end inside a block tile
    (S8, 3584, 3584, 16, 16, 64, 45),     # 45 chunks: steps left over after the eight phases
    (S8, 3501, 3584, 1, 16, 64, 40),      # row-major lhs and result
    (S8, 3584, 3584, 8, 8, 1, 2432),      # 1-byte row pieces, 38 chunks
    (F16, 3584, 3584, 16, 16, 16, 80),    # 40 chunks
    (BF16, 3520, 3616, 16, 16, 8, 200),   # 50 chunks, ragged
    (F16F16 | SKIP, 3584, 3584, 16, 16, 16, 76),   # 16-bit output: 8-byte quads
]


@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "t%x_%dx%d_%dx%dx%d_K%d" % c)
def test_staggered_tail(gpu_lib, oracle_lib, case, accumulate):
    flags, rows, cols, M0, N0, K0, K = case
    kind = flags & 0xFF
    M, N = -(-rows // M0), -(-cols // N0)
    g = torch.Generator(device="cuda").manual_seed(rows * 3 + cols + K + (7 if accumulate else 0))
    if kind == S8:
        in_dtype, out_dtype = torch.int8, torch.int32
        a = torch.randint(-128, 128, (M * M0, K * K0), dtype=in_dtype, device="cuda", generator=g)
        b = torch.randint(-128, 128, (N * N0, K * K0), dtype=in_dtype, device="cuda", generator=g)
        init = torch.randint(-2 ** 31, 2 ** 31 - 1, (M * M0, N * N0), dtype=torch.int64, device="cuda", generator=g).to(out_dtype)
    else:
        in_dtype = torch.bfloat16 if kind == BF16 else torch.float16
        out_dtype = torch.float16 if kind == F16F16 else torch.float32
        a = torch.randint(-3, 4, (M * M0, K * K0), device="cuda", generator=g).to(in_dtype)
        b = torch.randint(-3, 4, (N * N0, K * K0), device="cuda", generator=g).to(in_dtype)
        init = torch.randint(-100, 100, (M * M0, N * N0), device="cuda", generator=g).to(out_dtype)
    lhs = a.view(M, M0, K, K0).permute(0, 2, 1, 3).contiguous()
    rhs = b.view(N, N0, K, K0).permute(0, 2, 1, 3).contiguous()
    # Output rows of tiles with a gap of 16 elements between them; the gaps must survive.
    out_stride = N * M0 * N0 + 16
    out = torch.full((M, out_stride), 77, dtype=out_dtype, device="cuda")
    out[:, :N * M0 * N0] = init.view(M, M0, N, N0).permute(0, 2, 1, 3).reshape(M, N * M0 * N0)
    p = mm_params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0,
                  flags | (abi.MMT4D_ACCUMULATE if accumulate else 0), out_stride=out_stride)
    gpu_lib.iree_uk_mmt4d_p(C.byref(p))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_mfma_256x256"
    assert bool((out[:, N * M0 * N0:] == 77).all()), "gap between rows of tiles written"
    got = out[:, :N * M0 * N0].view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0)
    want = a.double() @ b.double().t()
    if accumulate:
        want = want + init.double()
    if kind == S8:
        want = (want.long() + 2 ** 31) % 2 ** 32 - 2 ** 31      # int32 wrap-around
        assert torch.equal(got.long(), want)
    else:
        # small integers: exact in f32 in any order; |values| < 2048 are exact in f16 too
        assert torch.equal(got.double(), want)
    # A sample of rows of lhs tiles against the oracle as well.
    if kind in (S8, F16, BF16):
        to_np = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16) if t.dtype in (torch.float16, torch.bfloat16) \
            else t.cpu().numpy()
        lhs_h, rhs_h = to_np(lhs).reshape(-1), to_np(rhs).reshape(-1)
        init_h = init.view(M, M0, N, N0).permute(0, 2, 1, 3).reshape(-1).cpu().numpy() if accumulate else \
            np.zeros(M * N * M0 * N0, dtype=np.int32 if kind == S8 else np.float32)
        sample = [0, M // 2, M - 1]
        ref = oracle_tile_rows(oracle_lib, sample, lhs_h, rhs_h, init_h, M, N, K, M0, N0, K0,
                               flags | (abi.MMT4D_ACCUMULATE if accumulate else 0))
        got_h = out[:, :N * M0 * N0].cpu().numpy()
        for i in sample:
            assert np.array_equal(got_h[i], ref[i]), "row of tiles %d differs from the oracle" % i
