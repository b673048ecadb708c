"""The chain of the reference's matmul benchmark on the GPU library, through the
C ABI: pack lhs, pack rhs (a [K, N] matrix, both transposes), pack the initial
output when accumulating, mmt4d, unpack (tools/e2e_matmul_benchmark.c:173-186),
at the tile sizes iree_uk_query_tile_sizes_2d returns for each operand role,
on ragged logical sizes, compared bit for bit with the row-major product
(:340-358: "bit-exact compare", which for floats relies on small-integer data
whose sums are exact in any order, tools/util.c:133-146). Every stage must run
on a specialised kernel, so that a mismatch between what the query hands out
and what pack and mmt4d accept together on the fast paths cannot hide behind a
generic fallback.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, library

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu_lib():
    assert torch.cuda.is_available()
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    return lib


def _query(lib, op, role):
    q, o = abi.QueryTileSizes2dParams(), abi.QueryTileSizes2dOutParams()
    q.flags = op | role
    lib.iree_uk_query_tile_sizes_2d(C.byref(q), C.byref(o))
    return o.tile_size0, o.tile_size1


# name -> (query op, mmt4d type, pack type of lhs/rhs, pack + unpack type of out, numpy/torch dtypes)
KINDS = {
    "i8": (abi.QTS_OP_MATMUL_I8I8I32, abi.MMT4D_TYPE_S8S8S32, abi.PACK_TYPE_I8I8, abi.PACK_TYPE_I32I32,
           abi.UNPACK_TYPE_I32I32, torch.int8, torch.int32),
    "f16": (abi.QTS_OP_MATMUL_F16F16F32, abi.MMT4D_TYPE_F16F16F32, abi.PACK_TYPE_F16F16, abi.PACK_TYPE_F32F32,
            abi.UNPACK_TYPE_F32F32, torch.float16, torch.float32),
    "bf16": (abi.QTS_OP_MATMUL_BF16BF16F32, abi.MMT4D_TYPE_BF16BF16F32, abi.PACK_TYPE_BF16BF16, abi.PACK_TYPE_F32F32,
             abi.UNPACK_TYPE_F32F32, torch.bfloat16, torch.float32),
    "f32": (abi.QTS_OP_MATMUL_F32F32F32, abi.MMT4D_TYPE_F32F32F32, abi.PACK_TYPE_F32F32, abi.PACK_TYPE_F32F32,
            abi.UNPACK_TYPE_F32F32, torch.float32, torch.float32),
}


def _pack(src, dst, rows, cols, o0, o1, t0, t1, flags):
    p = abi.PackParams()
    p.in_buffer, p.out_buffer = src.data_ptr(), dst.data_ptr()
    p.in_stride0, p.in_stride1, p.in_size0, p.in_size1 = cols, 1, rows, cols
    p.out_size0, p.out_size1, p.out_size2, p.out_size3 = o0, o1, t0, t1
    p.out_stride0, p.out_stride1 = o1 * t0 * t1, t0 * t1
    p.padding_value = 0
    p.flags = flags
    return p


@pytest.mark.parametrize("kind", ["i8", "f16", "bf16", "f32"])
@pytest.mark.parametrize("M,N,K", [(301, 517, 1000), (1, 4097, 130), (600, 33, 77), (1025, 1023, 2050)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_pack_mmt4d_unpack_equals_row_major_matmul(gpu_lib, kind, M, N, K, accumulate):
    op, mm_type, in_pack, out_pack, out_unpack, in_dtype, out_dtype = KINDS[kind]
    (m0, k0), (n0, k0r), (rm0, rn0) = (_query(gpu_lib, op, r) for r in
                                       (abi.QTS_ROLE_LHS, abi.QTS_ROLE_RHS, abi.QTS_ROLE_RESULT))
    assert k0 == k0r and (rm0, rn0) == (m0, n0)
    M1, N1, K1 = -(-M // m0), -(-N // n0), -(-K // k0)
    g = torch.Generator(device="cuda").manual_seed(M * 7 + N * 3 + K + (1 if accumulate else 0))
    if kind == "i8":
        a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device="cuda", generator=g)
        b = torch.randint(-128, 128, (K, N), dtype=torch.int8, device="cuda", generator=g)
        init = torch.randint(-100000, 100000, (M, N), dtype=torch.int32, device="cuda", generator=g)
    else:
        # Small integers: every product and partial sum is exact in f32 (|sum| <= K * 9 < 2^24).
        a = torch.randint(-3, 4, (M, K), device="cuda", generator=g).to(in_dtype)
        b = torch.randint(-3, 4, (K, N), device="cuda", generator=g).to(in_dtype)
        init = torch.randint(-1000, 1000, (M, N), device="cuda", generator=g).to(out_dtype)
    a4 = torch.full((M1 * K1 * m0 * k0,), 7, dtype=in_dtype, device="cuda")
    b4 = torch.full((N1 * K1 * n0 * k0,), 7, dtype=in_dtype, device="cuda")
    c4 = torch.full((M1 * N1 * m0 * n0,), 7, dtype=out_dtype, device="cuda")
    c = torch.full((M + 1, N + 1), 55, dtype=out_dtype, device="cuda")   # one guard row and column

    kernels = []

    def call(fn, p):
        fn(C.byref(p))
        kernels.append(gpu_lib.iree_uk_mi355x_last_kernel().decode())

    call(gpu_lib.iree_uk_pack_p, _pack(a, a4, M, K, M1, K1, m0, k0, in_pack))
    call(gpu_lib.iree_uk_pack_p, _pack(b, b4, K, N, N1, K1, n0, k0,
                                       in_pack | abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER))
    if accumulate:
        call(gpu_lib.iree_uk_pack_p, _pack(init, c4, M, N, M1, N1, m0, n0, out_pack))
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = a4.data_ptr(), b4.data_ptr(), c4.data_ptr()
    p.lhs_stride0, p.rhs_stride0, p.out_stride0 = K1 * m0 * k0, K1 * n0 * k0, N1 * m0 * n0
    p.M, p.N, p.K, p.M0, p.N0, p.K0 = M1, N1, K1, m0, n0, k0
    p.flags = mm_type | (abi.MMT4D_ACCUMULATE if accumulate else 0)
    call(gpu_lib.iree_uk_mmt4d_p, p)
    u = abi.UnpackParams()
    u.in_buffer, u.out_buffer = c4.data_ptr(), c.data_ptr()
    u.in_size0, u.in_size1, u.in_size2, u.in_size3 = M1, N1, m0, n0
    u.in_stride0, u.in_stride1 = N1 * m0 * n0, m0 * n0
    u.out_size0, u.out_size1, u.out_stride0, u.out_stride1 = M, N, N + 1, 1
    u.flags = out_unpack
    call(gpu_lib.iree_uk_unpack_p, u)

    # No stage on a one-thread-per-element kernel.
    assert all(k and "generic" not in k for k in kernels), kernels
    mm_kernel = kernels[3 if accumulate else 2]
    assert mm_kernel.startswith("mmt4d_mfma") or mm_kernel.startswith("mmt4d_gemv") or \
        mm_kernel.startswith("mmt4d_skinny"), kernels

    want = a.double() @ b.double()
    if accumulate:
        want = want + init.double()
    if kind == "i8":
        want = want.long()
        want = ((want + 2 ** 31) % 2 ** 32 - 2 ** 31)     # int32 wrap-around, like the reference's accumulators
        assert torch.equal(c[:M, :N].long(), want), kernels
    else:
        assert torch.equal(c[:M, :N].double(), want), kernels
    assert bool((c[M, :] == 55).all()) and bool((c[:, N] == 55).all())


@pytest.mark.parametrize("kind", ["i8", "f16", "bf16", "f32"])
@pytest.mark.parametrize("M,N,K", [(301, 517, 1000), (1, 4097, 130), (600, 33, 77), (1025, 1023, 2050), (256, 512, 4096)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_row_major_lhs_and_result_need_no_pack_or_unpack(gpu_lib, kind, M, N, K, accumulate):
    """The fused form of the chain: a row-major [M, K] matrix IS the mmt4d lhs [M][K1][1][K0] (tiles one row
    tall follow each other along the row), and the mmt4d result [M][N1][1][N0] IS the row-major [M, N1*N0]
    matrix, so with M0 = 1 only the rhs is packed (mmt4d.c:12-48 puts no lower bound on M0; operand
    addressing mmt4d.c:55-99). Same comparison as above, tools/e2e_matmul_benchmark.c:340-358. K is padded
    to whole tiles by the row pitch of the lhs; what lies in that padding meets the zero padding of the
    packed rhs."""
    op, mm_type, in_pack, _, _, in_dtype, out_dtype = KINDS[kind]
    (_, k0), (n0, _) = (_query(gpu_lib, op, r) for r in (abi.QTS_ROLE_LHS, abi.QTS_ROLE_RHS))
    N1, K1 = -(-N // n0), -(-K // k0)
    g = torch.Generator(device="cuda").manual_seed(M * 7 + N * 3 + K + (1 if accumulate else 0))
    if kind == "i8":
        a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device="cuda", generator=g)
        b = torch.randint(-128, 128, (K, N), dtype=torch.int8, device="cuda", generator=g)
        init = torch.randint(-100000, 100000, (M, N), dtype=torch.int32, device="cuda", generator=g)
    else:
        a = torch.randint(-3, 4, (M, K), device="cuda", generator=g).to(in_dtype)
        b = torch.randint(-3, 4, (K, N), device="cuda", generator=g).to(in_dtype)
        init = torch.randint(-1000, 1000, (M, N), device="cuda", generator=g).to(out_dtype)
    # lhs rows padded to whole tiles with something that is not zero; one guard row after the matrix.
    a_pitch = K1 * k0
    a_rm = torch.full((M + 1, a_pitch), 7, dtype=in_dtype, device="cuda")
    a_rm[:M, :K] = a
    b4 = torch.full((N1 * K1 * n0 * k0,), 7, dtype=in_dtype, device="cuda")
    # Result: rows of N1*N0 values, pitch with 5 guard columns, one guard row.
    c_pitch = N1 * n0 + 8
    c = torch.full((M + 1, c_pitch), 55, dtype=out_dtype, device="cuda")
    if accumulate:
        c[:M, :N] = init
        c[:M, N:N1 * n0] = 0
    kernels = []

    def call(fn, p):
        fn(C.byref(p))
        kernels.append(gpu_lib.iree_uk_mi355x_last_kernel().decode())

    call(gpu_lib.iree_uk_pack_p, _pack(b, b4, K, N, N1, K1, n0, k0,
                                       in_pack | abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER))
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = a_rm.data_ptr(), b4.data_ptr(), c.data_ptr()
    p.lhs_stride0, p.rhs_stride0, p.out_stride0 = a_pitch, K1 * n0 * k0, c_pitch
    p.M, p.N, p.K, p.M0, p.N0, p.K0 = M, N1, K1, 1, n0, k0
    p.flags = mm_type | (abi.MMT4D_ACCUMULATE if accumulate else 0)
    call(gpu_lib.iree_uk_mmt4d_p, p)
    assert all(k and "generic" not in k for k in kernels), kernels
    assert kernels[1].startswith("mmt4d_mfma") or kernels[1].startswith("mmt4d_gemv") or \
        kernels[1].startswith("mmt4d_skinny"), kernels

    want = a.double() @ b.double()
    if accumulate:
        want = want + init.double()
    if kind == "i8":
        want = ((want.long() + 2 ** 31) % 2 ** 32 - 2 ** 31)
        assert torch.equal(c[:M, :N].long(), want), kernels
    else:
        assert torch.equal(c[:M, :N].double(), want), kernels
    assert bool((c[:M, N:N1 * n0] == 0).all()), "columns of the padded rhs rows are zero"
    assert bool((c[M, :] == 55).all()) and bool((c[:, N1 * n0:] == 55).all())
