"""GPU parity for unpack of 4-byte (and 2-byte) elements into rows that do not start on
128-byte lines (unpack.c:190-247 is the semantics; tools/unpack_test.c draws
such shapes all the time: any odd row length). The LDS-staged kernel then moves
every row's windows to that row's own line boundaries, so a block stores
columns that belong to the tiles after its own and leaves its first columns to
the block before it. The cases walk through what that changes: row strides of
every residue that matters (odd, 2 mod 4, just below and above a line), output
offsets that move the first row off a line, first and last blocks of a row
(short last block, last block one column wide, exactly full), rows beyond the
matrix in the last tile row, tiles wider than a line, inner transposes, and a
gap between rows whose bytes must survive. Bit-exact against the oracle over the
whole destination buffer.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, synth
from test_gpu_configs import gpu_lib  # noqa: F401

pytestmark = pytest.mark.gpu

TI, TO = abi.UNPACK_TRANSPOSE_INNER, abi.UNPACK_TRANSPOSE_OUTER

CASES = [
    # type, rows, cols, tile rows, tile cols, flags, row gap (elements), out offset (elements)
    (abi.UNPACK_TYPE_F32F32, 8191 // 8, 8190, 16, 1, 0, 0, 0),   # the benchmark's row length
    (abi.UNPACK_TYPE_F32F32, 100, 1025, 16, 1, 0, 0, 0),          # odd stride; last block one column wide
    (abi.UNPACK_TYPE_F32F32, 67, 1024, 16, 1, 0, 1, 0),           # full last block, stride 1025
    (abi.UNPACK_TYPE_F32F32, 67, 1024, 16, 1, 0, 0, 3),           # rows a whole number of lines apart, off by 12 bytes
    (abi.UNPACK_TYPE_I32I32, 50, 3 * 256 + 31, 16, 1, 0, 0, 1),   # stride 799: every residue mod 32 comes up
    (abi.UNPACK_TYPE_I32I32, 33, 2 * 256 + 2, 16, 1, 0, 29, 31),  # next block's first columns only
    (abi.UNPACK_TYPE_F32F32, 45, 1300, 8, 8, 0, 0, 0),            # 8x8 tiles, blocks 512 columns wide
    (abi.UNPACK_TYPE_F32F32, 45, 1300, 8, 8, TI, 2, 5),
    (abi.UNPACK_TYPE_F32F32, 130, 1111, 16, 16, 0, 0, 0),
    (abi.UNPACK_TYPE_I32I32, 130, 1111, 16, 16, TI, 0, 7),
    (abi.UNPACK_TYPE_F32F32, 40, 9000, 1, 16, 0, 0, 0),           # tiles one row tall: blocks of 4096 columns
    (abi.UNPACK_TYPE_F32F32, 70, 700, 4, 64, 0, 1, 0),            # tiles two lines wide
    (abi.UNPACK_TYPE_F32F32, 70, 700, 64, 4, TI, 0, 2),           # blocks 64 columns wide, 64 rows tall
    (abi.UNPACK_TYPE_I32I32, 200, 70, 64, 1, 0, 0, 0),            # two blocks per row, the second 6 columns
    (abi.UNPACK_TYPE_F32F32, 19, 513, 2, 2, 0, 0, 0),             # small tiles, blocks of 2048 columns: one block per row
    (abi.UNPACK_TYPE_F32F32, 19, 4099, 2, 2, TI, 0, 0),
    # 2-byte elements: rows a whole number of dwords apart take the same path, others the plain one.
    (abi.UNPACK_TYPE_F16F16, 200, 8190, 16, 1, 0, 0, 0),
    (abi.UNPACK_TYPE_BF16BF16, 77, 2 * 512 + 66, 16, 1, 0, 2, 6),
    (abi.UNPACK_TYPE_F16F16, 77, 1100, 8, 8, 0, 0, 2),
    (abi.UNPACK_TYPE_BF16BF16, 50, 3000, 16, 16, TI, 4, 0),
    (abi.UNPACK_TYPE_F16F16, 40, 5000, 1, 16, 0, 0, 0),
    (abi.UNPACK_TYPE_F16F16, 33, 700, 32, 8, TI, 0, 4),
    (abi.UNPACK_TYPE_F16F16, 60, 2049, 16, 1, 0, 0, 0),          # odd row length: shifts of odd halfwords, plain path
    (abi.UNPACK_TYPE_BF16BF16, 60, 2048, 16, 1, 0, 0, 3),        # odd offset
    # Outer transposes: the tiled side is one run per tile column, the columns after the block's own are further runs.
    (abi.UNPACK_TYPE_F32F32, 300, 2 * 256 + 200, 16, 1, TO, 0, 0),
    (abi.UNPACK_TYPE_F32F32, 300, 1025, 16, 16, TO, 1, 3),
    (abi.UNPACK_TYPE_I32I32, 130, 1300, 8, 8, TO | TI, 0, 5),
    (abi.UNPACK_TYPE_F32F32, 77, 3 * 256 + 31, 1, 16, TO, 2, 0),
    (abi.UNPACK_TYPE_F32F32, 200, 600, 64, 4, TO | TI, 0, 0),
    (abi.UNPACK_TYPE_F16F16, 300, 2 * 512 + 66, 16, 16, TO, 0, 2),
    (abi.UNPACK_TYPE_BF16BF16, 140, 5000, 16, 1, TO | TI, 2, 0),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%dx%d_t%dx%d_f%x_gap%d_off%d" % (
    c[1], c[2], c[3], c[4], c[5], c[6], c[7]))
def test_unpack_into_rows_off_the_cache_lines(gpu_lib, oracle_lib, case):
    typ, rows, cols, t0, t1, flags, row_gap, out_off = case
    e = abi.UNPACK_ELEM_BYTES[typ]
    o0, o1 = -(-rows // t0), -(-cols // t1)
    s0, s1 = (o1, o0) if flags & TO else (o0, o1)
    s2, s3 = (t1, t0) if flags & TI else (t0, t1)
    in_stride0 = s1 * s2 * s3
    out_stride0 = cols + row_gap
    in_off = 16 // e
    src = synth.uniform_int8(61, 0, (in_off + s0 * in_stride0) * e)
    n_out = out_off + rows * out_stride0 + 64

    def params(src_ptr, dst_ptr):
        p = abi.UnpackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_offset, p.out_offset = in_off, out_off
        p.in_stride0, p.in_stride1 = in_stride0, s2 * s3
        p.out_stride0, p.out_stride1 = out_stride0, 1
        p.in_size0, p.in_size1, p.in_size2, p.in_size3 = s0, s1, s2, s3
        p.out_size0, p.out_size1 = rows, cols
        p.flags = typ | flags
        return p

    # The destination starts as a pattern: row gaps, the bytes in front of the first row and behind the last survive.
    start = synth.uniform_int8(61, 1, n_out * e)
    want = start.copy()
    oracle_lib.oracle_unpack(C.byref(params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_out = torch.from_numpy(start.copy()).cuda()
    gpu_lib.iree_uk_unpack_p(C.byref(params(d_src.data_ptr(), d_out.data_ptr())))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"unpack_tiled"
    got = d_out.cpu().numpy()
    if not np.array_equal(got, want):
        bad = np.flatnonzero(got != want)
        where = (bad[0] // e - out_off)
        raise AssertionError("%d bytes differ, first at byte %d (row %d, column %d): got %d want %d" % (
            bad.size, bad[0], where // out_stride0, where % out_stride0, got[bad[0]], want[bad[0]]))
    assert not np.array_equal(want, start)
