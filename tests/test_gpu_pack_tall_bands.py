"""GPU parity for pack / unpack of 4-byte elements with an outer transpose where the runs of neighbouring tile
columns on the tiled side lie a multiple of 127 or 129 times 4 KiB apart (row counts such as 8128 and 8256 with
16-wide f32 tiles: 512 KiB -+ 4 KiB). The LDS-staged kernel then walks bands of 64 rows of blocks instead of 16
(pack.c:254-313 and unpack.c:190-247 are the semantics; the block order is this library's). Against the oracle,
over the whole destination, with ragged last tiles and columns that do not fill a block.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, synth
from test_gpu_configs import gpu_lib  # noqa: F401

pytestmark = pytest.mark.gpu

TI, TO = abi.PACK_TRANSPOSE_INNER, abi.PACK_TRANSPOSE_OUTER

CASES = [
    # rows, cols, tile rows, tile cols, flags
    (8256, 600, 1, 16, TI | TO),     # tile columns 8256 * 64 B = 512 KiB + 4 KiB apart (tiles stored as [16][1])
    (8128, 333, 1, 16, TI | TO),     # 512 KiB - 4 KiB, ragged last tile column
    (8250, 300, 1, 16, TO),          # within 2.5 KiB of that distance, tiles stored as [1][16]
    (16512, 270, 1, 16, TI | TO),    # 1 MiB + 8 KiB
    (4125, 520, 8, 8, TO),           # 8x8 tiles: 516 row tiles * 256 B apart is no such distance; stays on bands of 16
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%dx%d_t%dx%d_f%x" % c)
def test_pack_and_unpack_with_tall_bands(gpu_lib, oracle_lib, case):
    rows, cols, t0, t1, flags = case
    e = 4
    o0, o1 = -(-rows // t0), -(-cols // t1)
    s0, s1 = (o1, o0) if flags & TO else (o0, o1)
    s2, s3 = (t1, t0) if flags & TI else (t0, t1)
    packed_stride0 = s1 * s2 * s3
    src = synth.uniform_int8(71, 0, rows * cols * e)
    n_packed = s0 * packed_stride0

    def pack_params(src_ptr, dst_ptr):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_stride0, p.in_stride1 = cols, 1
        p.out_stride0, p.out_stride1 = packed_stride0, s2 * s3
        p.in_size0, p.in_size1 = rows, cols
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = s0, s1, s2, s3
        p.padding_value = 0x5AA55AA5
        p.flags = abi.PACK_TYPE_F32F32 | flags
        return p

    def unpack_params(src_ptr, dst_ptr):
        p = abi.UnpackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_stride0, p.in_stride1 = packed_stride0, s2 * s3
        p.out_stride0, p.out_stride1 = cols, 1
        p.in_size0, p.in_size1, p.in_size2, p.in_size3 = s0, s1, s2, s3
        p.out_size0, p.out_size1 = rows, cols
        p.flags = abi.UNPACK_TYPE_F32F32 | flags
        return p

    want = np.full(n_packed * e, 0x77, dtype=np.int8)
    oracle_lib.oracle_pack(C.byref(pack_params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_packed = torch.full((n_packed * e,), 0x77, dtype=torch.int8, device="cuda")
    gpu_lib.iree_uk_pack_p(C.byref(pack_params(d_src.data_ptr(), d_packed.data_ptr())))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"pack_tiled"
    got = d_packed.cpu().numpy()
    if not np.array_equal(got, want):
        bad = np.flatnonzero(got != want)
        raise AssertionError("pack: %d bytes differ, first at %d" % (bad.size, bad[0]))

    start = synth.uniform_int8(71, 1, rows * cols * e)
    want_back = start.copy()
    oracle_lib.oracle_unpack(C.byref(unpack_params(want.ctypes.data, want_back.ctypes.data)))
    d_back = torch.from_numpy(start.copy()).cuda()
    gpu_lib.iree_uk_unpack_p(C.byref(unpack_params(d_packed.data_ptr(), d_back.data_ptr())))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"unpack_tiled"
    got_back = d_back.cpu().numpy()
    if not np.array_equal(got_back, want_back):
        bad = np.flatnonzero(got_back != want_back)
        raise AssertionError("unpack: %d bytes differ, first at %d" % (bad.size, bad[0]))
    assert np.array_equal(got_back, src)
