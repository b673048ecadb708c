"""GPU parity for pack with an inner transpose on 1- and 2-byte elements (the
register-transposing kernel in pack_unpack_tiled.hip), against the oracle
restatement of pack.c:254-313 on the same bytes: ragged edges, padding value,
row and tile strides with gaps, buffer offsets, tiles narrower and wider than
a 16-byte vector, with and without the outer transpose. Bit-exact, gap bytes
of the destination included.
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
    # type, rows, cols, tile rows (of the source), tile cols, flags, row stride pad, tile stride pad
    (abi.PACK_TYPE_I8I8, 1021, 3001 + 3, 64, 16, TI | TO, 0, 0),     # rhs of 16x16x64: [n][k][16][64]
    (abi.PACK_TYPE_I8I8, 1021, 3004, 4, 8, TI | TO, 0, 0),           # rhs of 8x8x4: tiles narrower than a vector
    (abi.PACK_TYPE_I8I8, 777, 1000, 32, 16, TI, 24, 0),              # no outer transpose, row stride with a gap
    (abi.PACK_TYPE_I8I8, 513, 2052, 2, 16, TI | TO, 0, 0),           # [16][2] tiles (x86 dot-product rhs): 2 rows x 2 columns per dword
    (abi.PACK_TYPE_I8I8, 1001, 777, 2, 8, TI, 5, 16),                # [8][2] tiles, odd row stride
    (abi.PACK_TYPE_I8I8, 300, 500, 1, 16, TI | TO, 0, 0),            # one-row int8 tiles: the older kernel
    (abi.PACK_TYPE_I8I8, 300, 4100, 64, 64, TI | TO, 0, 64),         # 4 KiB tiles (the reference's limit), outer stride with a gap
    (abi.PACK_TYPE_I8I8, 2050, 260, 16, 2, TI, 0, 0),                # 2-column tiles
    (abi.PACK_TYPE_F16F16, 1000, 2002, 16, 16, TI | TO, 0, 0),
    (abi.PACK_TYPE_BF16BF16, 999, 1602, 8, 16, TI | TO, 6, 32),
    (abi.PACK_TYPE_BF16BF16, 640, 770, 2, 8, TI, 0, 0),
    (abi.PACK_TYPE_F16F16, 515, 1030, 1, 8, TI | TO, 0, 0),          # one-row tiles: the older kernel
    (abi.PACK_TYPE_I8I8, 64, 48, 16, 16, TI | TO, 0, 0),             # smaller than one block
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "e%d_%dx%d_t%dx%d_f%x" % (abi.PACK_ELEM_BYTES[c[0]], c[1], c[2], c[3], c[4], c[5]))
def test_pack_inner_transpose_small_elements(gpu_lib, oracle_lib, case):
    typ, rows, cols, t0, t1, flags, row_gap, tile_gap = case
    e = abi.PACK_ELEM_BYTES[typ]
    o0, o1 = -(-rows // t0) + 1, -(-cols // t1)          # one extra tile row of pure padding
    s0, s1 = (o1, o0) if flags & TO else (o0, o1)
    s2, s3 = (t1, t0) if flags & TI else (t0, t1)
    in_stride0 = cols + row_gap
    out_stride0 = s1 * s2 * s3 + tile_gap
    in_off, out_off = 4, 16 // e                         # element offsets; keep the 4- and 16-byte alignments
    src = synth.uniform_int8(31, 0, (in_off + rows * in_stride0) * e)
    n_out = out_off + s0 * out_stride0
    pad = 0xA55A

    def params(src_ptr, dst_ptr):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_offset, p.out_offset = in_off, out_off
        p.in_stride0, p.in_stride1 = in_stride0, 1
        p.out_stride0, p.out_stride1 = out_stride0, s2 * s3
        p.in_size0, p.in_size1 = rows, cols
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = s0, s1, s2, s3
        p.padding_value = pad
        p.flags = typ | flags
        return p

    want = np.full(n_out * e, 0x77, dtype=np.int8)
    oracle_lib.oracle_pack(C.byref(params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_out = torch.full((n_out * e,), 0x77, dtype=torch.int8, device="cuda")
    gpu_lib.iree_uk_pack_p(C.byref(params(d_src.data_ptr(), d_out.data_ptr())))
    expected_kernel = b"pack_transposing" if t0 * e >= 4 or (e == 1 and t0 == 2) else b"pack_tiled"
    assert gpu_lib.iree_uk_mi355x_last_kernel() == expected_kernel
    got = d_out.cpu().numpy()
    if not np.array_equal(got, want):
        bad = np.flatnonzero(got != want)
        raise AssertionError("%d bytes differ, first at %d: got %d want %d" % (bad.size, bad[0], got[bad[0]], want[bad[0]]))


def test_pack_inner_transpose_rows_only_byte_aligned(gpu_lib, oracle_lib):
    # Row stride 1001 bytes: rows are only byte aligned; the 16-byte loads do not mind.
    rows, cols, t0, t1 = 300, 1001, 16, 16
    flags = abi.PACK_TYPE_I8I8 | TI | TO
    o0, o1 = -(-rows // t0), -(-cols // t1)
    src = synth.uniform_int8(32, 0, rows * cols)

    def params(src_ptr, dst_ptr):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_stride0, p.in_stride1 = cols, 1
        p.out_stride0, p.out_stride1 = o0 * t0 * t1, t0 * t1
        p.in_size0, p.in_size1 = rows, cols
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = o1, o0, t1, t0
        p.flags = flags
        return p

    want = np.zeros(o0 * o1 * t0 * t1, dtype=np.int8)
    oracle_lib.oracle_pack(C.byref(params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_out = torch.full((want.size,), 0x11, dtype=torch.int8, device="cuda")
    gpu_lib.iree_uk_pack_p(C.byref(params(d_src.data_ptr(), d_out.data_ptr())))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"pack_transposing"
    assert np.array_equal(d_out.cpu().numpy(), want)
