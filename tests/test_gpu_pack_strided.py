"""GPU parity for pack and unpack with an element stride on the 2-D side
(in_stride1 / out_stride1 other than 1), which the reference's tests draw
(tools/pack_test.c:80-93, in_stride1 in {1, 2}) and its implementation handles
in the tile path through a temporary row (pack.c:227, unpack.c:190-247).
Against the oracle restatement on the same bytes: ragged edges, padding, row
gaps, all transpose combinations, 1-, 2- and 4-byte elements; bit-exact over
the whole destination, for unpack including the bytes BETWEEN the strided
elements, which must not be written. These calls must stay on the LDS-staged
kernels rather than fall to the one-thread-per-element ones.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, synth
from test_gpu_configs import gpu_lib  # noqa: F401

pytestmark = pytest.mark.gpu

TI, TO = abi.PACK_TRANSPOSE_INNER, abi.PACK_TRANSPOSE_OUTER

PACK_CASES = [
    # type, rows, cols, tile rows (of the source), tile cols, flags, element stride, row gap
    (abi.PACK_TYPE_F32F32, 517, 1030, 16, 1, 0, 2, 0),
    (abi.PACK_TYPE_F32F32, 300, 777, 8, 8, TI, 2, 3),
    (abi.PACK_TYPE_F32F32, 1025, 260, 1, 16, TO, 3, 1),
    (abi.PACK_TYPE_I32I32, 333, 500, 16, 4, TI | TO, 2, 0),
    (abi.PACK_TYPE_I8I8, 1021, 3004, 16, 64, 0, 2, 0),
    (abi.PACK_TYPE_I8I8, 700, 2050, 64, 16, TI | TO, 2, 7),
    (abi.PACK_TYPE_I8I8, 515, 300, 4, 8, TI, 5, 0),
    (abi.PACK_TYPE_F16F16, 1000, 1002, 16, 16, TI | TO, 2, 0),
    (abi.PACK_TYPE_BF16BF16, 64, 48, 8, 8, 0, 2, 2),
]


@pytest.mark.parametrize("case", PACK_CASES, ids=lambda c: "e%d_%dx%d_t%dx%d_f%x_s%d" % (
    abi.PACK_ELEM_BYTES[c[0]], c[1], c[2], c[3], c[4], c[5], c[6]))
def test_pack_with_an_element_stride(gpu_lib, oracle_lib, case):
    typ, rows, cols, t0, t1, flags, stride1, row_gap = case
    e = abi.PACK_ELEM_BYTES[typ]
    o0, o1 = -(-rows // t0) + 1, -(-cols // t1)          # one extra tile row of pure padding
    s0, s1 = (o1, o0) if flags & TO else (o0, o1)
    s2, s3 = (t1, t0) if flags & TI else (t0, t1)
    in_stride0 = cols * stride1 + row_gap
    out_stride0 = s1 * s2 * s3
    in_off, out_off = 4, 16 // e
    src = synth.uniform_int8(51, 0, (in_off + rows * in_stride0) * e)
    n_out = out_off + s0 * out_stride0

    def params(src_ptr, dst_ptr):
        p = abi.PackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_offset, p.out_offset = in_off, out_off
        p.in_stride0, p.in_stride1 = in_stride0, stride1
        p.out_stride0, p.out_stride1 = out_stride0, s2 * s3
        p.in_size0, p.in_size1 = rows, cols
        p.out_size0, p.out_size1, p.out_size2, p.out_size3 = s0, s1, s2, s3
        p.padding_value = 0x5AA55AA5
        p.flags = typ | flags
        return p

    want = np.full(n_out * e, 0x77, dtype=np.int8)
    oracle_lib.oracle_pack(C.byref(params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_out = torch.full((n_out * e,), 0x77, dtype=torch.int8, device="cuda")
    gpu_lib.iree_uk_pack_p(C.byref(params(d_src.data_ptr(), d_out.data_ptr())))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"pack_tiled"
    got = d_out.cpu().numpy()
    if not np.array_equal(got, want):
        bad = np.flatnonzero(got != want)
        raise AssertionError("%d bytes differ, first at %d: got %d want %d" % (bad.size, bad[0], got[bad[0]], want[bad[0]]))


UNPACK_CASES = [
    # type, rows, cols, tile rows (of the destination), tile cols, flags, element stride, row gap
    (abi.UNPACK_TYPE_F32F32, 517, 1030, 16, 1, 0, 2, 0),
    (abi.UNPACK_TYPE_F32F32, 300, 777, 8, 8, TI, 2, 3),
    (abi.UNPACK_TYPE_I32I32, 1025, 260, 16, 16, TO, 3, 1),
    (abi.UNPACK_TYPE_I32I32, 333, 500, 16, 4, TI | TO, 2, 0),
    (abi.UNPACK_TYPE_F16F16, 1000, 1002, 16, 16, TI | TO, 2, 0),
    (abi.UNPACK_TYPE_BF16BF16, 64, 48, 8, 8, 0, 2, 2),
]


@pytest.mark.parametrize("case", UNPACK_CASES, ids=lambda c: "e%d_%dx%d_t%dx%d_f%x_s%d" % (
    abi.UNPACK_ELEM_BYTES[c[0]], c[1], c[2], c[3], c[4], c[5], c[6]))
def test_unpack_with_an_element_stride(gpu_lib, oracle_lib, case):
    typ, rows, cols, t0, t1, flags, stride1, row_gap = case
    e = abi.UNPACK_ELEM_BYTES[typ]
    o0, o1 = -(-rows // t0), -(-cols // t1)
    s0, s1 = (o1, o0) if flags & TO else (o0, o1)
    s2, s3 = (t1, t0) if flags & TI else (t0, t1)
    in_stride0 = s1 * s2 * s3
    out_stride0 = cols * stride1 + row_gap
    in_off, out_off = 16 // e, 4
    src = synth.uniform_int8(52, 0, (in_off + s0 * in_stride0) * e)
    n_out = out_off + rows * out_stride0

    def params(src_ptr, dst_ptr):
        p = abi.UnpackParams()
        p.in_buffer, p.out_buffer = src_ptr, dst_ptr
        p.in_offset, p.out_offset = in_off, out_off
        p.in_stride0, p.in_stride1 = in_stride0, s2 * s3
        p.out_stride0, p.out_stride1 = out_stride0, stride1
        p.in_size0, p.in_size1, p.in_size2, p.in_size3 = s0, s1, s2, s3
        p.out_size0, p.out_size1 = rows, cols
        p.flags = typ | flags
        return p

    # The destination starts as a pattern: what lies between the elements and in the row gaps must survive.
    start = synth.uniform_int8(52, 1, n_out * e)
    want = start.copy()
    oracle_lib.oracle_unpack(C.byref(params(src.ctypes.data, want.ctypes.data)))
    d_src = torch.from_numpy(src).cuda()
    d_out = torch.from_numpy(start.copy()).cuda()
    gpu_lib.iree_uk_unpack_p(C.byref(params(d_src.data_ptr(), d_out.data_ptr())))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"unpack_tiled"
    got = d_out.cpu().numpy()
    if not np.array_equal(got, want):
        bad = np.flatnonzero(got != want)
        raise AssertionError("%d bytes differ, first at %d: got %d want %d" % (bad.size, bad[0], got[bad[0]], want[bad[0]]))
    assert not np.array_equal(want, start)
