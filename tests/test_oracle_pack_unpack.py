"""Pins oracle_pack / oracle_unpack (oracle/uk_oracle.c).

Anchors:
  1. the compiled reference over the reference's own grids
     (tools/pack_test.c:132-241, tools/unpack_test.c:118-216), comparing the
     region the reference's tests compare and checking that nothing else in the
     output buffer changed;
  2. the literal tensors of tests/e2e/tensor_ops/pack.mlir:21-28,51-69 and
     unpack.mlir:24-31,50-61, kept as data in tests/golden/tensor_ops.json;
  3. pack without padding == reshape + transpose (pack.mlir:96-136,
     pack_i8.mlir:26-68), with numpy as the library routine;
  4. unpack(pack(x)) == x.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

import ukcases
from iree_amd import abi

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tensor_ops.json")


def _pack_ids(tiles):
    return ["%s_%dx%d" % (ukcases.PACK_NAMES[t[0]], t[1], t[2]) for t in tiles]


PACK_TILES = ukcases.PACK_TILES_GENERIC + ukcases.PACK_TILES_X86 + ukcases.PACK_TILES_GPU
UNPACK_TILES = ukcases.UNPACK_TILES_GENERIC + ukcases.UNPACK_TILES_X86 + ukcases.UNPACK_TILES_GPU


@pytest.mark.parametrize("tile", PACK_TILES, ids=_pack_ids(PACK_TILES))
def test_pack_oracle_matches_compiled_reference(tile, oracle_lib, ref_lib):
    import oracle
    cpu = oracle.host_cpu_data()
    for case in ukcases.pack_cases(tile):
        def run_ref(pp):
            pp._obj.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
            ref_lib.ref_pack(pp)
        want = case.run_host(run_ref)
        got = case.run_host(oracle_lib.oracle_pack)
        mask = case.written_mask()
        assert np.array_equal(got[mask], want[mask]), case.label()
        # Stride-gap bytes keep their initial contents in both.
        assert np.array_equal(got[~mask], case.out_init[~mask]), case.label()
        assert np.array_equal(want[~mask], case.out_init[~mask]), case.label()
    assert ref_lib.ref_fail_count() == 0


@pytest.mark.parametrize("tile", UNPACK_TILES, ids=_pack_ids(UNPACK_TILES))
def test_unpack_oracle_matches_compiled_reference(tile, oracle_lib, ref_lib):
    import oracle
    cpu = oracle.host_cpu_data()
    for case in ukcases.unpack_cases(tile):
        def run_ref(pp):
            pp._obj.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
            ref_lib.ref_unpack(pp)
        want = case.run_host(run_ref)
        got = case.run_host(oracle_lib.oracle_unpack)
        # Whole buffer: the logical region equals the reference's and every
        # other byte (stride gaps) is untouched in both.
        assert np.array_equal(got, want), case.label()
    assert ref_lib.ref_fail_count() == 0


def _pack_np(oracle_lib, src, out_shape, tile_flags, pad=0, type_flag=abi.PACK_TYPE_I32I32):
    src = np.ascontiguousarray(src)
    out = np.full(out_shape, -77, dtype=src.dtype)
    p = abi.PackParams()
    p.in_buffer, p.out_buffer = src.ctypes.data, out.ctypes.data
    p.in_stride0, p.in_stride1 = src.shape[1], 1
    p.out_stride0, p.out_stride1 = out_shape[1] * out_shape[2] * out_shape[3], out_shape[2] * out_shape[3]
    p.in_size0, p.in_size1 = src.shape
    p.out_size0, p.out_size1, p.out_size2, p.out_size3 = out_shape
    p.padding_value = pad
    p.flags = type_flag | tile_flags
    oracle_lib.oracle_pack(C.byref(p))
    return out


def _unpack_np(oracle_lib, src, out_shape, tile_flags):
    src = np.ascontiguousarray(src)
    out = np.full(out_shape, -77, dtype=src.dtype)
    p = abi.UnpackParams()
    p.in_buffer, p.out_buffer = src.ctypes.data, out.ctypes.data
    s = src.shape
    p.in_stride0, p.in_stride1 = s[1] * s[2] * s[3], s[2] * s[3]
    p.out_stride0, p.out_stride1 = out_shape[1], 1
    p.in_size0, p.in_size1, p.in_size2, p.in_size3 = s
    p.out_size0, p.out_size1 = out_shape
    p.flags = abi.UNPACK_TYPE_I32I32 | tile_flags
    oracle_lib.oracle_unpack(C.byref(p))
    return out


def test_golden_tensors_from_reference_e2e_tests(oracle_lib):
    g = json.load(open(GOLDEN))
    for c in g["pack"]:
        src = np.array(c["input"], dtype=np.int32)
        want = np.array(c["expected"], dtype=np.int32)
        got = _pack_np(oracle_lib, src, want.shape, 0, pad=c["pad"])
        assert np.array_equal(got, want), c["name"]
    for c in g["unpack"]:
        src = np.array(c["input"], dtype=np.int32)
        want = np.array(c["expected"], dtype=np.int32)
        got = _unpack_np(oracle_lib, src, want.shape, 0)
        assert np.array_equal(got, want), c["name"]


# (inner tiles as in the out tensor, tensor.pack inner_dims_pos, outer_dims_perm,
#  the transpose permutation the reference test states)
IDENTITIES = [
    ((32, 16), (0, 1), (0, 1), (0, 2, 1, 3)),
    ((16, 32), (1, 0), (0, 1), (0, 2, 3, 1)),
    ((32, 16), (0, 1), (1, 0), (2, 0, 1, 3)),
    ((16, 32), (1, 0), (1, 0), (2, 0, 3, 1)),
]


@pytest.mark.parametrize("tiles,inner_pos,outer_perm,perm", IDENTITIES)
@pytest.mark.parametrize("shape", [(128, 256), (100, 250)])
def test_pack_is_reshape_transpose(oracle_lib, tiles, inner_pos, outer_perm, perm, shape):
    h, w = shape
    src = np.arange(h * w, dtype=np.int32).reshape(h, w)
    t_dim0 = tiles[inner_pos.index(0)]   # tile size applied to dim 0
    t_dim1 = tiles[inner_pos.index(1)]
    o0, o1 = -(-h // t_dim0), -(-w // t_dim1)
    padded = np.zeros((o0 * t_dim0, o1 * t_dim1), dtype=np.int32)
    padded[:h, :w] = src
    want = padded.reshape(o0, t_dim0, o1, t_dim1).transpose(perm)
    flags = (abi.PACK_TRANSPOSE_INNER if inner_pos == (1, 0) else 0) | \
            (abi.PACK_TRANSPOSE_OUTER if outer_perm == (1, 0) else 0)
    got = _pack_np(oracle_lib, src, want.shape, flags, pad=0)
    assert np.array_equal(got, want)
    # and back
    uflags = (abi.UNPACK_TRANSPOSE_INNER if inner_pos == (1, 0) else 0) | \
             (abi.UNPACK_TRANSPOSE_OUTER if outer_perm == (1, 0) else 0)
    back = _unpack_np(oracle_lib, got, (h, w), uflags)
    assert np.array_equal(back, src)


def test_pack_i8_vnni_layouts(oracle_lib):
    # pack_i8.mlir:26-68: LHS 128x256 i8 -> [8,128,16,2]; RHS 256x128 -> [8,128,16,2]
    # with inner_dims_pos=[1,0], outer_dims_perm=[1,0].
    lhs = (np.arange(128 * 256) % 251).astype(np.int8).reshape(128, 256)
    want = lhs.reshape(8, 16, 128, 2).transpose(0, 2, 1, 3)
    got = _pack_np(oracle_lib, lhs, want.shape, 0, type_flag=abi.PACK_TYPE_I8I8)
    assert np.array_equal(got, want)
    rhs = (np.arange(256 * 128) % 251).astype(np.int8).reshape(256, 128)
    want = rhs.reshape(128, 2, 8, 16).transpose(2, 0, 3, 1)
    got = _pack_np(oracle_lib, rhs, want.shape, abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER,
                   type_flag=abi.PACK_TYPE_I8I8)
    assert np.array_equal(got, want)


def test_padding_value_uses_low_element_bits(oracle_lib):
    src = np.array([[1, 2, 3]], dtype=np.int8)
    got = _pack_np(oracle_lib, src, (1, 2, 2, 2), 0, pad=0x1122334455667788,
                   type_flag=abi.PACK_TYPE_I8I8)
    assert got.astype(np.uint8).reshape(-1).tolist() == [1, 2, 0x88, 0x88, 3, 0x88, 0x88, 0x88]
    src16 = np.array([[1, 2, 3]], dtype=np.int16)
    got = _pack_np(oracle_lib, src16, (1, 2, 1, 2), 0, pad=0x1122334455667788,
                   type_flag=abi.PACK_TYPE_F16F16)
    assert got.astype(np.uint16).reshape(-1).tolist() == [1, 2, 3, 0x7788]
