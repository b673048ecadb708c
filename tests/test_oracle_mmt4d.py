"""Pins oracle_mmt4d (oracle/uk_oracle.c).

Three independent anchors:
  1. the compiled reference over the reference's own test grid
     (tools/mmt4d_test.c:459-603), whole out buffer compared byte for byte as
     at tools/mmt4d_test.c:430-440, stride gaps included;
  2. integer matmul in numpy on the unpacked operands (closed form);
  3. hand-computed known answers for the int4 nibble order and sign extension
     (mmt4d_tile_generic.c:35-45) and the f16 subnormal flush
     (common.h:685-686).
"""
import ctypes as C

import numpy as np
import pytest

import ukcases
from iree_amd import abi


def _ids(tiles):
    return ["%s_%dx%dx%d%s" % (abi.MMT4D_NAMES[t[0] & 0xFF], t[1], t[2], t[3],
                               "_skipround" if t[0] & abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS else "")
            for t in tiles]


ALL_TILES = ukcases.MMT4D_TILES_GENERIC + ukcases.MMT4D_TILES_X86 + ukcases.MMT4D_TILES_GPU


@pytest.mark.parametrize("tile", ALL_TILES, ids=_ids(ALL_TILES))
def test_oracle_matches_compiled_reference(tile, oracle_lib, ref_lib):
    import oracle
    cpu = oracle.host_cpu_data()
    for case in ukcases.mmt4d_cases(tile):
        def run_ref(pp):
            pp._obj.cpu_data = C.cast(cpu, C.POINTER(C.c_uint64))
            ref_lib.ref_mmt4d(pp)
        want = case.run_host(run_ref)
        got = case.run_host(oracle_lib.oracle_mmt4d)
        assert np.array_equal(got, want), case.label()
    assert ref_lib.ref_fail_count() == 0


def _unpack_int(case, which):
    """Row-major int64 matrix [rows*T, K*K0] of an integer operand."""
    kind = case.kinds[which]
    raw = case.lhs if which == 0 else case.rhs
    rows, t = (case.M, case.M0) if which == 0 else (case.N, case.N0)
    stride = case.lhs_stride0 if which == 0 else case.rhs_stride0
    n = case.K * t * case.K0
    if kind in ("s4", "u4"):
        lo = (raw & 0xF).astype(np.int64)
        hi = (raw >> 4).astype(np.int64)
        el = np.stack([lo, hi], axis=1).reshape(-1)
        if kind == "s4":
            el = (el ^ 8) - 8
    else:
        el = raw.view({"s8": np.int8, "s16": np.int16}[kind]).astype(np.int64)
    el = el[:rows * stride].reshape(rows, stride)[:, :n].reshape(rows, case.K, t, case.K0)
    return el.transpose(0, 2, 1, 3).reshape(rows * t, case.K * case.K0)


INT_TILES = [t for t in ALL_TILES if abi.MMT4D_NAMES[t[0] & 0xFF].startswith("s")]


@pytest.mark.parametrize("tile", INT_TILES, ids=_ids(INT_TILES))
def test_oracle_integer_closed_form(tile, oracle_lib):
    for case in ukcases.mmt4d_cases(tile):
        got = case.run_host(oracle_lib.oracle_mmt4d).view(np.int32)
        init = case.out_init.view(np.int32)
        want = init.copy()
        if case.M and case.N and not (case.K == 0 and case.flags & abi.MMT4D_ACCUMULATE):
            a = _unpack_int(case, 0)
            b = _unpack_int(case, 1)
            c = (a @ b.T).reshape(case.M, case.M0, case.N, case.N0).transpose(0, 2, 1, 3)
            c = c.reshape(case.M, case.N * case.M0 * case.N0)
            view = want.reshape(case.M, case.out_stride0)[:, :case.N * case.M0 * case.N0]
            if case.flags & abi.MMT4D_ACCUMULATE:
                c = c + view
            view[...] = (c & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
        assert np.array_equal(got, want), case.label()


def _one_tile(oracle_lib, flags, lhs, rhs, out, M0, N0, K0, K=1):
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data
    p.lhs_stride0 = p.rhs_stride0 = p.out_stride0 = 0
    p.M = p.N = 1
    p.K = K
    p.M0, p.N0, p.K0 = M0, N0, K0
    p.flags = flags
    oracle_lib.oracle_mmt4d(C.byref(p))


def test_int4_nibble_order_known_answer(oracle_lib):
    # One row, one column, K0=2: byte 0x8F holds element 0 = 0xF = -1 (low
    # nibble) and element 1 = 0x8 = -8 (high nibble). lhs = (3, 5):
    # 3*(-1) + 5*(-8) = -43.
    lhs = np.array([3, 5], dtype=np.int8)
    rhs = np.array([0x8F], dtype=np.uint8)
    out = np.zeros(1, dtype=np.int32)
    _one_tile(oracle_lib, abi.MMT4D_TYPE_S8S4S32, lhs, rhs, out, 1, 1, 2)
    assert out[0] == -43
    # Two columns: second column byte 0x17 -> (7, 1): 3*7 + 5*1 = 26.
    rhs = np.array([0x8F, 0x17], dtype=np.uint8)
    out = np.zeros(2, dtype=np.int32)
    _one_tile(oracle_lib, abi.MMT4D_TYPE_S8S4S32, lhs, rhs, out, 1, 2, 2)
    assert out.tolist() == [-43, 26]
    # Unsigned nibbles for s16u4s32: (15, 8): 3*15 + 5*8 = 85.
    lhs16 = np.array([3, 5], dtype=np.int16)
    out = np.zeros(1, dtype=np.int32)
    _one_tile(oracle_lib, abi.MMT4D_TYPE_S16U4S32, lhs16, np.array([0x8F], np.uint8), out, 1, 1, 2)
    assert out[0] == 85


def test_f16_subnormal_flush_known_answer(oracle_lib):
    assert oracle_lib.oracle_f16_to_f32(0x0001) == 0.0
    assert oracle_lib.oracle_f16_to_f32(0x03FF) == 0.0
    assert oracle_lib.oracle_f16_to_f32(0x0400) == 2.0 ** -14
    assert oracle_lib.oracle_f16_to_f32(0x3C00) == 1.0
    assert oracle_lib.oracle_f16_to_f32(0xC000) == -2.0
    assert oracle_lib.oracle_bf16_to_f32(0x3F80) == 1.0
    assert oracle_lib.oracle_bf16_to_f32(0x0001) == 0.0
    # A subnormal times a large value contributes nothing: 0x0001 * 65504.
    lhs = np.array([0x0001, 0x3C00], dtype=np.uint16)  # (subnormal, 1.0)
    rhs = np.array([0x7BFF, 0x4000], dtype=np.uint16)  # (65504, 2.0)
    out = np.zeros(1, dtype=np.float32)
    _one_tile(oracle_lib, abi.MMT4D_TYPE_F16F16F32, lhs, rhs, out, 1, 1, 2)
    assert out[0] == 2.0


def test_f16_conversions_agree_with_numpy_on_normals(oracle_lib):
    # numpy's float16 is IEEE binary16; on normal values both directions agree.
    bits = np.arange(0x0400, 0x7C00, 7, dtype=np.uint16)
    for b in bits[::13]:
        f = oracle_lib.oracle_f16_to_f32(int(b))
        assert f == float(np.uint16(b).view(np.float16))
        assert oracle_lib.oracle_f32_to_f16(f) == int(b)
    # Round to nearest even: 1 + 2^-11 is a tie -> 1.0; 1 + 3*2^-11 -> 1 + 2^-9... check vs numpy.
    with np.errstate(over="ignore"):
        for x in (1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65519.0, 65520.0, 1e-3, -0.3):
            assert oracle_lib.oracle_f32_to_f16(x) == int(np.float32(x).astype(np.float16).view(np.uint16))
    assert oracle_lib.oracle_f32_to_bf16(1.0) == 0x3F80
    assert oracle_lib.oracle_f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80  # tie to even
    assert oracle_lib.oracle_f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82


def test_accumulate_and_degenerate_shapes(oracle_lib):
    # K == 0 without ACCUMULATE zeroes the M*N tiles; with it nothing changes;
    # M == 0 or N == 0 never touches memory (mmt4d.c:105-113).
    rng = ukcases.Lcg()
    for (M, N, K, acc) in [(5, 7, 0, 0), (5, 7, 0, 1), (0, 5, 7, 0), (5, 0, 7, 0)]:
        case = ukcases.Mmt4dCase(abi.MMT4D_TYPE_S8S8S32 | (abi.MMT4D_ACCUMULATE if acc else 0),
                                 M, N, K, 8, 8, 4, rng)
        got = case.run_host(oracle_lib.oracle_mmt4d).view(np.int32)
        want = case.out_init.view(np.int32).copy()
        if M and N and not acc:
            want.reshape(M, case.out_stride0)[:, :N * 64] = 0
        assert np.array_equal(got, want)
