"""Host-side checks that need no GPU: the library loads, exports what the
header declares, keeps the reference's struct layouts, rejects what the
reference's assertions reject and returns early where the reference does.
"""
import ctypes as C
import os
import re

import numpy as np
import pytest

from iree_amd import abi, library

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "iree_uk_mi355x.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(iree_uk_[a-z0-9_]+)\s*\(", text)
    return sorted(set(n for n in names if not n.endswith("_t")))


def test_every_declared_symbol_is_exported():
    lib = library.load()
    names = _declared_functions()
    assert "iree_uk_mmt4d" in names and "iree_uk_unpack_p" in names and len(names) >= 14
    for n in names:
        assert hasattr(lib, n), n


def test_struct_layouts_match_reference_abi():
    # Sizes and offsets on LP64 of the reference's structs
    # (mmt4d_internal.h:14-32, pack_internal.h:12-30, unpack_internal.h:12-29).
    assert C.sizeof(abi.Mmt4dParams) == 9 * 8 + 3 * 8 + 4 * 4 + 8
    assert abi.Mmt4dParams.M0.offset == 96 and abi.Mmt4dParams.flags.offset == 108
    assert abi.Mmt4dParams.cpu_data.offset == 112
    assert C.sizeof(abi.PackParams) == 14 * 8 + 8 + 8 + 8
    assert abi.PackParams.padding_value.offset == 112 and abi.PackParams.flags.offset == 120
    assert C.sizeof(abi.UnpackParams) == 14 * 8 + 8 + 8
    assert abi.UnpackParams.flags.offset == 112
    assert C.sizeof(abi.QueryTileSizes2dParams) == 32


def test_flag_values_in_header_match_reference_constants():
    text = open(HEADER).read()
    defs = dict(re.findall(r"#define (IREE_UK_FLAG_[A-Z0-9_]+) (0x[0-9A-Fa-f]+)", text))
    want = {
        "IREE_UK_FLAG_MMT4D_TYPE_S8S8S32": 0x02, "IREE_UK_FLAG_MMT4D_TYPE_F16F16F32": 0x03,
        "IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32": 0x05, "IREE_UK_FLAG_MMT4D_TYPE_S8S4S32": 0x0A,
        "IREE_UK_FLAG_MMT4D_ACCUMULATE": 0x100,
        "IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION": 0x200,
        "IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS": 0x400,
        "IREE_UK_FLAG_PACK_TYPE_F32F32": 0x01, "IREE_UK_FLAG_PACK_TYPE_I8I8": 0x02,
        "IREE_UK_FLAG_PACK_TRANSPOSE_INNER": 0x100, "IREE_UK_FLAG_PACK_TRANSPOSE_OUTER": 0x200,
        "IREE_UK_FLAG_UNPACK_TYPE_I32I32": 0x03, "IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER": 0x200,
    }
    for k, v in want.items():
        assert int(defs[k], 16) == v, k
    # The lit test of the reference's lowering pins flags as decimal constants,
    # e.g. 1281 = f32f32f32 | ACCUMULATE | SKIP_INTERMEDIATE_ROUNDINGS.
    assert abi.MMT4D_TYPE_F32F32F32 | abi.MMT4D_ACCUMULATE | abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS == 1281


class Failures:
    """Installs a failure handler that records instead of aborting."""

    def __init__(self):
        self.seen = []
        self._cb = library.FAIL_HANDLER(lambda f, l, fn, cond: self.seen.append(cond.decode()))

    def __enter__(self):
        library.load().iree_uk_mi355x_set_fail_handler(self._cb)
        return self

    def __exit__(self, *exc):
        library.load().iree_uk_mi355x_set_fail_handler(library.FAIL_HANDLER(0))


def _mmt4d_params(**kw):
    p = abi.Mmt4dParams()
    p.M = p.N = p.K = 1
    p.M0 = p.N0 = 8
    p.K0 = 4
    p.flags = abi.MMT4D_TYPE_S8S8S32
    for k, v in kw.items():
        setattr(p, k, v)
    return p


@pytest.mark.parametrize("kw", [
    dict(flags=abi.MMT4D_TYPE_S8S8S32 | 0x800),      # unknown flag bit
    dict(flags=0x0B), dict(flags=0x00),               # type out of range / none
    dict(M=-1), dict(N=1 << 31), dict(K=-5),
    dict(M0=1 << 15), dict(N0=-1), dict(K0=40000),
    dict(flags=abi.MMT4D_TYPE_S8S4S32, K0=3),         # K0 * 4 bits not whole bytes
    dict(flags=abi.MMT4D_TYPE_S8S4S32, K0=2, rhs_stride0=3),
])
def test_mmt4d_rejects_what_reference_asserts(kw):
    with Failures() as f:
        library.load().iree_uk_mmt4d_p(C.byref(_mmt4d_params(**kw)))
    assert len(f.seen) == 1, kw


def test_mmt4d_operand_rows_may_overlap_output_rows_may_not():
    # The reference puts no condition on strides (mmt4d.c:12-48): a zero or short
    # lhs/rhs stride is a broadcast or an overlap of rows that are only read.
    # Rows of the output are written concurrently here, so those must not
    # overlap; strides that walk backwards are not supported.
    lib = library.load()
    buf = (C.c_int8 * 4096)()
    base = dict(M=2, N=2, K=1, lhs_buffer=C.addressof(buf), rhs_buffer=C.addressof(buf),
                out_buffer=C.addressof(buf), lhs_stride0=32, rhs_stride0=32, out_stride0=128)
    for kw in (dict(lhs_stride0=0), dict(rhs_stride0=0), dict(lhs_stride0=8, rhs_stride0=4)):
        with Failures() as f:
            lib.iree_uk_mmt4d_p(C.byref(_mmt4d_params(**dict(base, **kw))))
        # Without a GPU the call fails later, in the HIP runtime; with one it runs.
        assert not any("stride" in m or "pitch" in m for m in f.seen), f.seen
    for kw in (dict(out_stride0=64), dict(out_stride0=0), dict(lhs_stride0=-32), dict(rhs_stride0=-32)):
        with Failures() as f:
            lib.iree_uk_mmt4d_p(C.byref(_mmt4d_params(**dict(base, **kw))))
        assert len(f.seen) == 1 and ("stride" in f.seen[0] or "pitch" in f.seen[0]), (kw, f.seen)


def test_mmt4d_early_exits_touch_nothing():
    # M == 0, N == 0 and (K == 0 with ACCUMULATE) return before any pointer is
    # looked at (mmt4d.c:105-113): null buffers must be fine, even without a GPU.
    lib = library.load()
    with Failures() as f:
        lib.iree_uk_mmt4d_p(C.byref(_mmt4d_params(M=0)))
        lib.iree_uk_mmt4d_p(C.byref(_mmt4d_params(N=0)))
        lib.iree_uk_mmt4d_p(C.byref(_mmt4d_params(K=0, flags=abi.MMT4D_TYPE_S8S8S32 | abi.MMT4D_ACCUMULATE)))
    assert f.seen == []
    assert lib.iree_uk_mi355x_last_kernel() == b""


def _pack_params(**kw):
    p = abi.PackParams()
    p.flags = abi.PACK_TYPE_F32F32
    p.in_size0 = p.in_size1 = 4
    p.in_stride0, p.in_stride1 = 4, 1
    p.out_size0 = p.out_size1 = 2
    p.out_size2 = p.out_size3 = 2
    p.out_stride1, p.out_stride0 = 4, 8
    for k, v in kw.items():
        setattr(p, k, v)
    return p


@pytest.mark.parametrize("kw", [
    dict(flags=abi.PACK_TYPE_F32F32 | 0x400), dict(flags=0x06), dict(flags=0),
    dict(in_size0=-1), dict(out_size3=-2), dict(in_stride1=-1),
    dict(out_stride1=5),                   # must equal out_size2 * out_size3
    dict(in_size0=5),                      # more rows than the tiles hold
    dict(in_size1=9),
])
def test_pack_rejects_what_reference_asserts(kw):
    with Failures() as f:
        library.load().iree_uk_pack_p(C.byref(_pack_params(**kw)))
    assert len(f.seen) == 1, kw


def test_pack_unpack_early_exits():
    lib = library.load()
    with Failures() as f:
        lib.iree_uk_pack_p(C.byref(_pack_params(out_size0=0, in_size0=0)))
        lib.iree_uk_pack_p(C.byref(_pack_params(out_size2=0, out_stride1=0, in_size0=0)))
        u = abi.UnpackParams()
        u.flags = abi.UNPACK_TYPE_F32F32
        u.in_size0 = u.in_size1 = u.in_size2 = u.in_size3 = 2
        u.in_stride1, u.in_stride0 = 4, 8
        u.out_size0, u.out_size1 = 0, 4
        lib.iree_uk_unpack_p(C.byref(u))
    assert f.seen == []


@pytest.mark.parametrize("kw", [
    dict(flags=0x02),                       # unpack has no i8 type
    dict(in_stride1=3), dict(out_size0=5), dict(out_stride1=-1),
])
def test_unpack_rejects_what_reference_asserts(kw):
    u = abi.UnpackParams()
    u.flags = abi.UNPACK_TYPE_F32F32
    u.in_size0 = u.in_size1 = u.in_size2 = u.in_size3 = 2
    u.in_stride1, u.in_stride0 = 4, 8
    u.out_size0 = u.out_size1 = 4
    u.out_stride0, u.out_stride1 = 4, 1
    for k, v in kw.items():
        setattr(u, k, v)
    with Failures() as f:
        library.load().iree_uk_unpack_p(C.byref(u))
    assert len(f.seen) == 1, kw


def test_mmt4d_info_reports_specialised_kernels():
    lib = library.load()
    for (t, m0, n0, k0) in [(abi.MMT4D_TYPE_S8S8S32, 8, 8, 4), (abi.MMT4D_TYPE_F16F16F32, 16, 16, 16),
                            (abi.MMT4D_TYPE_S8S4S32, 16, 16, 32), (abi.MMT4D_TYPE_BF16BF16F32, 1, 16, 8),
                            (abi.MMT4D_TYPE_BF16BF16F32, 4, 16, 8), (abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 8)]:
        assert lib.iree_uk_mmt4d_info(m0, n0, k0, t, None) == 1, (t, m0, n0, k0)
    # The tile shapes the reference's x86-64 and Arm targets compile in (mmt4d_x86_64_tiles.inl,
    # mmt4d_arm_64_tiles.inl), wide and narrow; 16-bit outputs with the roundings between k steps skipped.
    skip = abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
    for (t, m0, n0, k0) in [(abi.MMT4D_TYPE_S8S8S32, 16, 16, 2), (abi.MMT4D_TYPE_S8S8S32, 1, 16, 2),
                            (abi.MMT4D_TYPE_S8S8S32, 4, 8, 2), (abi.MMT4D_TYPE_F16F16F32, 16, 16, 1),
                            (abi.MMT4D_TYPE_F16F16F32, 1, 8, 1), (abi.MMT4D_TYPE_F16F16F16 | skip, 16, 16, 1),
                            (abi.MMT4D_TYPE_BF16BF16F32, 2, 16, 2), (abi.MMT4D_TYPE_BF16BF16BF16 | skip, 8, 8, 4),
                            (abi.MMT4D_TYPE_F32F32F32, 1, 16, 1), (abi.MMT4D_TYPE_F32F32F32, 16, 16, 1),
                            (abi.MMT4D_TYPE_S8S8S32, 8, 8, 8), (abi.MMT4D_TYPE_S8S8S32, 2, 8, 4),
                            (abi.MMT4D_TYPE_S16S16S32, 1, 16, 2), (abi.MMT4D_TYPE_S16S16S32, 16, 16, 2), (abi.MMT4D_TYPE_S16U4S32, 1, 32, 8),
                            (abi.MMT4D_TYPE_S8S4S32, 4, 8, 8), (abi.MMT4D_TYPE_S8S4S32, 1, 8, 16),
                            (abi.MMT4D_TYPE_S8S4S32, 4, 16, 2), (abi.MMT4D_TYPE_S16S8S32, 16, 16, 2),
                            (abi.MMT4D_TYPE_S16S8S32, 1, 8, 8), (abi.MMT4D_TYPE_S8S8S32, 4, 8, 1)]:
        assert lib.iree_uk_mmt4d_info(m0, n0, k0, t, None) == 1, (hex(t), m0, n0, k0)
    assert lib.iree_uk_mmt4d_info(9, 6, 3, abi.MMT4D_TYPE_S8S8S32, None) == 0
    assert lib.iree_uk_mmt4d_info(8, 8, 4, 0x0B, None) == 0
    # What only the generic kernel takes: tile sizes that are not powers of two (the reference tests s16s8s32 on
    # 7x5x6), one-byte row pieces in shapes no CPU target uses, f16f16f16 with a rounding after every k step.
    assert lib.iree_uk_mmt4d_info(4, 4, 1, abi.MMT4D_TYPE_S8S8S32, None) == 0
    assert lib.iree_uk_mmt4d_info(8, 8, 1, abi.MMT4D_TYPE_S8S8S32, None) == 1   # k-major int8: transposing LDS reads
    assert lib.iree_uk_mmt4d_info(7, 5, 6, abi.MMT4D_TYPE_S16S8S32, None) == 0
    assert lib.iree_uk_mmt4d_info(16, 16, 1, abi.MMT4D_TYPE_F16F16F16, None) == 0


def test_query_tile_sizes_roles_are_consistent():
    def query(flags):
        p, o = abi.QueryTileSizes2dParams(flags=flags), abi.QueryTileSizes2dOutParams()
        library.load().iree_uk_query_tile_sizes_2d(C.byref(p), C.byref(o))
        return o.tile_size0, o.tile_size1
    for op in (abi.QTS_OP_MATMUL_I8I8I32, abi.QTS_OP_MATMUL_F16F16F32, abi.QTS_OP_MATMUL_BF16BF16F32,
               abi.QTS_OP_MATMUL_F32F32F32):
        m0, k0 = query(op | abi.QTS_ROLE_LHS)
        n0, k0r = query(op | abi.QTS_ROLE_RHS)
        assert k0 == k0r
        assert query(op | abi.QTS_ROLE_RESULT) == (m0, n0)


def test_every_tile_shape_of_the_reference_cpu_targets_has_a_specialised_kernel():
    # tests/golden/reference_arch_tiles.json lists the reference's tables of architecture-specific tile functions
    # (mmt4d_x86_64_tiles.inl, mmt4d_arm_64_tiles.inl; written by tests/golden/make_tile_list.py): the tile shapes a
    # caller compiled for those CPUs passes. None of them may end up on the one-thread-per-element kernel.
    import json
    import os
    lib = library.load()
    skip = abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS   # what the compiler sets for 16-bit outputs
    flag = {"f32f32f32": abi.MMT4D_TYPE_F32F32F32, "f16f16f32": abi.MMT4D_TYPE_F16F16F32,
            "f16f16f16": abi.MMT4D_TYPE_F16F16F16 | skip, "bf16bf16f32": abi.MMT4D_TYPE_BF16BF16F32,
            "bf16bf16bf16": abi.MMT4D_TYPE_BF16BF16BF16 | skip, "s8s8s32": abi.MMT4D_TYPE_S8S8S32,
            "s16s16s32": abi.MMT4D_TYPE_S16S16S32, "s16u4s32": abi.MMT4D_TYPE_S16U4S32, "s8s4s32": abi.MMT4D_TYPE_S8S4S32}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_arch_tiles.json")
    tiles = json.load(open(path))["tiles"]
    assert len(tiles) >= 90 and {t["arch"] for t in tiles} == {"x86_64", "arm_64"}
    missing = [(t["arch"], t["type"], t["M0"], t["N0"], t["K0"]) for t in tiles
               if lib.iree_uk_mmt4d_info(t["M0"], t["N0"], t["K0"], flag[t["type"]], None) != 1]
    assert not missing, missing
