"""The HAL executable plugin (iree_amd/libiree_uk_mi355x_plugin.so): the
interface the reference runtime binds at load time
(runtime/src/iree/hal/local/executable_plugin.h:185-191, 404-460) and the
imports it resolves. Without a GPU: query / resolve behaviour and a layout
check of the restated interface structs against the reference's own header.
With a GPU: the imports called the way a compiled dispatch calls them (operands
packed in a struct, host pointers) against the oracle.
"""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np
import pytest

from iree_amd import abi, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = os.path.join(ROOT, "iree_amd", "libiree_uk_mi355x_plugin.so")
REFERENCE_SRC = "/root/reference/runtime/src"


class Header(C.Structure):
    _fields_ = [("version", C.c_uint32), ("name", C.c_char_p), ("description", C.c_char_p),
                ("features", C.c_uint32), ("sanitizer", C.c_int32), ("reserved", C.c_uint64 * 8)]


LOAD_FN = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.POINTER(C.c_void_p))
UNLOAD_FN = C.CFUNCTYPE(None, C.c_void_p)


class ResolveParams(C.Structure):
    _fields_ = [("count", C.c_size_t), ("symbol_names", C.POINTER(C.c_char_p)),
                ("out_fn_ptrs", C.POINTER(C.c_void_p)), ("out_fn_contexts", C.POINTER(C.c_void_p))]


RESOLVE_FN = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.POINTER(ResolveParams), C.POINTER(C.c_uint32))
IMPORT_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_void_p)


class PluginV0(C.Structure):
    _fields_ = [("header", C.POINTER(Header)), ("load", LOAD_FN), ("unload", UNLOAD_FN), ("resolve", RESOLVE_FN)]


class Environment(C.Structure):
    _fields_ = [("allocator_self", C.c_void_p), ("allocator_ctl", C.c_void_p)]


@pytest.fixture(scope="module")
def plugin():
    assert os.path.exists(PLUGIN), "build first: python -m iree_amd.build"
    lib = C.CDLL(PLUGIN)
    lib.iree_hal_executable_plugin_query.restype = C.POINTER(PluginV0)
    lib.iree_hal_executable_plugin_query.argtypes = [C.c_uint32, C.c_void_p]
    p = lib.iree_hal_executable_plugin_query(1, None)
    assert p
    return lib, p.contents


def _resolve(plugin_v0, names, preset=None):
    n = len(names)
    c_names = (C.c_char_p * n)(*[s.encode() for s in names])
    fns = (C.c_void_p * n)(*(preset or [None] * n))
    ctxs = (C.c_void_p * n)()
    params = ResolveParams(n, c_names, fns, ctxs)
    resolution = C.c_uint32(0xFFFFFFFF)
    status = plugin_v0.resolve(None, C.byref(params), C.byref(resolution))
    return (status or 0), resolution.value, list(fns)


def test_query_returns_a_v0_interface(plugin):
    lib, v0 = plugin
    h = v0.header.contents
    assert h.version == 1
    assert h.name == b"iree_uk_mi355x"
    assert h.features == 0 and h.sanitizer == 0   # needs the HIP runtime: not "standalone"
    assert all(x == 0 for x in h.reserved)
    # A runtime that only knows older interface versions gets nothing.
    assert not lib.iree_hal_executable_plugin_query(0, None)


def test_resolve_known_optional_and_unknown_symbols(plugin):
    _, v0 = plugin
    status, resolution, fns = _resolve(v0, ["iree_uk_mmt4d", "iree_uk_pack", "iree_uk_query_tile_sizes.2d",
                                            "iree_uk_query_tile_sizes_2d", "iree_uk_unpack"])
    assert status == 0 and resolution == 0 and all(fns) and len(set(fns)) == 4 and fns[2] == fns[3]
    # Optional (leading '?') and missing: OK, with the bit set.
    status, resolution, fns = _resolve(v0, ["?iree_uk_mmt4d", "?iree_uk_softmax"])
    assert status == 0 and resolution == 1 and fns[0] and not fns[1]
    # Required and missing: NOT_FOUND (5), what is available is still filled in.
    status, resolution, fns = _resolve(v0, ["iree_uk_mmt4d", "iree_uk_softmax"])
    assert status == 5 and fns[0] and not fns[1]
    # Entries another provider has already resolved are left alone.
    status, _, fns = _resolve(v0, ["iree_uk_mmt4d", "iree_uk_pack"], preset=[0x1234, None])
    assert status == 0 and fns[0] == 0x1234 and fns[1]


def test_load_reports_a_missing_gpu(plugin):
    from iree_amd import library
    _, v0 = plugin
    env = Environment(None, None)
    self_ptr = C.c_void_p(0xDEAD)
    status = v0.load(C.byref(env), 0, None, C.byref(self_ptr)) or 0
    assert self_ptr.value is None
    # OK where the library finds a gfx950 device, UNAVAILABLE (14) elsewhere.
    usable = library.load().iree_uk_mi355x_init(-1) == 0
    assert status == (0 if usable else 14)
    if usable:
        v0.unload(None)


@pytest.mark.skipif(not os.path.exists(os.path.join(REFERENCE_SRC, "iree/hal/local/executable_plugin.h")),
                    reason="reference tree not present")
def test_restated_interface_matches_the_reference_header():
    checks = []
    pairs = {
        ("ukp_header_t", "iree_hal_executable_plugin_header_t"):
            ["version", "name", "description", "features", "sanitizer", "reserved"],
        ("ukp_allocator_t", "iree_hal_executable_plugin_allocator_t"): ["self", "ctl"],
        ("ukp_string_view_t", "iree_hal_executable_plugin_string_view_t"): ["data", "size"],
        ("ukp_string_pair_t", "iree_hal_executable_plugin_string_pair_t"): ["first", "second"],
        ("ukp_environment_v0_t", "iree_hal_executable_plugin_environment_v0_t"): ["host_allocator"],
        ("ukp_resolve_params_v0_t", "iree_hal_executable_plugin_resolve_params_v0_t"):
            ["count", "symbol_names", "out_fn_ptrs", "out_fn_contexts"],
        ("ukp_plugin_v0_t", "iree_hal_executable_plugin_v0_t"): ["header", "load", "unload", "resolve"],
    }
    for (mine, theirs), fields in pairs.items():
        checks.append("_Static_assert(sizeof(%s) == sizeof(%s), \"size of %s\");" % (mine, theirs, mine))
        for f in fields:
            checks.append("_Static_assert(offsetof(%s, %s) == offsetof(%s, %s), \"%s.%s\");" % (mine, f, theirs, f, mine, f))
    checks += [
        "_Static_assert(UKP_VERSION_0_1 == IREE_HAL_EXECUTABLE_PLUGIN_VERSION_LATEST, \"version\");",
        "_Static_assert(UKP_FEATURE_NONE == IREE_HAL_EXECUTABLE_PLUGIN_FEATURE_NONE, \"features\");",
        "_Static_assert(UKP_SANITIZER_NONE == IREE_HAL_EXECUTABLE_PLUGIN_SANITIZER_NONE, \"sanitizer\");",
        "_Static_assert(sizeof(ukp_status_t) == sizeof(iree_hal_executable_plugin_status_t), \"status\");",
        "_Static_assert(5 == IREE_HAL_EXECUTABLE_PLUGIN_STATUS_NOT_FOUND, \"not found\");",
        "_Static_assert(14 == IREE_HAL_EXECUTABLE_PLUGIN_STATUS_UNAVAILABLE, \"unavailable\");",
        "_Static_assert(UKP_RESOLUTION_MISSING_OPTIONAL == IREE_HAL_EXECUTABLE_PLUGIN_RESOLUTION_MISSING_OPTIONAL, \"bit\");",
        "_Static_assert(sizeof(UKP_EXPORT_NAME) == sizeof(IREE_HAL_EXECUTABLE_PLUGIN_EXPORT_NAME), \"name\");",
        # the query function has the type the runtime looks up
        "extern const ukp_header_t** iree_hal_executable_plugin_query(uint32_t, void*);",
        "static iree_hal_executable_plugin_query_fn_t check_fn = "
        "(iree_hal_executable_plugin_query_fn_t)iree_hal_executable_plugin_query;",
    ]
    src = "#include <stddef.h>\n#include \"iree/hal/local/executable_plugin.h\"\n#include \"plugin_abi.h\"\n" + \
          "\n".join(checks) + "\nint main(void) { return check_fn == 0; }\n"
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "check.c")
        open(path, "w").write(src)
        r = subprocess.run(["gcc", "-std=c11", "-fsyntax-only", "-I", REFERENCE_SRC,
                            "-I", os.path.join(ROOT, "iree_amd", "csrc", "plugin"), path],
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert r.returncode == 0, r.stdout


# ---------------------------------------------------------------------------
# With a GPU: the imports, called as a dispatch calls them
# ---------------------------------------------------------------------------

class Mmt4dOperands(C.Structure):
    _fields_ = [("lhs", C.c_void_p), ("lhs_offset", C.c_size_t), ("lhs_stride0", C.c_size_t),
                ("rhs", C.c_void_p), ("rhs_offset", C.c_size_t), ("rhs_stride0", C.c_size_t),
                ("out", C.c_void_p), ("out_offset", C.c_size_t), ("out_stride0", C.c_size_t),
                ("M", C.c_size_t), ("N", C.c_size_t), ("K", C.c_size_t),
                ("M0", C.c_int32), ("N0", C.c_int32), ("K0", C.c_int32), ("flags", C.c_uint32),
                ("processor_data", C.c_void_p)]


class PackOperands(C.Structure):
    _fields_ = [("in_", C.c_void_p), ("in_offset", C.c_size_t), ("in_stride0", C.c_size_t), ("in_stride1", C.c_size_t),
                ("out", C.c_void_p), ("out_offset", C.c_size_t), ("out_stride0", C.c_size_t), ("out_stride1", C.c_size_t),
                ("in_size0", C.c_size_t), ("in_size1", C.c_size_t),
                ("out_size0", C.c_size_t), ("out_size1", C.c_size_t), ("out_size2", C.c_size_t), ("out_size3", C.c_size_t),
                ("padding_value", C.c_uint64), ("flags", C.c_uint32), ("processor_data", C.c_void_p)]


class UnpackOperands(C.Structure):
    _fields_ = [("in_", C.c_void_p), ("in_offset", C.c_size_t), ("in_stride0", C.c_size_t), ("in_stride1", C.c_size_t),
                ("out", C.c_void_p), ("out_offset", C.c_size_t), ("out_stride0", C.c_size_t), ("out_stride1", C.c_size_t),
                ("in_size0", C.c_size_t), ("in_size1", C.c_size_t), ("in_size2", C.c_size_t), ("in_size3", C.c_size_t),
                ("out_size0", C.c_size_t), ("out_size1", C.c_size_t),
                ("flags", C.c_uint32), ("processor_data", C.c_void_p)]


class QueryOperands(C.Structure):
    _fields_ = [("tile_size0", C.c_size_t), ("tile_size1", C.c_size_t), ("size0", C.c_size_t), ("size1", C.c_size_t),
                ("flags", C.c_uint32), ("processor_data", C.c_void_p)]


def _imports(v0):
    names = ["iree_uk_mmt4d", "iree_uk_pack", "iree_uk_query_tile_sizes_2d", "iree_uk_unpack"]
    status, _, fns = _resolve(v0, names)
    assert status == 0
    return {n: IMPORT_FN(f) for n, f in zip(names, fns)}


@pytest.mark.gpu
def test_imports_compute_what_the_oracle_computes(plugin, oracle_lib):
    _, v0 = plugin
    env = Environment(None, None)
    self_ptr = C.c_void_p()
    assert not v0.load(C.byref(env), 0, None, C.byref(self_ptr))
    imp = _imports(v0)

    # mmt4d, s8s8s32, with offsets into larger host buffers.
    M, N, K, M0, N0, K0 = 12, 20, 32, 8, 8, 4
    lhs = synth.uniform_int8(31, 0, 64 + M * K * M0 * K0)
    rhs = synth.uniform_int8(31, 1, 128 + N * K * N0 * K0)
    out = np.full(32 + M * N * M0 * N0, 7, dtype=np.int32)
    want = out.copy()
    flags = abi.MMT4D_TYPE_S8S8S32 | abi.MMT4D_ACCUMULATE | abi.MMT4D_ALLOW_GENERIC_FALLBACK
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data
    p.lhs_offset, p.rhs_offset, p.out_offset = 64, 128, 32
    p.lhs_stride0, p.rhs_stride0, p.out_stride0 = K * M0 * K0, K * N0 * K0, N * M0 * N0
    p.M, p.N, p.K, p.M0, p.N0, p.K0, p.flags = M, N, K, M0, N0, K0, flags
    oracle_lib.oracle_mmt4d(C.byref(p))
    ops = Mmt4dOperands(lhs.ctypes.data, 64, K * M0 * K0, rhs.ctypes.data, 128, K * N0 * K0,
                        out.ctypes.data, 32, N * M0 * N0, M, N, K, M0, N0, K0, flags, None)
    assert imp["iree_uk_mmt4d"](C.byref(ops), None, None) == 0
    assert np.array_equal(out, want)

    # pack then unpack, f32, ragged sizes: round trip and padding.
    R, Cc, T0, T1 = 37, 53, 8, 4
    O0, O1 = -(-R // T0), -(-Cc // T1)
    src = synth.normal_f32(32, 0, R * Cc)
    packed = np.full(O0 * O1 * T0 * T1, np.nan, dtype=np.float32)
    pk = PackOperands(src.ctypes.data, 0, Cc, 1, packed.ctypes.data, 0, O1 * T0 * T1, T0 * T1, R, Cc,
                      O0, O1, T0, T1, 0, abi.PACK_TYPE_F32F32, None)
    assert imp["iree_uk_pack"](C.byref(pk), None, None) == 0
    want_packed = np.empty_like(packed)
    q = abi.PackParams()
    q.in_buffer, q.out_buffer = src.ctypes.data, want_packed.ctypes.data
    q.in_stride0, q.in_stride1, q.out_stride0, q.out_stride1 = Cc, 1, O1 * T0 * T1, T0 * T1
    q.in_size0, q.in_size1 = R, Cc
    q.out_size0, q.out_size1, q.out_size2, q.out_size3 = O0, O1, T0, T1
    q.padding_value, q.flags = 0, abi.PACK_TYPE_F32F32
    oracle_lib.oracle_pack(C.byref(q))
    assert np.array_equal(packed.view(np.uint32), want_packed.view(np.uint32))
    back = np.full(R * Cc, -1.0, dtype=np.float32)
    up = UnpackOperands(packed.ctypes.data, 0, O1 * T0 * T1, T0 * T1, back.ctypes.data, 0, Cc, 1,
                        O0, O1, T0, T1, R, Cc, abi.UNPACK_TYPE_F32F32, None)
    assert imp["iree_uk_unpack"](C.byref(up), None, None) == 0
    assert np.array_equal(back, src)

    # query_tile_sizes_2d: results are the first fields of the operand struct.
    qo = QueryOperands(0, 0, 4096, 4096, 0x0200 | 0x01, None)   # matmul i8i8i32, lhs role
    assert imp["iree_uk_query_tile_sizes_2d"](C.byref(qo), None, None) == 0
    assert (qo.tile_size0, qo.tile_size1) == (16, 64)
    v0.unload(None)
