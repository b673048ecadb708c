"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

ctypes access to the two CPU checkers built by oracle/Makefile:

* ``liboracle.so``  this repository's scalar restatement (uk_oracle.c);
* ``_ref/libiree_uk_ref[_dbg].so``  the reference's ukernel sources compiled
  unchanged, present only where the reference tree was available at build time.

Only tests/, the smoke check in __graft_entry__.py and the cpu_baseline leg of
bench.py may import this package.
"""
import ctypes as C
import os
import subprocess

from iree_amd import abi

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "liboracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libiree_uk_ref.so")
_REF_DBG_SO = os.path.join(_HERE, "_ref", "libiree_uk_ref_dbg.so")

_cache = {}


def build(quiet=True):
    """Runs oracle/Makefile (liboracle.so always, _ref when sources exist)."""
    subprocess.run(["make", "-C", _HERE, "-j8", "all"], check=True,
                   stdout=subprocess.DEVNULL if quiet else None)
    _cache.clear()


def lib():
    """The scalar restatement; built on first use if missing."""
    if "oracle" not in _cache:
        if not os.path.exists(_ORACLE_SO):
            build()
        l = C.CDLL(_ORACLE_SO)
        l.oracle_mmt4d.argtypes = [C.POINTER(abi.Mmt4dParams)]
        l.oracle_mmt4d.restype = None
        l.oracle_mmt4d_mt.argtypes = [C.POINTER(abi.Mmt4dParams), C.c_int]
        l.oracle_mmt4d_mt.restype = None
        l.oracle_pack.argtypes = [C.POINTER(abi.PackParams)]
        l.oracle_pack.restype = None
        l.oracle_unpack.argtypes = [C.POINTER(abi.UnpackParams)]
        l.oracle_unpack.restype = None
        l.oracle_f16_to_f32.argtypes = [C.c_uint16]
        l.oracle_f16_to_f32.restype = C.c_float
        l.oracle_bf16_to_f32.argtypes = [C.c_uint16]
        l.oracle_bf16_to_f32.restype = C.c_float
        l.oracle_f32_to_f16.argtypes = [C.c_float]
        l.oracle_f32_to_f16.restype = C.c_uint16
        l.oracle_f32_to_bf16.argtypes = [C.c_float]
        l.oracle_f32_to_bf16.restype = C.c_uint16
        _cache["oracle"] = l
    return _cache["oracle"]


def ref_lib(debug=False):
    """The compiled reference, or None where it was not built."""
    key = "ref_dbg" if debug else "ref"
    if key not in _cache:
        path = _REF_DBG_SO if debug else _REF_SO
        if not os.path.exists(path):
            _cache[key] = None
        else:
            l = C.CDLL(path)
            l.ref_mmt4d.argtypes = [C.POINTER(abi.Mmt4dParams)]
            l.ref_mmt4d.restype = None
            l.ref_mmt4d_info.argtypes = [C.POINTER(abi.Mmt4dParams)]
            l.ref_mmt4d_info.restype = C.c_uint32
            l.ref_mmt4d_mt.argtypes = [C.POINTER(abi.Mmt4dParams), C.c_int]
            l.ref_mmt4d_mt.restype = None
            l.ref_pack.argtypes = [C.POINTER(abi.PackParams)]
            l.ref_pack.restype = None
            l.ref_pack_mt.argtypes = [C.POINTER(abi.PackParams), C.c_int]
            l.ref_pack_mt.restype = C.c_int
            l.ref_unpack.argtypes = [C.POINTER(abi.UnpackParams)]
            l.ref_unpack.restype = None
            l.ref_unpack_mt.argtypes = [C.POINTER(abi.UnpackParams), C.c_int]
            l.ref_unpack_mt.restype = C.c_int
            l.ref_query_tile_sizes_2d.argtypes = [
                C.POINTER(abi.QueryTileSizes2dParams),
                C.POINTER(abi.QueryTileSizes2dOutParams)]
            l.ref_query_tile_sizes_2d.restype = None
            l.ref_host_cpu_data.argtypes = [C.POINTER(C.c_uint64)]
            l.ref_host_cpu_data.restype = None
            l.ref_fail_count.restype = C.c_int
            l.ref_set_abort_on_fail.argtypes = [C.c_int]
            _cache[key] = l
    return _cache[key]


def host_cpu_data():
    """8 feature words for this host, or zeros without the compiled reference."""
    words = (C.c_uint64 * 8)()
    r = ref_lib()
    if r is not None:
        r.ref_host_cpu_data(words)
    return words
