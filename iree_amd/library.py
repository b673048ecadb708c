"""Loads the HIP microkernel library and binds its C ABI with ctypes.

There is no CPU fallback: if libiree_uk_mi355x.so is missing, loading raises.
"""
import ctypes as C
import os

from . import abi

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libiree_uk_mi355x.so")

FAIL_HANDLER = C.CFUNCTYPE(None, C.c_char_p, C.c_int, C.c_char_p, C.c_char_p)

_lib = None


def load():
    """Returns the bound library; builds nothing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s not found: build it with `python -m iree_amd.build` "
            "(there is no CPU fallback for the microkernels)" % LIB_PATH)
    l = C.CDLL(LIB_PATH)
    ix, vp, u64p = abi.index_t, C.c_void_p, C.POINTER(C.c_uint64)
    l.iree_uk_mmt4d.argtypes = [vp, ix, ix, vp, ix, ix, vp, ix, ix, ix, ix, ix,
                                C.c_int32, C.c_int32, C.c_int32, C.c_uint32, u64p]
    l.iree_uk_mmt4d.restype = None
    l.iree_uk_mmt4d_p.argtypes = [C.POINTER(abi.Mmt4dParams)]
    l.iree_uk_mmt4d_p.restype = None
    l.iree_uk_mi355x_mmt4d_noalloc_p.argtypes = [C.POINTER(abi.Mmt4dParams)]
    l.iree_uk_mi355x_mmt4d_noalloc_p.restype = None
    l.iree_uk_mmt4d_info.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_uint32, u64p]
    l.iree_uk_mmt4d_info.restype = C.c_uint32
    l.iree_uk_mmt4d_info_p.argtypes = [C.POINTER(abi.Mmt4dParams)]
    l.iree_uk_mmt4d_info_p.restype = C.c_uint32
    l.iree_uk_pack.argtypes = [vp, ix, ix, ix, vp, ix, ix, ix, ix, ix, ix, ix, ix, ix,
                               C.c_uint64, C.c_uint32, u64p]
    l.iree_uk_pack.restype = None
    l.iree_uk_pack_p.argtypes = [C.POINTER(abi.PackParams)]
    l.iree_uk_pack_p.restype = None
    l.iree_uk_unpack.argtypes = [vp, ix, ix, ix, vp, ix, ix, ix, ix, ix, ix, ix, ix, ix,
                                 C.c_uint32, u64p]
    l.iree_uk_unpack.restype = None
    l.iree_uk_unpack_p.argtypes = [C.POINTER(abi.UnpackParams)]
    l.iree_uk_unpack_p.restype = None
    l.iree_uk_query_tile_sizes_2d.argtypes = [C.POINTER(abi.QueryTileSizes2dParams),
                                              C.POINTER(abi.QueryTileSizes2dOutParams)]
    l.iree_uk_query_tile_sizes_2d.restype = None
    l.iree_uk_mi355x_version.restype = C.c_int
    l.iree_uk_mi355x_multi_mma_i32_16x16x64_i8.argtypes = [vp, vp, vp, C.c_longlong, C.c_longlong] + [C.c_int32] * 6
    l.iree_uk_mi355x_multi_mma_i32_16x16x64_i8.restype = C.c_int
    l.iree_uk_mi355x_init.argtypes = [C.c_int]
    l.iree_uk_mi355x_init.restype = C.c_int
    l.iree_uk_mi355x_set_stream.argtypes = [vp, C.c_int]
    l.iree_uk_mi355x_set_stream.restype = None
    l.iree_uk_mi355x_set_fail_handler.argtypes = [FAIL_HANDLER]
    l.iree_uk_mi355x_set_fail_handler.restype = None
    l.iree_uk_mi355x_last_kernel.restype = C.c_char_p
    _lib = l
    return l


_bench_probe = None


def load_bench_probe():
    """The benchmark's probes (csrc/bench/), a helper library of its own: what the
    matrix pipe sustains on given operand bytes, what the device streams to and
    from HBM with plain read, fill and copy kernels, and where the time of one
    launch of the 256x256 int8 kernel goes (the kernel's own source compiled
    with its timeline readings on). Not part of the microkernel ABI."""
    global _bench_probe
    if _bench_probe is None:
        path = os.path.join(HERE, "libuk_bench_probe.so")
        if not os.path.exists(path):
            raise RuntimeError("%s not found: build it with `python -m iree_amd.build`" % path)
        l = C.CDLL(path)
        l.uk_bench_probe_matrix_pipe.argtypes = [C.c_uint32, C.c_void_p, C.c_longlong, C.c_int, C.c_int,
                                                 C.POINTER(C.c_double), C.POINTER(C.c_double)]
        l.uk_bench_probe_matrix_pipe.restype = C.c_int
        l.uk_bench_probe_hbm_stream.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_longlong, C.c_int, C.c_int,
                                                C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        l.uk_bench_probe_hbm_stream.restype = C.c_int
        l.uk_bench_probe_mmt4d_timeline.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_longlong, C.c_longlong,
                                                    C.c_longlong, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                                    C.POINTER(C.c_double), C.POINTER(C.c_int)]
        l.uk_bench_probe_mmt4d_timeline.restype = C.c_int
        l.uk_bench_probe_mmt4d_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_longlong, C.c_longlong,
                                                  C.c_longlong, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
        l.uk_bench_probe_mmt4d_launch.restype = C.c_int
        _bench_probe = l
    return _bench_probe
