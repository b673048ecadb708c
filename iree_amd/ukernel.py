"""Host-side entry points with the reference's names and argument order.

Each function forwards to the C ABI of libiree_uk_mi355x.so. Buffer arguments
may be integers (addresses), torch tensors (their data_ptr) or numpy arrays
(their data address); offsets and strides are in elements, as in the
reference (mmt4d.h:14-21, pack.h:26-34, unpack.h:17-25).
"""
import ctypes as C

from . import abi, library


def _addr(buf):
    if buf is None:
        return None
    if isinstance(buf, int):
        return buf
    if hasattr(buf, "data_ptr"):
        return buf.data_ptr()
    if hasattr(buf, "ctypes"):
        return buf.ctypes.data
    raise TypeError("unsupported buffer type %r" % type(buf))


def mmt4d(lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0,
          out_buffer, out_offset, out_stride0, M, N, K, M0, N0, K0, flags, cpu_data=None):
    library.load().iree_uk_mmt4d(_addr(lhs_buffer), lhs_offset, lhs_stride0,
                                 _addr(rhs_buffer), rhs_offset, rhs_stride0,
                                 _addr(out_buffer), out_offset, out_stride0,
                                 M, N, K, M0, N0, K0, flags, cpu_data)


def mmt4d_info(M0, N0, K0, flags, cpu_data=None):
    return library.load().iree_uk_mmt4d_info(M0, N0, K0, flags, cpu_data)


def pack(in_buffer, in_offset, in_stride0, in_stride1, out_buffer, out_offset, out_stride0,
         out_stride1, in_size0, in_size1, out_size0, out_size1, out_size2, out_size3,
         padding_value, flags, cpu_data=None):
    library.load().iree_uk_pack(_addr(in_buffer), in_offset, in_stride0, in_stride1,
                                _addr(out_buffer), out_offset, out_stride0, out_stride1,
                                in_size0, in_size1, out_size0, out_size1, out_size2, out_size3,
                                padding_value, flags, cpu_data)


def unpack(in_buffer, in_offset, in_stride0, in_stride1, out_buffer, out_offset, out_stride0,
           out_stride1, in_size0, in_size1, in_size2, in_size3, out_size0, out_size1, flags,
           cpu_data=None):
    library.load().iree_uk_unpack(_addr(in_buffer), in_offset, in_stride0, in_stride1,
                                  _addr(out_buffer), out_offset, out_stride0, out_stride1,
                                  in_size0, in_size1, in_size2, in_size3, out_size0, out_size1,
                                  flags, cpu_data)


def query_tile_sizes_2d(flags, size0=0, size1=0, cpu_data=None):
    p = abi.QueryTileSizes2dParams(flags=flags, size0=size0, size1=size1)
    o = abi.QueryTileSizes2dOutParams()
    library.load().iree_uk_query_tile_sizes_2d(C.byref(p), C.byref(o))
    return o.tile_size0, o.tile_size1


def set_stream(stream=None, asynchronous=False):
    """stream: None (HIP null stream), an int handle or a torch.cuda.Stream."""
    handle = None
    if stream is not None:
        handle = stream if isinstance(stream, int) else stream.cuda_stream
    library.load().iree_uk_mi355x_set_stream(handle, 1 if asynchronous else 0)


def last_kernel():
    return library.load().iree_uk_mi355x_last_kernel().decode()
