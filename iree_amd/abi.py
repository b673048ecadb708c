"""ctypes mirror of include/iree_uk_mi355x.h.

Struct layouts follow the reference's parameter structs field for field
(mmt4d_internal.h:14-32, pack_internal.h:12-30, unpack_internal.h:12-29,
query_tile_sizes.h:17-27); flag values follow exported_bits.h:29-83.
"""
import ctypes as C

index_t = C.c_longlong

# --- mmt4d flags (exported_bits.h:29-49) -----------------------------------
MMT4D_TYPE_MASK = 0xFF
MMT4D_TYPE_F32F32F32 = 0x01
MMT4D_TYPE_S8S8S32 = 0x02
MMT4D_TYPE_F16F16F32 = 0x03
MMT4D_TYPE_F16F16F16 = 0x04
MMT4D_TYPE_BF16BF16F32 = 0x05
MMT4D_TYPE_BF16BF16BF16 = 0x06
MMT4D_TYPE_S16S16S32 = 0x07
MMT4D_TYPE_S16U4S32 = 0x08
MMT4D_TYPE_S16S8S32 = 0x09
MMT4D_TYPE_S8S4S32 = 0x0A
MMT4D_TYPE_END = 0x0B
MMT4D_ACCUMULATE = 0x100
MMT4D_ALLOW_GENERIC_FALLBACK = 0x200
MMT4D_SKIP_INTERMEDIATE_ROUNDINGS = 0x400
MMT4D_INFO_HAVE_ARCH_TILE_FUNCTION = 0x1

# --- pack / unpack flags (exported_bits.h:56-83) ---------------------------
PACK_TYPE_MASK = 0xFF
PACK_TYPE_F32F32 = 0x01
PACK_TYPE_I8I8 = 0x02
PACK_TYPE_I32I32 = 0x03
PACK_TYPE_F16F16 = 0x04
PACK_TYPE_BF16BF16 = 0x05
PACK_TRANSPOSE_INNER = 0x100
PACK_TRANSPOSE_OUTER = 0x200
UNPACK_TYPE_MASK = 0xFF
UNPACK_TYPE_F32F32 = 0x01
UNPACK_TYPE_I32I32 = 0x03
UNPACK_TYPE_F16F16 = 0x04
UNPACK_TYPE_BF16BF16 = 0x05
UNPACK_TRANSPOSE_INNER = 0x100
UNPACK_TRANSPOSE_OUTER = 0x200

# --- query_tile_sizes flags (exported_bits.h:91-107) -----------------------
QTS_ROLE_LHS = 0x01
QTS_ROLE_RHS = 0x02
QTS_ROLE_RESULT = 0x03
QTS_OP_MATMUL_F32F32F32 = 0x0100
QTS_OP_MATMUL_I8I8I32 = 0x0200
QTS_OP_MATMUL_F16F16F32 = 0x0300
QTS_OP_MATMUL_F16F16F16 = 0x0400
QTS_OP_MATMUL_BF16BF16F32 = 0x0500
QTS_OP_MATMUL_BF16BF16BF16 = 0x0600

# (lhs bits, rhs bits, out bits) per mmt4d type flag.
MMT4D_BITS = {
    MMT4D_TYPE_F32F32F32: (32, 32, 32),
    MMT4D_TYPE_S8S8S32: (8, 8, 32),
    MMT4D_TYPE_F16F16F32: (16, 16, 32),
    MMT4D_TYPE_F16F16F16: (16, 16, 16),
    MMT4D_TYPE_BF16BF16F32: (16, 16, 32),
    MMT4D_TYPE_BF16BF16BF16: (16, 16, 16),
    MMT4D_TYPE_S16S16S32: (16, 16, 32),
    MMT4D_TYPE_S16U4S32: (16, 4, 32),
    MMT4D_TYPE_S16S8S32: (16, 8, 32),
    MMT4D_TYPE_S8S4S32: (8, 4, 32),
}
MMT4D_NAMES = {
    MMT4D_TYPE_F32F32F32: "f32f32f32", MMT4D_TYPE_S8S8S32: "s8s8s32",
    MMT4D_TYPE_F16F16F32: "f16f16f32", MMT4D_TYPE_F16F16F16: "f16f16f16",
    MMT4D_TYPE_BF16BF16F32: "bf16bf16f32", MMT4D_TYPE_BF16BF16BF16: "bf16bf16bf16",
    MMT4D_TYPE_S16S16S32: "s16s16s32", MMT4D_TYPE_S16U4S32: "s16u4s32",
    MMT4D_TYPE_S16S8S32: "s16s8s32", MMT4D_TYPE_S8S4S32: "s8s4s32",
}
PACK_ELEM_BYTES = {PACK_TYPE_F32F32: 4, PACK_TYPE_I8I8: 1, PACK_TYPE_I32I32: 4,
                   PACK_TYPE_F16F16: 2, PACK_TYPE_BF16BF16: 2}
UNPACK_ELEM_BYTES = {UNPACK_TYPE_F32F32: 4, UNPACK_TYPE_I32I32: 4,
                     UNPACK_TYPE_F16F16: 2, UNPACK_TYPE_BF16BF16: 2}


class Mmt4dParams(C.Structure):
    _fields_ = [
        ("lhs_buffer", C.c_void_p), ("lhs_offset", index_t), ("lhs_stride0", index_t),
        ("rhs_buffer", C.c_void_p), ("rhs_offset", index_t), ("rhs_stride0", index_t),
        ("out_buffer", C.c_void_p), ("out_offset", index_t), ("out_stride0", index_t),
        ("M", index_t), ("N", index_t), ("K", index_t),
        ("M0", C.c_int32), ("N0", C.c_int32), ("K0", C.c_int32),
        ("flags", C.c_uint32), ("cpu_data", C.POINTER(C.c_uint64)),
    ]


class PackParams(C.Structure):
    _fields_ = [
        ("in_buffer", C.c_void_p), ("in_offset", index_t),
        ("in_stride0", index_t), ("in_stride1", index_t),
        ("out_buffer", C.c_void_p), ("out_offset", index_t),
        ("out_stride0", index_t), ("out_stride1", index_t),
        ("in_size0", index_t), ("in_size1", index_t),
        ("out_size0", index_t), ("out_size1", index_t),
        ("out_size2", index_t), ("out_size3", index_t),
        ("padding_value", C.c_uint64), ("flags", C.c_uint32),
        ("cpu_data", C.POINTER(C.c_uint64)),
    ]


class UnpackParams(C.Structure):
    _fields_ = [
        ("in_buffer", C.c_void_p), ("in_offset", index_t),
        ("in_stride0", index_t), ("in_stride1", index_t),
        ("out_buffer", C.c_void_p), ("out_offset", index_t),
        ("out_stride0", index_t), ("out_stride1", index_t),
        ("in_size0", index_t), ("in_size1", index_t),
        ("in_size2", index_t), ("in_size3", index_t),
        ("out_size0", index_t), ("out_size1", index_t),
        ("flags", C.c_uint32), ("cpu_data", C.POINTER(C.c_uint64)),
    ]


class QueryTileSizes2dParams(C.Structure):
    _fields_ = [("flags", C.c_uint32), ("size0", index_t), ("size1", index_t),
                ("cpu_data", C.POINTER(C.c_uint64))]


class QueryTileSizes2dOutParams(C.Structure):
    _fields_ = [("tile_size0", index_t), ("tile_size1", index_t)]


def mmt4d_spans(p):
    """Bytes of (lhs, rhs, out) reachable from `buffer + offset` for params p."""
    lb, rb, ob = MMT4D_BITS[p.flags & MMT4D_TYPE_MASK]

    def span(rows, stride, row_elems, bits):
        if rows <= 0:
            return 0
        return ((rows - 1) * stride + row_elems) * bits // 8

    return (span(p.M, p.lhs_stride0, p.K * p.M0 * p.K0, lb),
            span(p.N, p.rhs_stride0, p.K * p.N0 * p.K0, rb),
            span(p.M, p.out_stride0, p.N * p.M0 * p.N0, ob))
