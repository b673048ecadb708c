"""Test-case construction shared by the CPU and GPU parity tests.

The grids, value ranges and layout randomisation follow the reference's own
ukernel tests so that a run here exercises what a run of those would:
  PRNG            tools/util.h:27-29, tools/util.c:74-103 (minstd, bits 8..23)
  buffer contents tools/util.c:105-166
  mmt4d cases     tools/mmt4d_test.c:352-441 (strides, offsets, buffers),
                  :459-479 (shapes), :499-502 (accumulate), :545-603 (tiles)
  pack cases      tools/pack_test.c:73-130, :132-195, :215-241
  unpack cases    tools/unpack_test.c:60-116, :118-182, :202-216
"""
import ctypes as C

import numpy as np

from iree_amd import abi

_MULT = 48271
_MOD = 2147483647
_BLOCK = 4096
_POW = np.empty(_BLOCK + 1, dtype=np.uint64)
_POW[0] = 1
for _i in range(1, _BLOCK + 1):
    _POW[_i] = (int(_POW[_i - 1]) * _MULT) % _MOD


class Lcg:
    """minstd_rand with the reference's ways of drawing small integers."""

    def __init__(self):
        self.state = 1

    def u32(self):
        self.state = (self.state * _MULT) % _MOD
        return self.state

    def u64(self):
        hi = self.u32()
        return ((hi << 32) + self.u32()) & 0xFFFFFFFFFFFFFFFF

    def r16(self):
        return (self.u32() >> 8) & 0xFFFF

    def r8(self):
        return self.r16() & 0xFF

    def r1(self):
        return self.r16() & 1

    def r16_array(self, n):
        """n successive r16() draws as an int64 array."""
        out = np.empty(n, dtype=np.int64)
        done = 0
        while done < n:
            m = min(_BLOCK, n - done)
            states = (np.uint64(self.state) * _POW[1:m + 1]) % np.uint64(_MOD)
            self.state = int(states[-1])
            out[done:done + m] = ((states >> np.uint64(8)) & np.uint64(0xFFFF)).astype(np.int64)
            done += m
        return out


def f32_to_f16_bits(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f32_to_bf16_bits(x):
    # Exact for the small integers used here (no rounding needed).
    return (np.asarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def random_bytes(kind, nbytes, rng):
    """nbytes of test data of element kind `kind` as a uint8 array.

    kind: s8 u8 i8 s16 u16 s32 u32 i32 f32 f16 bf16 s4 u4. Signless ("i")
    kinds first draw whether to behave as signed or unsigned.
    """
    if kind in ("i8", "i16", "i32"):
        kind = ("s" if rng.r1() else "u") + kind[1:]
    if kind in ("s4", "u4"):
        return (rng.r16_array(nbytes) & 0xFF).astype(np.uint8)
    size = {"s8": 1, "u8": 1, "s16": 2, "u16": 2, "f16": 2, "bf16": 2,
            "s32": 4, "u32": 4, "f32": 4}[kind]
    n = nbytes // size
    v = rng.r16_array(n)
    if kind == "f32":
        a = ((v % 4) - 2).astype(np.float32)
    elif kind == "f16":
        a = f32_to_f16_bits((v % 16) - 8)
    elif kind == "bf16":
        a = f32_to_bf16_bits((v % 4) - 2)
    elif kind == "s32":
        a = ((v % 2048) - 512).astype(np.int32)
    elif kind == "u32":
        a = (v % 2048).astype(np.uint32)
    elif kind == "s16":
        a = ((v % 2048) - 512).astype(np.int16)
    elif kind == "u16":
        a = (v % 2048).astype(np.uint16)
    elif kind == "s8":
        a = ((v % 256) - 128).astype(np.int8)
    elif kind == "u8":
        a = (v % 256).astype(np.uint8)
    else:
        raise ValueError(kind)
    out = np.zeros(nbytes, dtype=np.uint8)
    out[:n * size] = a.view(np.uint8)
    return out


MMT4D_KINDS = {
    abi.MMT4D_TYPE_F32F32F32: ("f32", "f32", "f32"),
    abi.MMT4D_TYPE_S8S8S32: ("s8", "s8", "s32"),
    abi.MMT4D_TYPE_F16F16F32: ("f16", "f16", "f32"),
    abi.MMT4D_TYPE_F16F16F16: ("f16", "f16", "f16"),
    abi.MMT4D_TYPE_BF16BF16F32: ("bf16", "bf16", "f32"),
    abi.MMT4D_TYPE_BF16BF16BF16: ("bf16", "bf16", "bf16"),
    abi.MMT4D_TYPE_S16S16S32: ("s16", "s16", "s32"),
    abi.MMT4D_TYPE_S16U4S32: ("s16", "u4", "s32"),
    abi.MMT4D_TYPE_S16S8S32: ("s16", "s8", "s32"),
    abi.MMT4D_TYPE_S8S4S32: ("s8", "s4", "s32"),
}

# Outer shapes (M, N, K) in tiles.
def mmt4d_shapes(out_is_bf16=False):
    big = 100 if out_is_bf16 else 1000
    return [(0, 1, 1), (0, 5, 7), (1, 0, 1), (5, 0, 7), (1, 1, 0), (5, 7, 0),
            (1, 1, 1), (1, 1, 2), (1, 1, 10), (1, 1, big), (2, 1, 1), (1, 2, 1),
            (2, 2, 2), (5, 7, 13)]


def _narrowed(m0):
    out, v = [], 1
    while v < m0:
        out.append(v)
        v *= 2
    return out + [m0]


def _tiles(type_flag, m0, n0, k0):
    return [(type_flag, m, n0, k0) for m in _narrowed(m0)]


# Tile shapes of the reference's generic section plus those of its x86-64
# section (the latter are where the compiled reference runs AVX2/AVX-512 tile
# functions rather than its generic loops).
MMT4D_TILES_GENERIC = (
    _tiles(abi.MMT4D_TYPE_F32F32F32, 3, 5, 7) + _tiles(abi.MMT4D_TYPE_S8S8S32, 9, 6, 3)
    + _tiles(abi.MMT4D_TYPE_S8S4S32, 9, 12, 2) + _tiles(abi.MMT4D_TYPE_S16S16S32, 7, 3, 6)
    + _tiles(abi.MMT4D_TYPE_S16U4S32, 5, 3, 2) + _tiles(abi.MMT4D_TYPE_S16S8S32, 7, 5, 6)
    + _tiles(abi.MMT4D_TYPE_F16F16F32, 4, 6, 5) + _tiles(abi.MMT4D_TYPE_F16F16F16, 3, 5, 8)
    + _tiles(abi.MMT4D_TYPE_BF16BF16F32, 11, 4, 1) + _tiles(abi.MMT4D_TYPE_BF16BF16BF16, 2, 9, 3))
SKIP = abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
MMT4D_TILES_X86 = (
    _tiles(abi.MMT4D_TYPE_F32F32F32, 8, 8, 1) + _tiles(abi.MMT4D_TYPE_F16F16F32, 8, 8, 1)
    + _tiles(abi.MMT4D_TYPE_F16F16F16 | SKIP, 8, 8, 1) + _tiles(abi.MMT4D_TYPE_S8S8S32, 8, 8, 2)
    + _tiles(abi.MMT4D_TYPE_S16S16S32, 8, 8, 2) + _tiles(abi.MMT4D_TYPE_F32F32F32, 16, 16, 1)
    + _tiles(abi.MMT4D_TYPE_F16F16F32, 16, 16, 1) + _tiles(abi.MMT4D_TYPE_F16F16F16 | SKIP, 16, 16, 1)
    + _tiles(abi.MMT4D_TYPE_S8S8S32, 16, 16, 2) + _tiles(abi.MMT4D_TYPE_S16S16S32, 16, 16, 2)
    + _tiles(abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 2) + _tiles(abi.MMT4D_TYPE_BF16BF16BF16 | SKIP, 16, 16, 2)
    + _tiles(abi.MMT4D_TYPE_S16U4S32, 1, 32, 8))
# Tile shapes of this library's specialised GPU kernels (the benchmark configurations).
MMT4D_TILES_GPU = (
    _tiles(abi.MMT4D_TYPE_S8S8S32, 8, 8, 4) + _tiles(abi.MMT4D_TYPE_F16F16F32, 16, 16, 16)
    + _tiles(abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 8) + _tiles(abi.MMT4D_TYPE_S8S4S32, 16, 16, 32)
    + _tiles(abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 16) + _tiles(abi.MMT4D_TYPE_S8S8S32, 16, 16, 64))


def _even_up(v, bits):
    while (v * bits) % 8:
        v += 1
    return v


class Mmt4dCase:
    """One mmt4d problem with reference-style random layout and contents."""

    def __init__(self, flags, M, N, K, M0, N0, K0, rng, tight=False):
        self.flags = flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK
        t = flags & abi.MMT4D_TYPE_MASK
        self.kinds = MMT4D_KINDS[t]
        self.bits = abi.MMT4D_BITS[t]
        lb, rb, ob = self.bits
        self.M, self.N, self.K, self.M0, self.N0, self.K0 = M, N, K, M0, N0, K0
        slack = (lambda: 0) if tight else rng.r1
        self.lhs_stride0 = _even_up(K * M0 * K0 + slack(), lb)
        self.rhs_stride0 = _even_up(K * N0 * K0 + slack(), rb)
        self.out_stride0 = _even_up(N * M0 * N0 + slack(), ob)
        self.lhs = random_bytes(self.kinds[0], M * self.lhs_stride0 * lb // 8, rng)
        self.rhs = random_bytes(self.kinds[1], N * self.rhs_stride0 * rb // 8, rng)
        self.lhs_offset = _even_up(slack(), lb)
        self.rhs_offset = _even_up(slack(), rb)
        self.out_offset = _even_up(slack(), ob)
        self.out_init = random_bytes(self.kinds[2], M * self.out_stride0 * ob // 8, rng)

    def label(self):
        return "%s %dx%dx%d tiles %dx%dx%d flags=%#x" % (
            abi.MMT4D_NAMES[self.flags & 0xFF], self.M, self.N, self.K,
            self.M0, self.N0, self.K0, self.flags)

    def params(self, lhs_addr, rhs_addr, out_addr):
        """Params whose `buffer + offset` lands on the given addresses."""
        lb, rb, ob = self.bits
        p = abi.Mmt4dParams()
        p.lhs_buffer = lhs_addr - self.lhs_offset * lb // 8
        p.rhs_buffer = rhs_addr - self.rhs_offset * rb // 8
        p.out_buffer = out_addr - self.out_offset * ob // 8
        p.lhs_offset, p.rhs_offset, p.out_offset = self.lhs_offset, self.rhs_offset, self.out_offset
        p.lhs_stride0, p.rhs_stride0, p.out_stride0 = self.lhs_stride0, self.rhs_stride0, self.out_stride0
        p.M, p.N, p.K, p.M0, p.N0, p.K0 = self.M, self.N, self.K, self.M0, self.N0, self.K0
        p.flags = self.flags
        return p

    def run_host(self, fn):
        """Calls fn(byref(params)) on host copies; returns the out bytes."""
        # +16 so that zero-sized buffers still have an address.
        lhs = np.concatenate([self.lhs, np.zeros(16, np.uint8)])
        rhs = np.concatenate([self.rhs, np.zeros(16, np.uint8)])
        out = np.concatenate([self.out_init, np.zeros(16, np.uint8)])
        p = self.params(lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data)
        fn(C.byref(p))
        return out[:self.out_init.size].copy()


def mmt4d_cases(tile, rng=None):
    """All (shape x accumulate) cases of the reference grid for one tile."""
    flags, M0, N0, K0 = tile
    rng = rng or Lcg()
    out_bf16 = (flags & 0xFF) == abi.MMT4D_TYPE_BF16BF16BF16
    cases = []
    for (M, N, K) in mmt4d_shapes(out_bf16):
        for acc in (0, abi.MMT4D_ACCUMULATE):
            cases.append(Mmt4dCase(flags | acc, M, N, K, M0, N0, K0, rng))
    return cases


PACK_KINDS = {abi.PACK_TYPE_F32F32: "f32", abi.PACK_TYPE_I8I8: "i8", abi.PACK_TYPE_I32I32: "i32",
              abi.PACK_TYPE_F16F16: "f16", abi.PACK_TYPE_BF16BF16: "bf16"}
UNPACK_KINDS = {abi.UNPACK_TYPE_F32F32: "f32", abi.UNPACK_TYPE_I32I32: "i32",
                abi.UNPACK_TYPE_F16F16: "f16", abi.UNPACK_TYPE_BF16BF16: "bf16"}
PACK_NAMES = {1: "f32", 2: "i8", 3: "i32", 4: "f16", 5: "bf16"}

PACK_TILES_GENERIC = [(abi.PACK_TYPE_F32F32, 3, 5), (abi.PACK_TYPE_I8I8, 4, 2),
                      (abi.PACK_TYPE_I32I32, 3, 4), (abi.PACK_TYPE_F16F16, 6, 7),
                      (abi.PACK_TYPE_BF16BF16, 9, 2)]
PACK_TILES_X86 = [(abi.PACK_TYPE_F32F32, 8, 1), (abi.PACK_TYPE_I8I8, 8, 2),
                  (abi.PACK_TYPE_F32F32, 8, 8), (abi.PACK_TYPE_I32I32, 8, 8),
                  (abi.PACK_TYPE_F32F32, 16, 1), (abi.PACK_TYPE_BF16BF16, 16, 2),
                  (abi.PACK_TYPE_I8I8, 16, 2), (abi.PACK_TYPE_F32F32, 16, 16),
                  (abi.PACK_TYPE_I32I32, 16, 16)]
# Operand layouts of the benchmark's mmt4d configurations.
PACK_TILES_GPU = [(abi.PACK_TYPE_I8I8, 8, 4), (abi.PACK_TYPE_F16F16, 16, 16),
                  (abi.PACK_TYPE_BF16BF16, 16, 8), (abi.PACK_TYPE_I8I8, 16, 32),
                  (abi.PACK_TYPE_BF16BF16, 1, 8), (abi.PACK_TYPE_I32I32, 8, 8)]
UNPACK_TILES_GENERIC = [(abi.UNPACK_TYPE_F32F32, 3, 5), (abi.UNPACK_TYPE_I32I32, 3, 4),
                        (abi.UNPACK_TYPE_F16F16, 6, 7), (abi.UNPACK_TYPE_BF16BF16, 9, 2)]
UNPACK_TILES_X86 = [(abi.UNPACK_TYPE_F32F32, 8, 8), (abi.UNPACK_TYPE_I32I32, 8, 8),
                    (abi.UNPACK_TYPE_F32F32, 16, 16), (abi.UNPACK_TYPE_I32I32, 16, 16)]
UNPACK_TILES_GPU = [(abi.UNPACK_TYPE_F32F32, 16, 1), (abi.UNPACK_TYPE_I32I32, 8, 8),
                    (abi.UNPACK_TYPE_F32F32, 1, 16), (abi.UNPACK_TYPE_F32F32, 4, 16),
                    (abi.UNPACK_TYPE_BF16BF16, 16, 8)]

OUTER_SHAPES = [(0, 1), (1, 0), (1, 1), (3, 2), (9, 33)]
PAD_NONE, PAD_ONE_TILE, PAD_A_LOT = 0, 1, 2


class PackCase:
    def __init__(self, type_flag, tile0, tile1, outer, tr_inner, tr_outer, pad, rng):
        self.elem = abi.PACK_ELEM_BYTES[type_flag]
        self.kind = PACK_KINDS[type_flag]
        self.flags = type_flag
        o0, o1 = outer
        if pad == PAD_A_LOT:
            o0, o1 = o0 + 16, o1 + 16
        self.out_size0, self.out_size1 = o0, o1
        if tr_outer:
            self.flags |= abi.PACK_TRANSPOSE_OUTER
            self.out_size0, self.out_size1 = o1, o0
        self.out_size2, self.out_size3 = tile0, tile1
        t0, t1 = tile0, tile1
        if tr_inner:
            self.flags |= abi.PACK_TRANSPOSE_INNER
            t0, t1 = tile1, tile0
        self.in_size0, self.in_size1 = o0 * t0, o1 * t1
        if pad == PAD_ONE_TILE:
            self.in_size0 = max(0, self.in_size0 - rng.r16() % t0)
            self.in_size1 = max(0, self.in_size1 - rng.r16() % t1)
        self.padding_value = rng.u64()
        self.in_stride1 = 1 + rng.r1()
        self.in_stride0 = self.in_size1 * self.in_stride1 + rng.r1()
        self.out_stride1 = tile0 * tile1
        self.out_stride0 = self.out_size1 * self.out_stride1 + rng.r1()
        self.inp = random_bytes(self.kind, self.in_size0 * self.in_stride0 * self.elem, rng)
        self.in_offset = rng.r16()
        self.out_offset = rng.r16()
        self.out_init = random_bytes(self.kind, self.out_size0 * self.out_stride0 * self.elem, rng)

    def label(self):
        return "pack %s in %dx%d -> %dx%dx%dx%d flags=%#x" % (
            self.kind, self.in_size0, self.in_size1, self.out_size0, self.out_size1,
            self.out_size2, self.out_size3, self.flags)

    def params(self, in_addr, out_addr):
        p = abi.PackParams()
        p.in_buffer = in_addr - self.in_offset * self.elem
        p.out_buffer = out_addr - self.out_offset * self.elem
        p.in_offset, p.out_offset = self.in_offset, self.out_offset
        p.in_stride0, p.in_stride1 = self.in_stride0, self.in_stride1
        p.out_stride0, p.out_stride1 = self.out_stride0, self.out_stride1
        p.in_size0, p.in_size1 = self.in_size0, self.in_size1
        p.out_size0, p.out_size1 = self.out_size0, self.out_size1
        p.out_size2, p.out_size3 = self.out_size2, self.out_size3
        p.padding_value = self.padding_value
        p.flags = self.flags
        return p

    def run_host(self, fn):
        inp = np.concatenate([self.inp, np.zeros(16, np.uint8)])
        out = np.concatenate([self.out_init, np.zeros(16, np.uint8)])
        p = self.params(inp.ctypes.data, out.ctypes.data)
        fn(C.byref(p))
        return out[:self.out_init.size].copy()

    def written_mask(self):
        """Boolean per output byte: True where pack must have written."""
        n = self.out_size1 * self.out_size2 * self.out_size3
        m = np.zeros((self.out_size0, self.out_stride0 * self.elem), dtype=bool)
        m[:, :n * self.elem] = True
        return m.reshape(-1)


def pack_cases(tile, rng=None):
    type_flag, tile0, tile1 = tile
    rng = rng or Lcg()
    cases = []
    for outer in OUTER_SHAPES:
        for tr_inner in (0, 1):
            for tr_outer in (0, 1):
                for pad in (PAD_NONE, PAD_ONE_TILE, PAD_A_LOT):
                    cases.append(PackCase(type_flag, tile0, tile1, outer, tr_inner, tr_outer, pad, rng))
    return cases


class UnpackCase:
    def __init__(self, type_flag, tile0, tile1, outer, tr_inner, tr_outer, pad, rng):
        self.elem = abi.UNPACK_ELEM_BYTES[type_flag]
        self.kind = UNPACK_KINDS[type_flag]
        self.flags = type_flag
        o0, o1 = outer
        # The tiled input gets 16 extra tiles of pure padding per dimension in
        # the PAD_A_LOT case; the 2-D output size is derived without them.
        extra = 16 if pad == PAD_A_LOT else 0
        self.in_size0, self.in_size1 = o0 + extra, o1 + extra
        if tr_outer:
            self.flags |= abi.UNPACK_TRANSPOSE_OUTER
            o0, o1 = o1, o0
        self.in_size2, self.in_size3 = tile0, tile1
        t0, t1 = tile0, tile1
        if tr_inner:
            self.flags |= abi.UNPACK_TRANSPOSE_INNER
            t0, t1 = tile1, tile0
        self.out_size0, self.out_size1 = o0 * t0, o1 * t1
        if pad == PAD_ONE_TILE:
            self.out_size0 = max(0, self.out_size0 - rng.r16() % t0)
            self.out_size1 = max(0, self.out_size1 - rng.r16() % t1)
        self.out_stride1 = 1 + rng.r1()
        self.out_stride0 = self.out_size1 * self.out_stride1 + rng.r1()
        self.in_stride1 = tile0 * tile1
        self.in_stride0 = self.in_size1 * self.in_stride1 + rng.r1()
        self.inp = random_bytes(self.kind, self.in_size0 * self.in_stride0 * self.elem, rng)
        self.in_offset = rng.r16()
        self.out_offset = rng.r16()
        self.out_init = random_bytes(self.kind, self.out_size0 * self.out_stride0 * self.elem, rng)

    def label(self):
        return "unpack %s in %dx%dx%dx%d -> %dx%d flags=%#x" % (
            self.kind, self.in_size0, self.in_size1, self.in_size2, self.in_size3,
            self.out_size0, self.out_size1, self.flags)

    def params(self, in_addr, out_addr):
        p = abi.UnpackParams()
        p.in_buffer = in_addr - self.in_offset * self.elem
        p.out_buffer = out_addr - self.out_offset * self.elem
        p.in_offset, p.out_offset = self.in_offset, self.out_offset
        p.in_stride0, p.in_stride1 = self.in_stride0, self.in_stride1
        p.out_stride0, p.out_stride1 = self.out_stride0, self.out_stride1
        p.in_size0, p.in_size1 = self.in_size0, self.in_size1
        p.in_size2, p.in_size3 = self.in_size2, self.in_size3
        p.out_size0, p.out_size1 = self.out_size0, self.out_size1
        p.flags = self.flags
        return p

    def run_host(self, fn):
        inp = np.concatenate([self.inp, np.zeros(16, np.uint8)])
        out = np.concatenate([self.out_init, np.zeros(16, np.uint8)])
        p = self.params(inp.ctypes.data, out.ctypes.data)
        fn(C.byref(p))
        return out[:self.out_init.size].copy()


def unpack_cases(tile, rng=None):
    type_flag, tile0, tile1 = tile
    rng = rng or Lcg()
    cases = []
    for outer in OUTER_SHAPES:
        for tr_inner in (0, 1):
            for tr_outer in (0, 1):
                for pad in (PAD_NONE, PAD_ONE_TILE, PAD_A_LOT):
                    cases.append(UnpackCase(type_flag, tile0, tile1, outer, tr_inner, tr_outer, pad, rng))
    return cases
