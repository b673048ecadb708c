"""Deterministic synthetic operands for the benchmark and the parity tests.

Counter-based: element i of stream s under seed k depends only on (k, s, i),
through the splitmix64 finaliser, so any slice can be regenerated on its own.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def bits64(seed, stream, n, start=0):
    """n 64-bit words: splitmix64 finaliser of a per-(seed, stream) counter."""
    with np.errstate(over="ignore"):
        base = (np.uint64(seed) * np.uint64(0xD1342543DE82EF95)
                + np.uint64(stream) * np.uint64(0xA0761D6478BD642F) + np.uint64(1))
        z = (np.arange(start, start + n, dtype=np.uint64) + base) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def uniform_int8(seed, stream, n):
    """int8 uniform over [-128, 127]."""
    words = bits64(seed, stream, (n + 7) // 8)
    return words.view(np.int8)[:n].copy()


def uniform_int4_packed(seed, stream, n_elems):
    """n_elems 4-bit values uniform over [-8, 7], two per byte, element 2b in
    the low nibble of byte b."""
    assert n_elems % 2 == 0
    words = bits64(seed, stream, (n_elems // 2 + 7) // 8)
    return words.view(np.uint8)[:n_elems // 2].copy()


def normal_f32(seed, stream, n, sigma=1.0):
    """N(0, sigma^2) by Box-Muller in float64, rounded once to float32."""
    m = (n + 1) // 2
    w = bits64(seed, stream, 2 * m)
    u1 = ((w[:m] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    u2 = (w[m:] >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.empty(2 * m, dtype=np.float64)
    out[0::2] = r * np.cos(2.0 * np.pi * u2)
    out[1::2] = r * np.sin(2.0 * np.pi * u2)
    return (out[:n] * sigma).astype(np.float32)


def f16_bits(x):
    """float32 -> IEEE binary16 bit patterns, round to nearest even."""
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def bf16_bits(x):
    """float32 -> bfloat16 bit patterns, round to nearest even (finite inputs)."""
    b = np.asarray(x, dtype=np.float32).view(np.uint32)
    return ((b + np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
