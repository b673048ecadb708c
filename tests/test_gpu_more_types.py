"""GPU parity for the type flags beyond the four benchmarked ones that also run
on the matrix pipe: f32f32f32, and f16f16f16 / bf16bf16bf16 when the caller
skips intermediate roundings (mmt4d_tile_generic.c:229-286, 319-376). Without
that flag the reference rounds after every multiply-add, which only the generic
kernel reproduces; the tests assert which kernel ran.

Tolerances. f32 output: |got - ref| <= 1e-3 * max(|ref|, rms(ref)), ref being
the reference's sequential accumulation. 16-bit outputs: the f32 sums agree to
that tolerance and are then rounded once, so got and ref may differ by one unit
in the last place of the output type (2^-10 relative for f16, 2^-7 for bf16);
the bound used is 1e-3 * max(|ref|, rms) + one such unit.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, synth
from test_gpu_configs import REL_TOL, assert_float_close, gpu_lib, mm_params  # noqa: F401

pytestmark = pytest.mark.gpu


def _oracle(oracle_lib, lhs, rhs, init, M, N, K, M0, N0, K0, flags):
    want = init.copy()
    p = mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, M, N, K, M0, N0, K0,
                  flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK)
    oracle_lib.oracle_mmt4d_mt(C.byref(p), 16)
    return want


@pytest.mark.parametrize("M0,N0,K0", [(16, 16, 4), (8, 8, 1), (16, 16, 1), (8, 16, 16)])
@pytest.mark.parametrize("acc", [0, abi.MMT4D_ACCUMULATE])
def test_f32f32f32_random_data(gpu_lib, oracle_lib, M0, N0, K0, acc):
    M, N = 320 // M0, 448 // N0
    K = 512 // K0
    flags = abi.MMT4D_TYPE_F32F32F32 | acc
    lhs = synth.normal_f32(21, 0, M * K * M0 * K0, 1.0)
    rhs = synth.normal_f32(21, 1, N * K * N0 * K0, 1.0)
    init = synth.normal_f32(21, 2, M * N * M0 * N0, 1.0)
    want = _oracle(oracle_lib, lhs, rhs, init, M, N, K, M0, N0, K0, flags)
    d_l, d_r, d_o = (torch.from_numpy(x).cuda() for x in (lhs, rhs, init.copy()))
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    assert_float_close(d_o.cpu().numpy(), want, "f32 %dx%dx%d" % (M0, N0, K0))


def test_f32f32f32_exact_on_small_integer_data_and_ragged_k(gpu_lib, oracle_lib):
    # Small integers: every partial sum is exact, any order gives the same bits.
    # K = 37 steps of K0 = 1 does not end on a 64-byte chunk: the staged kernel's
    # zero-filling tail runs.
    rng = np.random.default_rng(5)
    for (M, N, K, M0, N0, K0) in [(20, 24, 64, 8, 8, 4), (9, 11, 37, 8, 8, 1), (5, 7, 3, 16, 16, 4)]:
        lhs = rng.integers(-8, 8, size=M * K * M0 * K0).astype(np.float32)
        rhs = rng.integers(-8, 8, size=N * K * N0 * K0).astype(np.float32)
        init = rng.integers(-50, 50, size=M * N * M0 * N0).astype(np.float32)
        flags = abi.MMT4D_TYPE_F32F32F32 | abi.MMT4D_ACCUMULATE
        want = _oracle(oracle_lib, lhs, rhs, init, M, N, K, M0, N0, K0, flags)
        d_l, d_r, d_o = (torch.from_numpy(x).cuda() for x in (lhs, rhs, init.copy()))
        gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)))
        assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
        assert np.array_equal(d_o.cpu().numpy().view(np.uint32), want.view(np.uint32)), (M, N, K, M0, N0, K0)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("acc", [0, abi.MMT4D_ACCUMULATE])
def test_16bit_outputs_with_skipped_roundings(gpu_lib, oracle_lib, kind, acc):
    M, N, K, M0, N0, K0 = 20, 28, 32, 16, 16, 16
    base = abi.MMT4D_TYPE_F16F16F16 if kind == "f16" else abi.MMT4D_TYPE_BF16BF16BF16
    to_bits = synth.f16_bits if kind == "f16" else synth.bf16_bits
    widen = oracle_lib.oracle_f16_to_f32 if kind == "f16" else oracle_lib.oracle_bf16_to_f32
    ulp = 2.0 ** -10 if kind == "f16" else 2.0 ** -7
    lhs = to_bits(synth.normal_f32(22, 0, M * K * M0 * K0, 1.0 / 16))
    rhs = to_bits(synth.normal_f32(22, 1, N * K * N0 * K0, 1.0 / 16))
    init = to_bits(synth.normal_f32(22, 2, M * N * M0 * N0, 1.0))

    def to_f32(bits):
        return np.array([widen(int(b)) for b in bits[:4096]], dtype=np.float32)

    # With the flag: matrix pipe, one rounding at the end.
    flags = base | acc | abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
    want = _oracle(oracle_lib, lhs, rhs, init, M, N, K, M0, N0, K0, flags)
    d_l, d_r, d_o = (torch.from_numpy(x.view(np.int16)).cuda() for x in (lhs, rhs, init.copy()))
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    got = d_o.cpu().numpy().view(np.uint16)
    # Most elements agree bit for bit; all of them within one unit in the last place.
    assert np.mean(got == want) > 0.9
    g, w = to_f32(got), to_f32(want)
    rms = float(np.sqrt(np.mean(w.astype(np.float64) ** 2)))
    bound = (REL_TOL + ulp) * np.maximum(np.abs(w), rms)
    assert np.all(np.abs(g - w) <= bound)

    # Without it: the generic kernel, bit-identical to the reference's
    # round-after-every-step arithmetic.
    flags = base | acc
    want = _oracle(oracle_lib, lhs, rhs, init, M, N, K, M0, N0, K0, flags)
    d_o = torch.from_numpy(init.copy().view(np.int16)).cuda()
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_generic"
    assert np.array_equal(d_o.cpu().numpy().view(np.uint16), want)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_16bit_outputs_exact_on_small_integer_data(gpu_lib, oracle_lib, kind):
    # Sums of small integers that stay representable in the 16-bit output: the
    # single final rounding is exact, so the result must match bit for bit.
    M, N, K, M0, N0, K0 = 6, 10, 8, 16, 16, 8
    base = abi.MMT4D_TYPE_F16F16F16 if kind == "f16" else abi.MMT4D_TYPE_BF16BF16BF16
    to_bits = synth.f16_bits if kind == "f16" else synth.bf16_bits
    rng = np.random.default_rng(9)
    lhs = to_bits(rng.integers(-1, 2, size=M * K * M0 * K0).astype(np.float32))
    rhs = to_bits(rng.integers(-1, 2, size=N * K * N0 * K0).astype(np.float32))
    init = to_bits(rng.integers(-8, 8, size=M * N * M0 * N0).astype(np.float32))
    flags = base | abi.MMT4D_ACCUMULATE | abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
    want = _oracle(oracle_lib, lhs, rhs, init, M, N, K, M0, N0, K0, flags)
    d_l, d_r, d_o = (torch.from_numpy(x.view(np.int16)).cuda() for x in (lhs, rhs, init.copy()))
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    assert np.array_equal(d_o.cpu().numpy().view(np.uint16), want)


def test_f32f32f32_4096_cubed_against_fp64_row_sample(gpu_lib):
    # Full-size f32 problem with the tile shape query_tile_sizes hands out
    # (16x16x4): sampled output rows against a float64 product of the same
    # operands, plus the column checksum of the whole output.
    M = N = 256
    K, M0, N0, K0 = 1024, 16, 16, 4
    g = torch.Generator(device="cuda").manual_seed(3)
    d_l = torch.randn(M * K * M0 * K0, device="cuda", generator=g)
    d_r = torch.randn(N * K * N0 * K0, device="cuda", generator=g)
    d_o = torch.empty(M * N * M0 * N0, device="cuda")
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0,
                                              abi.MMT4D_TYPE_F32F32F32)))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_mfma_256x256"
    a = d_l.view(M, K, M0, K0).permute(0, 2, 1, 3).reshape(M * M0, K * K0)
    b = d_r.view(N, K, N0, K0).permute(0, 2, 1, 3).reshape(N * N0, K * K0)
    out = d_o.view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0)
    rows = [0, 1, 777, 2048, 4095]
    ref = a[rows].double() @ b.double().t()
    rms = ref.pow(2).mean().sqrt()
    assert bool(((out[rows].double() - ref).abs() <= REL_TOL * torch.maximum(ref.abs(), rms)).all())
    # sum over rows of the output == (sum over rows of a) . b^T
    col_ref = a.double().sum(dim=0) @ b.double().t()
    col_got = out.double().sum(dim=0)
    assert bool(((col_got - col_ref).abs() <= 1e-3 * col_ref.abs().max()).all())


def _operand_values(kind, count, seed):
    """`count` finite, normal, nonzero 16-bit floats (as bit patterns) whose pairwise products cover what the final
    rounding distinguishes: every result exponent from far below the output's range to overflow, exact ties (a
    mantissa of 1.5 against odd multiples of the last place), values one place either side of a tie, all-ones
    mantissas that carry into the exponent, both signs."""
    ebits, mbits = (5, 10) if kind == "f16" else (8, 7)
    bias = (1 << (ebits - 1)) - 1
    rng = np.random.default_rng(seed)
    mantissas = [0, 1 << (mbits - 1), (1 << mbits) - 1, 1, 3, (1 << (mbits - 1)) + 1, (1 << mbits) - 2]
    out = []
    for n in range(count):
        # Exponent fields of normal numbers only. f16: all 30 of them; bf16: every other one, odd ones in one
        # operand and even ones in the other, so that the products run from far below f32's range to beyond it.
        e = 1 + (n * 7 + seed) % 30 if kind == "f16" else seed + 2 * (n % 127)
        m = mantissas[n % len(mantissas)] if n % 3 else int(rng.integers(0, 1 << mbits))
        sign = (n >> 2) & 1
        out.append((sign << 15) | (e << mbits) | m)
    assert bias > 0
    return np.array(out, dtype=np.uint16)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("K0", [16, 1])
def test_16bit_output_rounding_matches_the_reference_on_every_exponent_and_on_ties(gpu_lib, oracle_lib, kind, K0):
    # One product per output element (K = 1, the other K0 - 1 positions hold +0 in the lhs), so the f32 value that is
    # rounded is exact and identical on both sides and the comparison pins the rounding itself (common.h:701-770),
    # bit for bit: results below the output's exponent range (zero), in the lowest in-range exponent (exponent
    # field 0 with mantissa bits), ties to even, carries into the exponent and to infinity, f16 products beyond 65504.
    M, N, K, M0, N0 = 8, 8, 1, 16, 16
    base = abi.MMT4D_TYPE_F16F16F16 if kind == "f16" else abi.MMT4D_TYPE_BF16BF16BF16
    a = _operand_values(kind, M * M0, 1)
    b = _operand_values(kind, N * N0, 2)
    lhs = np.zeros((M, K, M0, K0), np.uint16)
    rhs = np.full((N, K, N0, K0), 0x3C00 if kind == "f16" else 0x3F80, np.uint16)   # 1.0 in the unused positions
    lhs[:, 0, :, 0] = a.reshape(M, M0)
    rhs[:, 0, :, 0] = b.reshape(N, N0)
    lhs, rhs = lhs.reshape(-1), rhs.reshape(-1)
    init = np.zeros(M * N * M0 * N0, np.uint16)
    flags = base | abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
    want = _oracle(oracle_lib, lhs, rhs, init, M, N, K, M0, N0, K0, flags)
    d_l, d_r, d_o = (torch.from_numpy(x.view(np.int16)).cuda() for x in (lhs, rhs, init.copy()))
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)))
    kernel = gpu_lib.iree_uk_mi355x_last_kernel()
    assert b"generic" not in kernel
    got = d_o.cpu().numpy().view(np.uint16)
    # The cases the test is for are all present in what the reference produced.
    emask = 0x7C00 if kind == "f16" else 0x7F80
    field = want & emask
    assert np.any((want & 0x7FFF) == 0) and np.any(field == emask)
    if kind == "f16":   # (bf16 has f32's exponent range: below it there are only f32 subnormals, which give zero)
        assert np.any((field == 0) & ((want & 0x7FFF) != 0))
    assert len(np.unique(field)) >= (30 if kind == "f16" else 120)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (kernel, [(hex(int(got[i])), hex(int(want[i]))) for i in bad[:8]])
