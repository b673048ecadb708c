"""Two places where the GPU library's semantics could drift from the reference's
and what pins them:

* operand strides the reference accepts without comment (mmt4d.c:12-48 checks
  none): a zero lhs or rhs stride broadcasts one panel, a short one overlaps
  panels; results must equal the oracle's, which follows the reference's
  addressing literally (mmt4d.c:70-83);
* f16 subnormal inputs: the reference's generic tile function widens them to
  zero (common.h:685-686), the matrix pipe multiplies them as they are. The
  difference is bounded per output element by the sum of |a*b| over the terms
  with a subnormal factor; the test makes a quarter of the lhs subnormal and
  checks that bound, and that the GPU result is the unflushed product.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, library, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu_lib():
    assert torch.cuda.is_available()
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    return lib


def _params(lhs, rhs, out, M, N, K, M0, N0, K0, flags, lhs_stride, rhs_stride):
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs, rhs, out
    p.lhs_stride0, p.rhs_stride0, p.out_stride0 = lhs_stride, rhs_stride, N * M0 * N0
    p.M, p.N, p.K, p.M0, p.N0, p.K0, p.flags = M, N, K, M0, N0, K0, flags
    return p


@pytest.mark.parametrize("M0,N0,K0,K,lhs_stride,rhs_stride", [
    (8, 8, 4, 64, 0, None),            # every lhs tile row is the same panel
    (8, 8, 4, 64, None, 0),            # every rhs panel is the same
    (16, 16, 64, 6, 16 * 64, None),    # lhs panels one k step apart: they overlap
    (16, 16, 16, 5, None, 16 * 16),    # f16-sized tiles on int8: rhs overlap
])
@pytest.mark.parametrize("device_operands", [True, False])
def test_zero_and_overlapping_operand_strides(gpu_lib, oracle_lib, M0, N0, K0, K, lhs_stride, rhs_stride,
                                              device_operands):
    M, N = 20, 12
    flags = abi.MMT4D_TYPE_S8S8S32
    ls = K * M0 * K0 if lhs_stride is None else lhs_stride
    rs = K * N0 * K0 if rhs_stride is None else rhs_stride
    lhs = synth.uniform_int8(31, 0, (M - 1) * ls + K * M0 * K0)
    rhs = synth.uniform_int8(31, 1, (N - 1) * rs + K * N0 * K0)
    want = np.zeros(M * N * M0 * N0, np.int32)
    oracle_lib.oracle_mmt4d(C.byref(_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, M, N, K, M0, N0, K0,
                                            flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK, ls, rs)))
    if device_operands:
        d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
        d_o = torch.full((want.size,), -1, dtype=torch.int32, device="cuda")
        gpu_lib.iree_uk_mmt4d_p(C.byref(_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0,
                                                flags, ls, rs)))
        got = d_o.cpu().numpy()
    else:
        got = np.full(want.size, -1, np.int32)
        gpu_lib.iree_uk_mmt4d_p(C.byref(_params(lhs.ctypes.data, rhs.ctypes.data, got.ctypes.data, M, N, K, M0, N0, K0,
                                                flags, ls, rs)))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    assert np.array_equal(got, want)


def test_f16_subnormal_inputs_deviate_from_the_flushing_reference_by_at_most_their_products(gpu_lib, oracle_lib):
    M, N, K, M0, N0, K0 = 8, 8, 32, 16, 16, 16      # logical 128 x 128 x 512
    flags = abi.MMT4D_TYPE_F16F16F32
    n_l, n_r = M * K * M0 * K0, N * K * N0 * K0
    lhs_f = synth.normal_f32(41, 0, n_l, 1.0)
    # A quarter of the lhs becomes f16 subnormal (|x| < 2^-14), sign kept, spread over the subnormal range.
    pick = (synth.bits64(41, 3, n_l) & np.uint64(3)) == 0
    lhs_f[pick] = np.sign(lhs_f[pick]) * (np.abs(lhs_f[pick]) % 1.0) * np.float32(2.0 ** -14)
    lhs = synth.f16_bits(lhs_f)
    rhs = synth.f16_bits(synth.normal_f32(41, 1, n_r, 1.0))
    lhs_h, rhs_h = lhs.view(np.float16), rhs.view(np.float16)
    sub_l = (np.abs(lhs_h) < np.float16(2.0 ** -14)) & (lhs_h != 0)
    assert 0.2 < sub_l.mean() < 0.3

    flushed = np.zeros(M * N * M0 * N0, np.float32)
    oracle_lib.oracle_mmt4d(C.byref(_params(lhs.ctypes.data, rhs.ctypes.data, flushed.ctypes.data, M, N, K, M0, N0, K0,
                                            flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK, K * M0 * K0, K * N0 * K0)))
    d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
    d_o = torch.zeros(flushed.size, dtype=torch.float32, device="cuda")
    gpu_lib.iree_uk_mmt4d_p(C.byref(_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags,
                                            K * M0 * K0, K * N0 * K0)))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    got = d_o.cpu().numpy().reshape(M, N, M0, N0).transpose(0, 2, 1, 3).reshape(M * M0, N * N0)
    flushed = flushed.reshape(M, N, M0, N0).transpose(0, 2, 1, 3).reshape(M * M0, N * N0)

    # Row-major logical operands in float64.
    a = lhs_h.astype(np.float64).reshape(M, K, M0, K0).transpose(0, 2, 1, 3).reshape(M * M0, K * K0)
    b = rhs_h.astype(np.float64).reshape(N, K, N0, K0).transpose(0, 2, 1, 3).reshape(N * N0, K * K0)
    a_sub = np.where(sub_l.reshape(M, K, M0, K0).transpose(0, 2, 1, 3).reshape(M * M0, K * K0), np.abs(a), 0.0)
    exact = a @ b.T                       # nothing flushed
    bound = a_sub @ np.abs(b).T           # sum of |a*b| over the terms the reference drops
    assert bound.max() > 0
    rms = float(np.sqrt(np.mean(exact ** 2)))
    tol = 1e-3 * np.maximum(np.abs(exact), rms)
    # The matrix pipe computes the unflushed product ...
    assert np.all(np.abs(got - exact) <= tol)
    # ... which is within the dropped terms (plus rounding) of the reference's,
    assert np.all(np.abs(got - flushed) <= bound + 1e-5 * rms)
    # ... and on this data that is far inside the tolerance stated for the float kernels.
    assert np.all(np.abs(got - flushed) <= tol)


@pytest.mark.parametrize("M,N,M0", [(2, 3, 16), (1, 40, 1)])
def test_int4_products_deeper_than_the_scaled_accumulators_hold(gpu_lib, oracle_lib, M, N, M0):
    # The int4 kernels keep 16x the sums in int32, good for a total depth below
    # 131072; a deeper product is chained over slices of K. Worst-case operands
    # (-128 x -8 everywhere) so that an overflow of a slice would show.
    N0, K0, K = 16, 32, 4100                      # depth 131200
    flags = abi.MMT4D_TYPE_S8S4S32
    lhs = synth.uniform_int8(51, 0, M * K * M0 * K0)
    rhs = synth.uniform_int4_packed(51, 1, N * K * N0 * K0)
    lhs[:K * M0 * K0] = -128                      # first lhs tile row: extreme values
    rhs[:K * N0 * K0 // 2] = 0x88                 # first rhs panel: -8 in every nibble
    init = (synth.bits64(51, 2, M * N * M0 * N0) & np.uint64(0xFFFF)).astype(np.int32)
    for accumulate in (0, abi.MMT4D_ACCUMULATE):
        want = init.copy()
        oracle_lib.oracle_mmt4d_mt(C.byref(_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, M, N, K, M0, N0,
                                                   K0, flags | accumulate | abi.MMT4D_ALLOW_GENERIC_FALLBACK,
                                                   K * M0 * K0, K * N0 * K0)), 8)
        d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
        d_o = torch.from_numpy(init).cuda()
        gpu_lib.iree_uk_mmt4d_p(C.byref(_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0,
                                                flags | accumulate, K * M0 * K0, K * N0 * K0)))
        assert b"generic" not in gpu_lib.iree_uk_mi355x_last_kernel()
        assert np.array_equal(d_o.cpu().numpy(), want), (M, N, accumulate)
    assert want[0] == init[0] + 131200 * 1024    # (-128) * (-8) * depth on top of the initial value
