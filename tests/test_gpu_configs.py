"""GPU parity at the sizes of the benchmark configurations, device buffers,
through the C ABI.

Where the scalar oracle finishes in seconds the whole output is compared; for
the 4096-cubed problems a sample of whole tile rows is compared with the oracle
and the full output is pinned through size-independent properties (row and
column checksums computed without any matmul, pack/unpack round trips).
Integer and pack/unpack results must be bit-exact. Float tolerance, as stated
for these kernels: |got - ref| <= 1e-3 * max(|ref|, rms(ref)) per element, ref
being the reference's sequential f32 accumulation.
"""
import ctypes as C
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest
import torch

from iree_amd import abi, library, synth

pytestmark = pytest.mark.gpu
REL_TOL = 1e-3


@pytest.fixture(scope="module")
def gpu_lib():
    assert torch.cuda.is_available()
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    return lib


def mm_params(lhs, rhs, out, M, N, K, M0, N0, K0, flags, lhs_off=0, rhs_off=0, out_off=0,
              lhs_stride=None, rhs_stride=None, out_stride=None):
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs, rhs, out
    p.lhs_offset, p.rhs_offset, p.out_offset = lhs_off, rhs_off, out_off
    p.lhs_stride0 = K * M0 * K0 if lhs_stride is None else lhs_stride
    p.rhs_stride0 = K * N0 * K0 if rhs_stride is None else rhs_stride
    p.out_stride0 = N * M0 * N0 if out_stride is None else out_stride
    p.M, p.N, p.K, p.M0, p.N0, p.K0, p.flags = M, N, K, M0, N0, K0, flags
    return p


def oracle_tile_rows(oracle_lib, rows, lhs, rhs, out_init, M, N, K, M0, N0, K0, flags, threads=16):
    """Oracle output for the given rows of lhs tiles; the rhs panels of each row
    are split over `threads` host threads. Returns {row: array [N*M0*N0]}."""
    lb, rb, ob = abi.MMT4D_BITS[flags & 0xFF]
    out_dtype = np.int32 if abi.MMT4D_NAMES[flags & 0xFF].startswith("s") else np.float32
    results = {i: np.array(out_init[i * N * M0 * N0:(i + 1) * N * M0 * N0], dtype=out_dtype, copy=True)
               for i in rows}
    jobs = []
    for i in rows:
        step = max(1, -(-N // threads))
        for j0 in range(0, N, step):
            jobs.append((i, j0, min(step, N - j0)))

    def run(job):
        i, j0, n = job
        p = mm_params(lhs.ctypes.data, rhs.ctypes.data, results[i].ctypes.data, 1, n, K, M0, N0, K0,
                      flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK,
                      lhs_off=i * K * M0 * K0, rhs_off=j0 * K * N0 * K0, out_off=j0 * M0 * N0)
        oracle_lib.oracle_mmt4d(C.byref(p))

    with ThreadPoolExecutor(threads) as pool:
        list(pool.map(run, jobs))
    return results


def assert_float_close(got, ref, what):
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    bound = REL_TOL * np.maximum(np.abs(ref), rms)
    err = np.abs(got - ref)
    worst = int(np.argmax(err - bound))
    assert np.all(err <= bound), "%s: |err|=%g at %d exceeds %g (ref %g)" % (
        what, err[worst], worst, bound[worst], ref[worst])


# ---------------------------------------------------------------------------
# config 1 and the headline shape: s8s8s32, tiles 8x8x4
# ---------------------------------------------------------------------------

def test_s8s8s32_1024_cubed_bit_exact_vs_oracle(gpu_lib, oracle_lib):
    M = N = 128
    K, M0, N0, K0 = 256, 8, 8, 4
    lhs = synth.uniform_int8(0, 0, M * K * M0 * K0)
    rhs = synth.uniform_int8(0, 1, N * K * N0 * K0)
    want = np.zeros(M * N * M0 * N0, dtype=np.int32)
    p = mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, M, N, K, M0, N0, K0,
                  abi.MMT4D_TYPE_S8S8S32)
    oracle_lib.oracle_mmt4d_mt(C.byref(p), 16)
    d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
    d_o = torch.full((M * N * M0 * N0,), 12345, dtype=torch.int32, device="cuda")
    q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0,
                  abi.MMT4D_TYPE_S8S8S32)
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    assert np.array_equal(d_o.cpu().numpy(), want)
    # ACCUMULATE on top of the previous result doubles it.
    q.flags |= abi.MMT4D_ACCUMULATE
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert np.array_equal(d_o.cpu().numpy(), 2 * want)


def test_s8s8s32_4096_cubed_checksums_and_sampled_rows(gpu_lib, oracle_lib):
    M = N = 512
    K, M0, N0, K0 = 1024, 8, 8, 4
    lhs = synth.uniform_int8(0, 0, M * K * M0 * K0)
    rhs = synth.uniform_int8(0, 1, N * K * N0 * K0)
    d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
    d_o = torch.empty(M * N * M0 * N0, dtype=torch.int32, device="cuda")
    q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0,
                  abi.MMT4D_TYPE_S8S8S32)
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    # Row-major views: A [4096, 4096], B [4096, 4096], C [4096, 4096] (int64 math).
    a = d_l.view(M, K, M0, K0).permute(0, 2, 1, 3).reshape(M * M0, K * K0).to(torch.int64)
    b = d_r.view(N, K, N0, K0).permute(0, 2, 1, 3).reshape(N * N0, K * K0).to(torch.int64)
    c = d_o.view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0).to(torch.int64)
    # Row sums of C = A . (column sums of B^T); column sums likewise. A wrong or
    # misplaced element changes one of each.
    assert torch.equal(c.sum(dim=1), (a * b.sum(dim=0)[None, :]).sum(dim=1))
    assert torch.equal(c.sum(dim=0), (b * a.sum(dim=0)[None, :]).sum(dim=1))
    rows = [0, 255, 511]
    want = oracle_tile_rows(oracle_lib, rows, lhs, rhs, np.zeros(M * N * M0 * N0, np.int32),
                            M, N, K, M0, N0, K0, abi.MMT4D_TYPE_S8S8S32)
    got = d_o.cpu().numpy()
    for i in rows:
        assert np.array_equal(got[i * N * M0 * N0:(i + 1) * N * M0 * N0], want[i]), i


# ---------------------------------------------------------------------------
# config 3: f16f16f32 4096^3, tiles 16x16x16, accumulate on
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_f16_4096_cubed_accumulate_sampled_rows(gpu_lib, oracle_lib, kind):
    M = N = 256
    K, M0, N0, K0 = 256, 16, 16, 16
    flags = (abi.MMT4D_TYPE_F16F16F32 if kind == "f16" else abi.MMT4D_TYPE_BF16BF16F32) | abi.MMT4D_ACCUMULATE
    to_bits = synth.f16_bits if kind == "f16" else synth.bf16_bits
    lhs = to_bits(synth.normal_f32(3, 0, M * K * M0 * K0, 1.0 / 64))
    rhs = to_bits(synth.normal_f32(3, 1, N * K * N0 * K0, 1.0 / 64))
    init = synth.normal_f32(3, 2, M * N * M0 * N0, 1.0)
    d_l = torch.from_numpy(lhs.view(np.int16)).cuda()
    d_r = torch.from_numpy(rhs.view(np.int16)).cuda()
    d_o = torch.from_numpy(init).cuda()
    q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    got = d_o.cpu().numpy()
    rows = [0, 131]
    want = oracle_tile_rows(oracle_lib, rows, lhs, rhs, init, M, N, K, M0, N0, K0, flags)
    for i in rows:
        assert_float_close(got[i * N * M0 * N0:(i + 1) * N * M0 * N0], want[i], "%s row %d" % (kind, i))
    # Whole output against an independent fp32 matmul of the same operands
    # (looser: fp32 GEMM libraries do not accumulate sequentially).
    dt = torch.float16 if kind == "f16" else torch.bfloat16
    a = d_l.view(dt).view(M, K, M0, K0).permute(0, 2, 1, 3).reshape(M * M0, K * K0).float()
    b = d_r.view(dt).view(N, K, N0, K0).permute(0, 2, 1, 3).reshape(N * N0, K * K0).float()
    c0 = torch.from_numpy(init).cuda().view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0)
    ref = (c0 + a @ b.t()).view(M, M0, N, N0).permute(0, 2, 1, 3).reshape(-1)
    assert torch.allclose(d_o, ref, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("flags,M0,N0,K0", [
    (abi.MMT4D_TYPE_F16F16F32, 16, 16, 16), (abi.MMT4D_TYPE_BF16BF16F32, 16, 16, 8),
    (abi.MMT4D_TYPE_BF16BF16F32, 4, 16, 8), (abi.MMT4D_TYPE_F16F16F32, 8, 8, 8)])
def test_float_kernels_exact_on_small_integer_data(gpu_lib, oracle_lib, flags, M0, N0, K0):
    # With inputs that are small integers every partial sum is representable, so
    # any summation order gives the same bits (the reference's own tests rely on
    # this, tools/util.c:133-146): the MFMA kernels must match the oracle exactly.
    M, N, K = 24, 40, 48
    rng = np.random.default_rng(11)
    vals = rng.integers(-4, 4, size=M * K * M0 * K0).astype(np.float32)
    wts = rng.integers(-4, 4, size=N * K * N0 * K0).astype(np.float32)
    to_bits = synth.f16_bits if (flags & 0xFF) == abi.MMT4D_TYPE_F16F16F32 else synth.bf16_bits
    lhs, rhs = to_bits(vals), to_bits(wts)
    init = rng.integers(-100, 100, size=M * N * M0 * N0).astype(np.float32)
    for acc in (0, abi.MMT4D_ACCUMULATE):
        want = init.copy()
        p = mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, M, N, K, M0, N0, K0, flags | acc)
        oracle_lib.oracle_mmt4d_mt(C.byref(p), 8)
        d_l = torch.from_numpy(lhs.view(np.int16)).cuda()
        d_r = torch.from_numpy(rhs.view(np.int16)).cuda()
        d_o = torch.from_numpy(init.copy()).cuda()
        q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags | acc)
        gpu_lib.iree_uk_mmt4d_p(C.byref(q))
        assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
        assert np.array_equal(d_o.cpu().numpy().view(np.uint32), want.view(np.uint32))


# ---------------------------------------------------------------------------
# config 4: bf16 decode shapes, M0 in {1, 4, 16}, N = 14336, K = 4096
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("m0", [1, 4, 16])
def test_bf16_skinny_decode_shapes(gpu_lib, oracle_lib, m0):
    N, K, N0, K0 = 896, 512, 16, 8
    flags = abi.MMT4D_TYPE_BF16BF16F32
    lhs = synth.bf16_bits(synth.normal_f32(4, m0, m0 * K * K0, 1.0))
    rhs = synth.bf16_bits(synth.normal_f32(4, 10, N * K * N0 * K0, 0.02))
    init = np.zeros(N * m0 * N0, dtype=np.float32)
    want = oracle_tile_rows(oracle_lib, [0], lhs, rhs, init, 1, N, K, m0, N0, K0, flags)[0]
    d_l = torch.from_numpy(lhs.view(np.int16)).cuda()
    d_r = torch.from_numpy(rhs.view(np.int16)).cuda()
    d_o = torch.full((N * m0 * N0,), 7.0, dtype=torch.float32, device="cuda")
    q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), 1, N, K, m0, N0, K0, flags)
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == (b"mmt4d_gemv_resident_lhs" if m0 == 16 else b"mmt4d_gemv")
    assert_float_close(d_o.cpu().numpy(), want, "bf16 skinny M0=%d" % m0)
    # accumulate: out += product, starting from a known buffer
    start = synth.normal_f32(4, 99, N * m0 * N0, 1.0)
    d_o.copy_(torch.from_numpy(start))
    q.flags |= abi.MMT4D_ACCUMULATE
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert_float_close(d_o.cpu().numpy(), want + start, "bf16 skinny accumulate M0=%d" % m0)


def test_skinny_kernel_exact_on_small_integer_data_and_ragged_k(gpu_lib, oracle_lib):
    # K not a multiple of the 4 k-steps one MFMA consumes; N odd.
    rng = np.random.default_rng(5)
    for (m0, N, K) in [(1, 33, 7), (4, 17, 130), (16, 21, 9)]:
        lhs = synth.bf16_bits(rng.integers(-3, 4, size=m0 * K * 8).astype(np.float32))
        rhs = synth.bf16_bits(rng.integers(-3, 4, size=N * K * 128).astype(np.float32))
        want = np.zeros(N * m0 * 16, dtype=np.float32)
        p = mm_params(lhs.ctypes.data, rhs.ctypes.data, want.ctypes.data, 1, N, K, m0, 16, 8,
                      abi.MMT4D_TYPE_BF16BF16F32)
        oracle_lib.oracle_mmt4d(C.byref(p))
        d_l = torch.from_numpy(lhs.view(np.int16)).cuda()
        d_r = torch.from_numpy(rhs.view(np.int16)).cuda()
        d_o = torch.full((N * m0 * 16,), -1.0, dtype=torch.float32, device="cuda")
        q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), 1, N, K, m0, 16, 8,
                      abi.MMT4D_TYPE_BF16BF16F32)
        gpu_lib.iree_uk_mmt4d_p(C.byref(q))
        assert gpu_lib.iree_uk_mi355x_last_kernel() == b"mmt4d_gemv"
        assert np.array_equal(d_o.cpu().numpy(), want), (m0, N, K)


# ---------------------------------------------------------------------------
# config 5: s8s4s32, 512 x 11008 x 4096, tiles 16x16x32
# ---------------------------------------------------------------------------

def test_s8s4s32_quantized_weights(gpu_lib, oracle_lib):
    M, N, K, M0, N0, K0 = 32, 688, 128, 16, 16, 32
    flags = abi.MMT4D_TYPE_S8S4S32
    lhs = synth.uniform_int8(5, 0, M * K * M0 * K0)
    rhs = synth.uniform_int4_packed(5, 1, N * K * N0 * K0)
    d_l = torch.from_numpy(lhs).cuda()
    d_r = torch.from_numpy(rhs).cuda()
    d_o = torch.empty(M * N * M0 * N0, dtype=torch.int32, device="cuda")
    q = mm_params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, M0, N0, K0, flags)
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    got = d_o.cpu().numpy()
    # Full-size checksums with the nibbles widened by torch: element 2b is the
    # low nibble of byte b, two's complement (mmt4d_tile_generic.c:35-45).
    lo = (d_r.to(torch.int16) & 0xF)
    hi = (d_r.to(torch.int16) >> 4) & 0xF
    w = torch.stack([lo, hi], dim=1).reshape(-1)
    w = ((w ^ 8) - 8).to(torch.int64)
    a = d_l.view(M, K, M0, K0).permute(0, 2, 1, 3).reshape(M * M0, K * K0).to(torch.int64)
    b = w.view(N, K, N0, K0).permute(0, 2, 1, 3).reshape(N * N0, K * K0)
    c = d_o.view(M, N, M0, N0).permute(0, 2, 1, 3).reshape(M * M0, N * N0).to(torch.int64)
    assert torch.equal(c.sum(dim=1), (a * b.sum(dim=0)[None, :]).sum(dim=1))
    assert torch.equal(c.sum(dim=0), (b * a.sum(dim=0)[None, :]).sum(dim=1))
    rows = [0, 17, 31]
    # The oracle takes rhs offsets in 4-bit elements.
    want = oracle_tile_rows(oracle_lib, rows, lhs, rhs, np.zeros(M * N * M0 * N0, np.int32),
                            M, N, K, M0, N0, K0, flags)
    for i in rows:
        assert np.array_equal(got[i * N * M0 * N0:(i + 1) * N * M0 * N0], want[i]), i
    # accumulate on top
    q.flags |= abi.MMT4D_ACCUMULATE
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    assert np.array_equal(d_o.cpu().numpy(), 2 * got)


# ---------------------------------------------------------------------------
# config 2: pack / unpack f32 [8191, 8190] with non-divisible edges
# ---------------------------------------------------------------------------

def _pack_params(src, dst, rows, cols, o0, o1, t0, t1, flags, pad=0):
    p = abi.PackParams()
    p.in_buffer, p.out_buffer = src, dst
    p.in_stride0, p.in_stride1 = cols, 1
    p.out_stride0, p.out_stride1 = o1 * t0 * t1, t0 * t1
    p.in_size0, p.in_size1 = rows, cols
    p.out_size0, p.out_size1, p.out_size2, p.out_size3 = o0, o1, t0, t1
    p.padding_value = pad
    p.flags = abi.PACK_TYPE_F32F32 | flags
    return p


def _unpack_params(src, dst, rows, cols, o0, o1, t0, t1, flags):
    p = abi.UnpackParams()
    p.in_buffer, p.out_buffer = src, dst
    p.in_stride0, p.in_stride1 = o1 * t0 * t1, t0 * t1
    p.out_stride0, p.out_stride1 = cols, 1
    p.in_size0, p.in_size1, p.in_size2, p.in_size3 = o0, o1, t0, t1
    p.out_size0, p.out_size1 = rows, cols
    p.flags = abi.UNPACK_TYPE_F32F32 | flags
    return p


@pytest.mark.parametrize("name,flags,o0,o1", [
    ("tiles16x1", 0, 512, 8190),
    ("transpose_inner", abi.PACK_TRANSPOSE_INNER, 8191, 512),
    ("rhs_form", abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER, 512, 8191),
])
def test_pack_unpack_f32_8191x8190(gpu_lib, oracle_lib, name, flags, o0, o1):
    R, Cc, t0, t1 = 8191, 8190, 16, 1
    src = synth.normal_f32(2, 0, R * Cc)
    n_out = o0 * o1 * t0 * t1
    want = np.empty(n_out, dtype=np.float32)
    oracle_lib.oracle_pack(C.byref(_pack_params(src.ctypes.data, want.ctypes.data, R, Cc, o0, o1, t0, t1, flags)))
    d_src = torch.from_numpy(src).cuda()
    d_packed = torch.full((n_out,), float("nan"), dtype=torch.float32, device="cuda")
    gpu_lib.iree_uk_pack_p(C.byref(_pack_params(d_src.data_ptr(), d_packed.data_ptr(), R, Cc, o0, o1, t0, t1, flags)))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"pack_tiled"
    assert np.array_equal(d_packed.cpu().numpy().view(np.uint32), want.view(np.uint32)), name
    # The padding is there and is +0.0: total zero count >= padded element count.
    assert int((d_packed == 0).sum().item()) >= n_out - R * Cc
    # Unpack into a sentinel-filled buffer one row and one column larger than
    # the logical output: everything outside [R, Cc] must stay untouched.
    d_back = torch.full(((R + 1) * (Cc + 1),), -123.0, dtype=torch.float32, device="cuda")
    up = _unpack_params(d_packed.data_ptr(), d_back.data_ptr(), R, Cc, o0, o1, t0, t1, flags)
    up.out_stride0 = Cc + 1
    gpu_lib.iree_uk_unpack_p(C.byref(up))
    assert gpu_lib.iree_uk_mi355x_last_kernel() == b"unpack_tiled"
    back = d_back.view(R + 1, Cc + 1)
    assert torch.equal(back[:R, :Cc], d_src.view(R, Cc)), name
    assert bool((back[R, :] == -123.0).all()) and bool((back[:, Cc] == -123.0).all())


def test_pack_nonzero_padding_value_and_i8_operand_layouts(gpu_lib, oracle_lib):
    # i8 operands of the 8x8x4 mmt4d: lhs [M1, K1, 8, 4] and rhs packed with
    # both transposes (the form the reference's matmul benchmark uses,
    # tools/e2e_matmul_benchmark.c:238-254), ragged sizes, padding value 0x5A.
    R, Cc = 1021, 3001
    src = synth.uniform_int8(9, 0, R * Cc)
    for flags, o0, o1, t0, t1 in [(0, 128, 751, 8, 4),
                                  (abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER, 376, 256, 8, 4)]:
        n_out = o0 * o1 * t0 * t1
        want = np.empty(n_out, dtype=np.int8)
        p = _pack_params(src.ctypes.data, want.ctypes.data, R, Cc, o0, o1, t0, t1, flags, pad=0x115A)
        p.flags = abi.PACK_TYPE_I8I8 | flags
        oracle_lib.oracle_pack(C.byref(p))
        d_src = torch.from_numpy(src).cuda()
        d_out = torch.zeros(n_out, dtype=torch.int8, device="cuda")
        q = _pack_params(d_src.data_ptr(), d_out.data_ptr(), R, Cc, o0, o1, t0, t1, flags, pad=0x115A)
        q.flags = abi.PACK_TYPE_I8I8 | flags
        gpu_lib.iree_uk_pack_p(C.byref(q))
        assert gpu_lib.iree_uk_mi355x_last_kernel() == (b"pack_transposing" if flags else b"pack_tiled")
        assert np.array_equal(d_out.cpu().numpy(), want)


def test_end_to_end_pack_mmt4d_unpack_equals_row_major_matmul(gpu_lib):
    # pack(lhs); pack(rhs, both transposes); mmt4d; unpack == A @ B for a ragged
    # int8 problem (tools/e2e_matmul_benchmark.c:173-186, 340-358).
    Mr, Kr, Nr = 500, 1000, 300
    M0, N0, K0 = 8, 8, 4
    M1, K1, N1 = -(-Mr // M0), -(-Kr // K0), -(-Nr // N0)
    rng = np.random.default_rng(3)
    a = torch.from_numpy(rng.integers(-128, 128, size=(Mr, Kr), dtype=np.int8)).cuda()
    b = torch.from_numpy(rng.integers(-128, 128, size=(Kr, Nr), dtype=np.int8)).cuda()
    pa = torch.empty(M1 * K1 * M0 * K0, dtype=torch.int8, device="cuda")
    pb = torch.empty(N1 * K1 * N0 * K0, dtype=torch.int8, device="cuda")
    pc = torch.empty(M1 * N1 * M0 * N0, dtype=torch.int32, device="cuda")
    c = torch.empty(Mr * Nr, dtype=torch.int32, device="cuda")
    p = _pack_params(a.data_ptr(), pa.data_ptr(), Mr, Kr, M1, K1, M0, K0, 0)
    p.flags = abi.PACK_TYPE_I8I8
    gpu_lib.iree_uk_pack_p(C.byref(p))
    p = _pack_params(b.data_ptr(), pb.data_ptr(), Kr, Nr, N1, K1, N0, K0,
                     abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER)
    p.flags = abi.PACK_TYPE_I8I8 | abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER
    gpu_lib.iree_uk_pack_p(C.byref(p))
    q = mm_params(pa.data_ptr(), pb.data_ptr(), pc.data_ptr(), M1, N1, K1, M0, N0, K0, abi.MMT4D_TYPE_S8S8S32)
    gpu_lib.iree_uk_mmt4d_p(C.byref(q))
    u = _unpack_params(pc.data_ptr(), c.data_ptr(), Mr, Nr, M1, N1, M0, N0, 0)
    u.flags = abi.UNPACK_TYPE_I32I32
    gpu_lib.iree_uk_unpack_p(C.byref(u))
    # float64 holds these sums exactly (|sum| <= 1000 * 2^14 < 2^53).
    want = (a.double() @ b.double()).to(torch.int32)
    assert torch.equal(c.view(Mr, Nr), want)
