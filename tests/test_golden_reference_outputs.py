"""tests/golden/reference_outputs.json holds what the reference's own compiled
ukernels produced (in a container that has the reference tree; script
tests/golden/make_golden.py) for the seeded inputs of the benchmark
configurations: a BLAKE2b-128 digest of the whole output and 1024 sampled
values each. Here the oracle (no GPU needed) and the GPU library are held
against those: integer outputs bit for bit over the WHOLE output, at full size,
the f16 configuration within the stated tolerance on the samples.
"""
import ctypes as C
import hashlib
import json
import os

import numpy as np
import pytest

from iree_amd import abi, synth

GOLDEN = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_outputs.json")))
REL_TOL = 1e-3


def digest(a):
    return hashlib.blake2b(np.ascontiguousarray(a).tobytes(), digest_size=16).hexdigest()


def params(lhs, rhs, out, M, N, K, M0, N0, K0, flags):
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs, rhs, out
    p.lhs_stride0, p.rhs_stride0, p.out_stride0 = K * M0 * K0, K * N0 * K0, N * M0 * N0
    p.M, p.N, p.K, p.M0, p.N0, p.K0, p.flags = M, N, K, M0, N0, K0, flags
    return p


def config1_inputs():
    M = N = 128
    K = 256
    return M, N, K, synth.uniform_int8(0, 0, M * K * 32), synth.uniform_int8(0, 1, N * K * 32)


def config5_inputs():
    Ms, N, K = 4, 688, 128
    lhs = synth.uniform_int8(5, 0, 512 * 4096)[:Ms * K * 16 * 32]
    return Ms, N, K, lhs, synth.uniform_int4_packed(5, 1, 11008 * 4096)


def config3_inputs():
    M = N = K = 256
    return (M, N, K, synth.f16_bits(synth.normal_f32(3, 0, M * K * 256, 1.0 / 64)),
            synth.f16_bits(synth.normal_f32(3, 1, N * K * 256, 1.0 / 64)), synth.normal_f32(3, 2, M * N * 256, 1.0))


# ---------------------------------------------------------------------------
# the oracle against the reference's outputs (CPU)
# ---------------------------------------------------------------------------

def test_oracle_reproduces_config1_bit_for_bit(oracle_lib):
    M, N, K, lhs, rhs = config1_inputs()
    out = np.zeros(M * N * 64, dtype=np.int32)
    oracle_lib.oracle_mmt4d_mt(C.byref(params(lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data, M, N, K, 8, 8, 4,
                                              abi.MMT4D_TYPE_S8S8S32)), 8)
    g = GOLDEN["s8s8s32_1024_8x8x4"]
    assert digest(out) == g["digest_of_tiled_output"]
    assert out[np.array(g["sample_index"])].tolist() == g["sample_value"]


def test_oracle_reproduces_int4_rows_bit_for_bit(oracle_lib):
    Ms, N, K, lhs, rhs = config5_inputs()
    out = np.zeros(Ms * N * 256, dtype=np.int32)
    oracle_lib.oracle_mmt4d_mt(C.byref(params(lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data, Ms, N, K, 16, 16, 32,
                                              abi.MMT4D_TYPE_S8S4S32)), 8)
    assert digest(out) == GOLDEN["s8s4s32_512x11008x4096_rows_0_63"]["digest_of_tiled_output"]


def test_oracle_reproduces_f16_samples_bit_for_bit(oracle_lib):
    M, N, K, lhs, rhs, init = config3_inputs()
    g = GOLDEN["f16f16f32_4096_16x16x16_accumulate"]
    row = g["rows_of_tiles"][0]
    out = init[row * N * 256:(row + 1) * N * 256].copy()
    oracle_lib.oracle_mmt4d_mt(C.byref(params(lhs[row * K * 256:].ctypes.data, rhs.ctypes.data, out.ctypes.data, 1, N, K, 16, 16, 16,
                                              abi.MMT4D_TYPE_F16F16F32 | abi.MMT4D_ACCUMULATE)), 8)
    want = np.array(g["sample_value"][0], dtype=np.float32)
    assert np.array_equal(out[np.array(g["sample_index"][0])].view(np.uint32), want.view(np.uint32))


PACK_VARIANTS = [("tiles16x1", 0, 512, 8190), ("transpose_inner", abi.PACK_TRANSPOSE_INNER, 8191, 512),
                 ("rhs_form", abi.PACK_TRANSPOSE_INNER | abi.PACK_TRANSPOSE_OUTER, 512, 8191)]


def pack_params(src, dst, flags, o0, o1):
    p = abi.PackParams()
    p.in_buffer, p.out_buffer = src, dst
    p.in_stride0, p.in_stride1, p.out_stride0, p.out_stride1 = 8190, 1, o1 * 16, 16
    p.in_size0, p.in_size1 = 8191, 8190
    p.out_size0, p.out_size1, p.out_size2, p.out_size3 = o0, o1, 16, 1
    p.padding_value, p.flags = 0, abi.PACK_TYPE_F32F32 | flags
    return p


def unpack_params(src, dst):
    u = abi.UnpackParams()
    u.in_buffer, u.out_buffer = src, dst
    u.in_stride0, u.in_stride1, u.out_stride0, u.out_stride1 = 8190 * 16, 16, 8190, 1
    u.in_size0, u.in_size1, u.in_size2, u.in_size3 = 512, 8190, 16, 1
    u.out_size0, u.out_size1, u.flags = 8191, 8190, abi.UNPACK_TYPE_F32F32
    return u


@pytest.mark.parametrize("name,flags,o0,o1", PACK_VARIANTS)
def test_oracle_reproduces_pack_bit_for_bit(oracle_lib, name, flags, o0, o1):
    g = GOLDEN["pack_unpack_f32_8191x8190"]
    src = synth.normal_f32(2, 0, 8191 * 8190)
    assert digest(src) == g["source"]   # the generator gives the same input everywhere
    packed = np.empty(o0 * o1 * 16, dtype=np.float32)
    oracle_lib.oracle_pack(C.byref(pack_params(src.ctypes.data, packed.ctypes.data, flags, o0, o1)))
    assert digest(packed) == g["pack_" + name]
    if name == "tiles16x1":
        back = np.full(8191 * 8190, -1.0, dtype=np.float32)
        oracle_lib.oracle_unpack(C.byref(unpack_params(packed.ctypes.data, back.ctypes.data)))
        assert digest(back) == g["unpack_tiles16x1"] == g["source"]


# ---------------------------------------------------------------------------
# the GPU library against the reference's outputs
# ---------------------------------------------------------------------------

@pytest.fixture(scope="module")
def gpu():
    import torch
    from iree_amd import library
    assert torch.cuda.is_available()
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    return lib, torch


@pytest.mark.gpu
def test_gpu_config1_whole_output(gpu):
    lib, torch = gpu
    M, N, K, lhs, rhs = config1_inputs()
    d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
    d_o = torch.empty(M * N * 64, dtype=torch.int32, device="cuda")
    lib.iree_uk_mmt4d_p(C.byref(params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, 8, 8, 4, abi.MMT4D_TYPE_S8S8S32)))
    assert lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    assert digest(d_o.cpu().numpy()) == GOLDEN["s8s8s32_1024_8x8x4"]["digest_of_tiled_output"]


@pytest.mark.gpu
def test_gpu_headline_4096_cubed_whole_output(gpu):
    lib, torch = gpu
    M = N = 512
    K = 1024
    d_l = torch.from_numpy(synth.uniform_int8(0, 0, M * K * 32)).cuda()
    d_r = torch.from_numpy(synth.uniform_int8(0, 1, N * K * 32)).cuda()
    d_o = torch.empty(M * N * 64, dtype=torch.int32, device="cuda")
    lib.iree_uk_mmt4d_p(C.byref(params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, 8, 8, 4, abi.MMT4D_TYPE_S8S8S32)))
    assert lib.iree_uk_mi355x_last_kernel() == b"mmt4d_mfma_256x256"
    # [512][512][8][8] tiles -> row-major logical 4096 x 4096, the order the digest was taken in
    logical = d_o.view(M, N, 8, 8).permute(0, 2, 1, 3).contiguous().cpu().numpy()
    g = GOLDEN["s8s8s32_4096_logical"]
    assert digest(logical) == g["digest_of_row_major_logical_output"]
    assert logical.reshape(-1)[np.array(g["sample_index"])].tolist() == g["sample_value"]


@pytest.mark.gpu
def test_gpu_int4_rows_whole_output(gpu):
    lib, torch = gpu
    Ms, N, K, lhs, rhs = config5_inputs()
    # the full 32-row-tile problem (so that the benchmark's kernel variant runs), compared on its first 4 rows of tiles
    full_lhs = synth.uniform_int8(5, 0, 512 * 4096)
    d_l, d_r = torch.from_numpy(full_lhs).cuda(), torch.from_numpy(rhs.view(np.int8)).cuda()
    d_o = torch.empty(32 * N * 256, dtype=torch.int32, device="cuda")
    lib.iree_uk_mmt4d_p(C.byref(params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), 32, N, K, 16, 16, 32, abi.MMT4D_TYPE_S8S4S32)))
    assert lib.iree_uk_mi355x_last_kernel().startswith(b"mmt4d_mfma")
    assert digest(d_o[:Ms * N * 256].cpu().numpy()) == GOLDEN["s8s4s32_512x11008x4096_rows_0_63"]["digest_of_tiled_output"]


@pytest.mark.gpu
def test_gpu_f16_accumulate_samples_within_tolerance(gpu):
    lib, torch = gpu
    M, N, K, lhs, rhs, init = config3_inputs()
    d_l = torch.from_numpy(lhs.view(np.int16)).cuda()
    d_r = torch.from_numpy(rhs.view(np.int16)).cuda()
    d_o = torch.from_numpy(init).cuda()
    lib.iree_uk_mmt4d_p(C.byref(params(d_l.data_ptr(), d_r.data_ptr(), d_o.data_ptr(), M, N, K, 16, 16, 16,
                                       abi.MMT4D_TYPE_F16F16F32 | abi.MMT4D_ACCUMULATE)))
    got = d_o.cpu().numpy()
    g = GOLDEN["f16f16f32_4096_16x16x16_accumulate"]
    for row, idx, val in zip(g["rows_of_tiles"], g["sample_index"], g["sample_value"]):
        ref = np.array(val, dtype=np.float32)
        have = got[row * N * 256:(row + 1) * N * 256][np.array(idx)]
        rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        assert np.all(np.abs(have - ref) <= REL_TOL * np.maximum(np.abs(ref), rms)), row


@pytest.mark.gpu
@pytest.mark.parametrize("name,flags,o0,o1", PACK_VARIANTS)
def test_gpu_pack_unpack_whole_output(gpu, name, flags, o0, o1):
    lib, torch = gpu
    g = GOLDEN["pack_unpack_f32_8191x8190"]
    d_src = torch.from_numpy(synth.normal_f32(2, 0, 8191 * 8190)).cuda()
    d_packed = torch.full((o0 * o1 * 16,), float("nan"), dtype=torch.float32, device="cuda")
    lib.iree_uk_pack_p(C.byref(pack_params(d_src.data_ptr(), d_packed.data_ptr(), flags, o0, o1)))
    assert lib.iree_uk_mi355x_last_kernel() == b"pack_tiled"
    assert digest(d_packed.cpu().numpy()) == g["pack_" + name]
    if name == "tiles16x1":
        d_back = torch.full((8191 * 8190,), -1.0, dtype=torch.float32, device="cuda")
        lib.iree_uk_unpack_p(C.byref(unpack_params(d_packed.data_ptr(), d_back.data_ptr())))
        assert lib.iree_uk_mi355x_last_kernel() == b"unpack_tiled"
        assert digest(d_back.cpu().numpy()) == g["unpack_tiles16x1"]
