"""The in-dispatch int8 microkernel for gfx950
(iree_amd/csrc/device/iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8.c, built as
AMDGPU bitcode and linked into its host-callable wrapper's kernels) through
that wrapper: bit-exact against an integer matrix product of the
same operands, for every instantiated parameter combination (tiles staged in
workgroup memory or read straight from global memory, one or two MFMA K-steps
per outer step, staged tiles smaller than or not a multiple of the workgroup's
threads, as the reference's heuristics pick them for narrow M:
GPUEncodingExternalModels.cpp, subgroups 1 x 4), with accumulation into
existing values.

The data-tiled layouts are those of the reference's gfx942 counterpart
(compiler/plugins/target/ROCM/builtins/ukernel/
iree_uk_amdgpu_multi_mma_mfma_i32_16x16x32_i8.c:82-181) with 16-byte vectors:
lane l of an A/B vector block holds row l % 16, K bytes 16*(l // 16)..+15;
lane l of a C block holds rows 4*(l // 16)+{0..3} of column l % 16.
"""
import numpy as np
import pytest
import torch

from iree_amd import library

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    l = library.load()
    assert l.iree_uk_mi355x_init(0) == 0
    l.iree_uk_mi355x_set_stream(None, 0)
    return l


def tile_ab(x, outer, k_size, S, I, IK):
    """[outer*16*I*S, k_size*64*IK] int8 -> [outer][k_size][S][I][64][IK][16]."""
    x = x.reshape(outer, S, I, 16, k_size, IK, 4, 16)          # om s m r | ko k q t
    return np.ascontiguousarray(x.transpose(0, 4, 1, 2, 6, 3, 5, 7)).reshape(-1)   # om ko s m q r k t


def tile_c(c, om, on, SM, SN, IM, IN):
    c = c.reshape(om, SM, IM, 4, 4, on, SN, IN, 16)             # om sm m q i | on sn n c
    return np.ascontiguousarray(c.transpose(0, 5, 1, 6, 2, 7, 3, 8, 4)).reshape(-1)  # om on sm sn m n q c i


def untile_c(flat, om, on, SM, SN, IM, IN):
    c = flat.reshape(om, on, SM, SN, IM, IN, 4, 16, 4)
    return np.ascontiguousarray(c.transpose(0, 2, 4, 6, 8, 1, 3, 5, 7)).reshape(om * SM * IM * 16, on * SN * IN * 16)


@pytest.mark.parametrize("IM,SM,IN,SN,IK", [(8, 2, 8, 2, 1), (8, 2, 8, 2, 2), (4, 2, 4, 2, 1), (4, 4, 4, 1, 1),
                                             (2, 1, 2, 2, 1), (2, 1, 2, 1, 2), (8, 1, 2, 4, 1), (1, 1, 2, 4, 1),
                                             (2, 1, 2, 4, 1), (3, 1, 2, 4, 2), (3, 2, 5, 2, 1)])
@pytest.mark.parametrize("k_size", [1, 2, 5])
def test_multi_mma_bit_exact(lib, IM, SM, IN, SN, IK, k_size):
    om, on = 3, 2
    rows, cols, depth = om * 16 * IM * SM, on * 16 * IN * SN, k_size * 64 * IK
    rng = np.random.default_rng(IM * 1000 + SM * 100 + IK * 10 + k_size + 7 * SN)
    a = rng.integers(-128, 128, size=(rows, depth), dtype=np.int8)
    b = rng.integers(-128, 128, size=(cols, depth), dtype=np.int8)
    c0 = rng.integers(-1000, 1000, size=(rows, cols), dtype=np.int32)
    want = c0.astype(np.int64) + a.astype(np.int64) @ b.astype(np.int64).T
    d_a = torch.from_numpy(tile_ab(a, om, k_size, SM, IM, IK)).cuda()
    d_b = torch.from_numpy(tile_ab(b, on, k_size, SN, IN, IK)).cuda()
    d_c = torch.from_numpy(tile_c(c0, om, on, SM, SN, IM, IN)).cuda()
    rc = lib.iree_uk_mi355x_multi_mma_i32_16x16x64_i8(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr(), om, on, k_size,
                                                      IM, SM, IN, SN, IK)
    assert rc == 0
    assert lib.iree_uk_mi355x_last_kernel() == b"multi_mma_i32_16x16x64_i8"
    got = untile_c(d_c.cpu().numpy(), om, on, SM, SN, IM, IN)
    assert np.array_equal(got.astype(np.int64), want)


def test_multi_mma_rejects_what_is_not_instantiated_and_host_pointers(lib):
    d = torch.zeros(1 << 20, dtype=torch.int8, device="cuda")
    assert lib.iree_uk_mi355x_multi_mma_i32_16x16x64_i8(d.data_ptr(), d.data_ptr(), d.data_ptr(), 1, 1, 1,
                                                        5, 2, 8, 2, 1) != 0
    h = np.zeros(1 << 20, dtype=np.int8)
    assert lib.iree_uk_mi355x_multi_mma_i32_16x16x64_i8(h.ctypes.data, d.data_ptr(), d.data_ptr(), 1, 1, 1,
                                                        8, 2, 8, 2, 1) != 0


def test_multi_mma_4096_cubed_checksum(lib):
    # Column sums of the whole product without any matmul: sum_i C[i][j] =
    # (sum_i A[i][:]) . B[j][:].
    IM, SM, IN, SN, IK = 8, 2, 8, 2, 1
    om = on = 16
    k_size = 64
    g = torch.Generator(device="cuda").manual_seed(7)
    a = torch.randint(-128, 128, (4096, 4096), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-128, 128, (4096, 4096), dtype=torch.int8, device="cuda", generator=g)
    ta = a.view(om, SM, IM, 16, k_size, IK, 4, 16).permute(0, 4, 1, 2, 6, 3, 5, 7).contiguous()
    tb = b.view(on, SN, IN, 16, k_size, IK, 4, 16).permute(0, 4, 1, 2, 6, 3, 5, 7).contiguous()
    tc = torch.zeros(4096 * 4096, dtype=torch.int32, device="cuda")
    assert lib.iree_uk_mi355x_multi_mma_i32_16x16x64_i8(ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), om, on, k_size,
                                                        IM, SM, IN, SN, IK) == 0
    c = tc.view(om, on, SM, SN, IM, IN, 4, 16, 4).permute(0, 2, 4, 6, 8, 1, 3, 5, 7).reshape(4096, 4096)
    col_ref = (a.double().sum(dim=0) @ b.double().t()).long()
    assert torch.equal(c.long().sum(dim=0), col_ref)
    rows = [0, 1000, 4095]
    ref = (a[rows].double() @ b.double().t()).long()
    assert torch.equal(c[rows].long(), ref)
