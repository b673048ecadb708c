"""Float results do not depend on scheduling: every kernel that splits a sum over
wavefronts or lanes (the K-splitting block kernels, the matrix-vector and
narrow-tile kernels) adds the parts in a fixed order, and nothing uses float
atomics. The same call three times must give the same bits, on every float
kernel, with other work in between. (The reference's CPU code is sequential and
therefore repeatable; a drop-in should not be less so.)
"""
import ctypes as C

import pytest
import torch

from iree_amd import abi
from test_gpu_configs import gpu_lib, mm_params  # noqa: F401

pytestmark = pytest.mark.gpu

F16, BF16, F32 = abi.MMT4D_TYPE_F16F16F32, abi.MMT4D_TYPE_BF16BF16F32, abi.MMT4D_TYPE_F32F32F32
SKIP = abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
CASES = [
    # flags, M, N, K, M0, N0, K0, kernel the case is meant to reach (prefix)
    (F16, 32, 32, 64, 16, 16, 16, b"mmt4d_mfma_"),
    (BF16, 64, 64, 32, 16, 16, 8, b"mmt4d_mfma_"),
    (BF16, 4, 4, 512, 16, 16, 8, b"mmt4d_mfma_64x64_split_k"),
    (BF16, 8, 300, 512, 16, 16, 8, b"mmt4d_mfma_128x64_split_k"),
    (F32, 16, 16, 64, 16, 16, 4, b"mmt4d_mfma_"),
    (abi.MMT4D_TYPE_F16F16F16 | SKIP, 16, 16, 64, 16, 16, 16, b"mmt4d_mfma_"),
    (BF16, 1, 100, 300, 16, 16, 8, b"mmt4d_gemv"),
    (F16, 1, 77, 1000, 4, 16, 8, b"mmt4d_gemv"),
    (BF16, 1, 333, 512, 16, 16, 8, b"mmt4d_gemv_resident_lhs"),
    (F16, 1, 50, 3000, 1, 16, 1, b"mmt4d_skinny"),
    (BF16, 1, 40, 2000, 4, 16, 2, b"mmt4d_skinny"),
    (F32, 1, 60, 1500, 2, 8, 1, b"mmt4d_skinny"),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "t%x_%dx%dx%d_%dx%dx%d" % c[:7])
def test_three_runs_give_the_same_bits(gpu_lib, case):
    flags, M, N, K, M0, N0, K0, kernel = case
    kind = flags & 0xFF
    in_dtype = {F16: torch.float16, BF16: torch.bfloat16, F32: torch.float32, abi.MMT4D_TYPE_F16F16F16: torch.float16}[kind]
    out_dtype = torch.float16 if kind == abi.MMT4D_TYPE_F16F16F16 else torch.float32
    g = torch.Generator(device="cuda").manual_seed(M * N + K)
    lhs = torch.randn(M * K * M0 * K0, device="cuda", generator=g).to(in_dtype)
    rhs = (torch.randn(N * K * N0 * K0, device="cuda", generator=g) / 8).to(in_dtype)
    init = torch.randn(M * N * M0 * N0, device="cuda", generator=g).to(out_dtype)
    noise = torch.randn(1 << 22, device="cuda", generator=g)
    results = []
    for run in range(3):
        out = init.clone()
        p = mm_params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0, flags | abi.MMT4D_ACCUMULATE)
        gpu_lib.iree_uk_mmt4d_p(C.byref(p))
        assert gpu_lib.iree_uk_mi355x_last_kernel().startswith(kernel), gpu_lib.iree_uk_mi355x_last_kernel()
        results.append(out.view(torch.int16 if out_dtype == torch.float16 else torch.int32).clone())
        noise = noise * 1.0001 + run       # unrelated work between the runs
        torch.cuda.synchronize()
    assert torch.equal(results[0], results[1]) and torch.equal(results[0], results[2])
    assert bool(torch.isfinite(results[0].view(out_dtype).float()).all())
