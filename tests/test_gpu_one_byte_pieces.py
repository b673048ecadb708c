"""int8 tiles with K0 = 1 (one-byte row pieces: the operands are k-major, M0
bytes per k step; the reference's Arm target without dot-product instructions
uses s8s8s32 Mx8x1, mmt4d_arm_64_tiles.inl). On the GPU the transposition to
"a row's consecutive k" happens on the way out of LDS (transposing reads).
Bit-exact against a float64 product (test_gpu_big_tiles.run_case): every block
tile, ragged edges, K ending inside a 64-byte chunk, gaps and offsets,
accumulation, 8- and 16-row tiles mixed between lhs and rhs.
"""
import pytest

from iree_amd import abi
from test_gpu_big_tiles import run_case
from test_gpu_configs import gpu_lib  # noqa: F401

pytestmark = pytest.mark.gpu
S8 = abi.MMT4D_TYPE_S8S8S32


@pytest.mark.parametrize("M0,N0", [(8, 8), (16, 16), (8, 16), (16, 8)])
@pytest.mark.parametrize("M,N,K,kernel", [
    (3, 5, 64, "mmt4d_mfma_64x64"),           # one chunk exactly
    (3, 5, 200, "mmt4d_mfma_64x64"),          # K ends inside a chunk
    (9, 7, 130, "mmt4d_mfma_64x64"),
    (40, 33, 300, None),                      # ragged, several block tiles (whichever tile the cost model picks)
    (131, 135, 258, None),
])
def test_k_major_int8_tiles(gpu_lib, M0, N0, M, N, K, kernel):
    rows, cols = M * M0, N * N0
    for accumulate in (False, True):
        name = kernel or _picked(gpu_lib, M, N, K, M0, N0)
        assert name.startswith("mmt4d_mfma"), name
        run_case(gpu_lib, S8, M, N, K, M0, N0, 1, name, accumulate=accumulate, seed=K + M0 + rows + cols)


def _picked(gpu_lib, M, N, K, M0, N0):
    """Runs the problem once to learn which kernel the library selects."""
    import ctypes as C
    import torch
    from test_gpu_configs import mm_params
    l = torch.zeros(M * K * M0, dtype=torch.int8, device="cuda")
    r = torch.zeros(N * K * N0, dtype=torch.int8, device="cuda")
    o = torch.zeros(M * N * M0 * N0, dtype=torch.int32, device="cuda")
    gpu_lib.iree_uk_mmt4d_p(C.byref(mm_params(l.data_ptr(), r.data_ptr(), o.data_ptr(), M, N, K, M0, N0, 1, S8)))
    return gpu_lib.iree_uk_mi355x_last_kernel().decode()


def test_k_major_int8_tiles_strided_with_offsets(gpu_lib):
    name = _picked(gpu_lib, 70, 66, 500, 8, 8)
    assert name.startswith("mmt4d_mfma")
    run_case(gpu_lib, S8, 70, 66, 500, 8, 8, 1, name, lhs_pad=32, rhs_pad=48, out_pad=12, offsets=(16, 64, 8),
             accumulate=True, seed=11)


def test_odd_k_with_16_row_tiles(gpu_lib):
    # (with 8-row tiles an odd K leaves the tile rows 8-byte aligned only: generic kernel, below)
    run_case(gpu_lib, S8, 9, 7, 129, 16, 16, 1, "mmt4d_mfma_64x64", accumulate=True, seed=5)


def test_what_the_transposing_path_does_not_take_stays_exact(gpu_lib):
    # less than one chunk of K, 4-row tiles, an lhs that is not 16-byte aligned: the narrow-tile kernel
    # (tests/test_gpu_skinny_narrow.py); rhs tile rows that are not 16-byte multiples apart: the generic kernel
    run_case(gpu_lib, S8, 5, 4, 40, 8, 8, 1, "mmt4d_skinny", accumulate=True)
    run_case(gpu_lib, S8, 5, 4, 100, 4, 8, 1, "mmt4d_skinny")
    run_case(gpu_lib, S8, 5, 4, 100, 8, 8, 1, "mmt4d_skinny", offsets=(8, 0, 0))
    run_case(gpu_lib, S8, 5, 4, 129, 8, 8, 1, "mmt4d_generic")
