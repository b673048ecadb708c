"""GPU parity over the reference's own test grids, through the C ABI.

Every case of tools/mmt4d_test.c:459-603, tools/pack_test.c:132-241 and
tools/unpack_test.c:118-216 (plus the tile shapes of this library's
specialised kernels) is run on the GPU from host buffers and compared with the
CPU oracle byte for byte over the WHOLE output buffer, stride gaps included.
Float cases are exact too: inputs are small integers so every intermediate is
representable (tools/util.c:133-146), whatever the summation order.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import ukcases
from iree_amd import abi, library

pytestmark = pytest.mark.gpu


def _mm_ids(tiles):
    return ["%s_%dx%dx%d%s" % (abi.MMT4D_NAMES[t[0] & 0xFF], t[1], t[2], t[3],
                               "_skipround" if t[0] & abi.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS else "")
            for t in tiles]


def _pk_ids(tiles):
    return ["%s_%dx%d" % (ukcases.PACK_NAMES[t[0]], t[1], t[2]) for t in tiles]


MM_TILES = ukcases.MMT4D_TILES_GENERIC + ukcases.MMT4D_TILES_X86 + ukcases.MMT4D_TILES_GPU
PACK_TILES = ukcases.PACK_TILES_GENERIC + ukcases.PACK_TILES_X86 + ukcases.PACK_TILES_GPU
UNPACK_TILES = ukcases.UNPACK_TILES_GENERIC + ukcases.UNPACK_TILES_X86 + ukcases.UNPACK_TILES_GPU


@pytest.fixture(scope="module")
def gpu_lib():
    assert torch.cuda.is_available()
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    return lib


@pytest.mark.parametrize("tile", MM_TILES, ids=_mm_ids(MM_TILES))
def test_mmt4d_grid_host_buffers(tile, gpu_lib, oracle_lib):
    for case in ukcases.mmt4d_cases(tile):
        print("case:", case.label(), flush=True)
        want = case.run_host(oracle_lib.oracle_mmt4d)
        got = case.run_host(gpu_lib.iree_uk_mmt4d_p)
        assert np.array_equal(got, want), case.label()


@pytest.mark.parametrize("tile", MM_TILES, ids=_mm_ids(MM_TILES))
def test_mmt4d_grid_device_buffers(tile, gpu_lib, oracle_lib):
    for case in ukcases.mmt4d_cases(tile):
        print("case:", case.label(), flush=True)
        want = case.run_host(oracle_lib.oracle_mmt4d)
        pad = np.zeros(16, np.uint8)
        lhs = torch.from_numpy(np.concatenate([case.lhs, pad])).cuda()
        rhs = torch.from_numpy(np.concatenate([case.rhs, pad])).cuda()
        out = torch.from_numpy(np.concatenate([case.out_init, pad])).cuda()
        p = case.params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr())
        gpu_lib.iree_uk_mmt4d_p(C.byref(p))
        got = out.cpu().numpy()[:case.out_init.size]
        assert np.array_equal(got, want), case.label()


@pytest.mark.parametrize("tile", PACK_TILES, ids=_pk_ids(PACK_TILES))
def test_pack_grid(tile, gpu_lib, oracle_lib):
    for case in ukcases.pack_cases(tile):
        print("case:", case.label(), flush=True)
        want = case.run_host(oracle_lib.oracle_pack)
        got = case.run_host(gpu_lib.iree_uk_pack_p)
        assert np.array_equal(got, want), case.label()
        # device buffers
        pad = np.zeros(16, np.uint8)
        inp = torch.from_numpy(np.concatenate([case.inp, pad])).cuda()
        out = torch.from_numpy(np.concatenate([case.out_init, pad])).cuda()
        p = case.params(inp.data_ptr(), out.data_ptr())
        gpu_lib.iree_uk_pack_p(C.byref(p))
        assert np.array_equal(out.cpu().numpy()[:case.out_init.size], want), case.label()


@pytest.mark.parametrize("tile", UNPACK_TILES, ids=_pk_ids(UNPACK_TILES))
def test_unpack_grid(tile, gpu_lib, oracle_lib):
    for case in ukcases.unpack_cases(tile):
        print("case:", case.label(), flush=True)
        want = case.run_host(oracle_lib.oracle_unpack)
        got = case.run_host(gpu_lib.iree_uk_unpack_p)
        assert np.array_equal(got, want), case.label()
        pad = np.zeros(16, np.uint8)
        inp = torch.from_numpy(np.concatenate([case.inp, pad])).cuda()
        out = torch.from_numpy(np.concatenate([case.out_init, pad])).cuda()
        p = case.params(inp.data_ptr(), out.data_ptr())
        gpu_lib.iree_uk_unpack_p(C.byref(p))
        assert np.array_equal(out.cpu().numpy()[:case.out_init.size], want), case.label()
