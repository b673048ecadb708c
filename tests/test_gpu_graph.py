"""Asynchronous calls on device buffers can be recorded into a HIP graph and
replayed (what a serving loop does to get rid of launch overhead): each replay
is checked against the eagerly computed result, with eager work and
synchronisation between the replays.
"""
import ctypes as C

import pytest
import torch

from iree_amd import abi
from test_gpu_configs import gpu_lib, mm_params  # noqa: F401

pytestmark = pytest.mark.gpu


def test_mmt4d_and_pack_in_a_hip_graph(gpu_lib):
    M, N, K, M0, N0, K0 = 96, 80, 64, 8, 8, 4
    g = torch.Generator(device="cuda").manual_seed(1)
    lhs = torch.randint(-128, 128, (M * K * M0 * K0,), dtype=torch.int8, device="cuda", generator=g)
    rhs = torch.randint(-128, 128, (N * K * N0 * K0,), dtype=torch.int8, device="cuda", generator=g)
    out = torch.zeros(M * N * M0 * N0, dtype=torch.int32, device="cuda")
    p = mm_params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), M, N, K, M0, N0, K0, abi.MMT4D_TYPE_S8S8S32)
    src = torch.randn(300 * 200, device="cuda", generator=g)
    packed = torch.zeros(38 * 50 * 32, device="cuda")
    q = abi.PackParams()
    q.in_buffer, q.out_buffer = src.data_ptr(), packed.data_ptr()
    q.in_stride0, q.in_stride1, q.out_stride0, q.out_stride1 = 200, 1, 50 * 32, 32
    q.in_size0, q.in_size1 = 300, 200
    q.out_size0, q.out_size1, q.out_size2, q.out_size3 = 38, 50, 8, 4
    q.padding_value, q.flags = 0, abi.PACK_TYPE_F32F32
    # eager results
    gpu_lib.iree_uk_mi355x_set_stream(None, 0)
    gpu_lib.iree_uk_mmt4d_p(C.byref(p))
    gpu_lib.iree_uk_pack_p(C.byref(q))
    want_out, want_packed = out.clone(), packed.clone()
    try:
        s = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(s):
            gpu_lib.iree_uk_mi355x_set_stream(s.cuda_stream, 1)
            gpu_lib.iree_uk_mmt4d_p(C.byref(p))
            gpu_lib.iree_uk_pack_p(C.byref(q))
            s.synchronize()
            with torch.cuda.graph(graph, stream=s):
                gpu_lib.iree_uk_mi355x_set_stream(torch.cuda.current_stream().cuda_stream, 1)
                gpu_lib.iree_uk_mmt4d_p(C.byref(p))
                gpu_lib.iree_uk_pack_p(C.byref(q))
        for i in range(3):
            out.fill_(i)          # eager work between replays
            packed.fill_(float(i))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want_out), i
            assert torch.equal(packed, want_packed), i
    finally:
        gpu_lib.iree_uk_mi355x_set_stream(None, 0)
