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


def test_kernels_with_large_workgroup_memory_in_a_hip_graph(gpu_lib):
    # The 256x256 tile and the split-K tile use more than 64 KiB of workgroup memory, which is requested per kernel
    # right before the launch, also while a stream is being captured; the skinny kernel for narrow tiles rides along.
    g = torch.Generator(device="cuda").manual_seed(2)

    def int8(n):
        return torch.randint(-128, 128, (n,), dtype=torch.int8, device="cuda", generator=g)

    def bf16(n):
        return (torch.randn(n, device="cuda", generator=g) / 8).to(torch.bfloat16)

    cases = [
        # (lhs, rhs, out, M, N, K, M0, N0, K0, type, kernel)
        (int8(512 * 16 * 32), int8(512 * 16 * 32), torch.zeros(4096 * 4096, dtype=torch.int32, device="cuda"),
         512, 512, 16, 8, 8, 4, abi.MMT4D_TYPE_S8S8S32, b"mmt4d_mfma_256x256"),
        (bf16(5 * 256 * 128), bf16(7 * 256 * 128), torch.zeros(5 * 7 * 256, device="cuda"),
         5, 7, 256, 16, 16, 8, abi.MMT4D_TYPE_BF16BF16F32, b"mmt4d_mfma_64x64_split_k"),
        (int8(200 * 2), int8(64 * 200 * 32), torch.zeros(64 * 16, dtype=torch.int32, device="cuda"),
         1, 64, 200, 1, 16, 2, abi.MMT4D_TYPE_S8S8S32, b"mmt4d_skinny"),
    ]
    params = [mm_params(l.data_ptr(), r.data_ptr(), o.data_ptr(), M, N, K, M0, N0, K0, t)
              for (l, r, o, M, N, K, M0, N0, K0, t, _) in cases]
    gpu_lib.iree_uk_mi355x_set_stream(None, 0)
    want = []
    for p, case in zip(params, cases):
        gpu_lib.iree_uk_mmt4d_p(C.byref(p))
        assert gpu_lib.iree_uk_mi355x_last_kernel() == case[10]
        want.append(case[2].clone())
    try:
        s = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(s):
            gpu_lib.iree_uk_mi355x_set_stream(s.cuda_stream, 1)
            for p in params:
                gpu_lib.iree_uk_mmt4d_p(C.byref(p))
            s.synchronize()
            with torch.cuda.graph(graph, stream=s):
                gpu_lib.iree_uk_mi355x_set_stream(torch.cuda.current_stream().cuda_stream, 1)
                for p in params:
                    gpu_lib.iree_uk_mmt4d_p(C.byref(p))
        for i in range(3):
            for case in cases:
                case[2].fill_(i + 1)  # eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for case, w in zip(cases, want):
                assert torch.equal(case[2], w), (i, case[10])
    finally:
        gpu_lib.iree_uk_mi355x_set_stream(None, 0)
