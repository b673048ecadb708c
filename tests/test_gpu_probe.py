"""The benchmark's matrix-pipe probe (its own helper library, no counterpart in
the reference): argument checks, and that its figures are those of an MFMA loop on
this device (below the published int8 peak, at a plausible shader clock, the
cycle count per step that 32 MFMAs of 8 passes x 4 cycles take)."""
import ctypes as C

import pytest
import torch

from iree_amd import abi, library

pytestmark = pytest.mark.gpu


def _probe(lib, buf, traffic, steps=1024, type_flag=abi.MMT4D_TYPE_S8S8S32):
    tops, mhz = C.c_double(), C.c_double()
    rc = library.load_bench_probe().uk_bench_probe_matrix_pipe(type_flag, buf.data_ptr(), buf.numel(), traffic, steps,
                                              C.byref(tops), C.byref(mhz))
    return rc, tops.value, mhz.value


def test_probe_reports_mfma_loop_rates():
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    zeros = torch.zeros(2 << 20, dtype=torch.int8, device="cuda")
    rand = torch.randint(-128, 128, (2 << 20,), dtype=torch.int8, device="cuda")
    for buf in (zeros, rand):
        for traffic in (0, 1):
            rc, tops, mhz = _probe(lib, buf, traffic)
            assert rc == 0
            assert 500.0 < tops < 5033.0
            assert 500.0 < mhz < 2600.0
            # ops = CUs * 4 wavefronts * steps * 32 MFMAs * 65536; with the clock
            # that is cycles per step: 32 MFMAs x 32 cycles = 1024 when the pipe
            # never waits (5 % allowed for the memory instructions and the ends).
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            cycles_per_step = mhz * 1e6 / (tops * 1e12 / (cus * 4 * 32 * 65536.0))
            assert 1024.0 <= cycles_per_step < 1024.0 * 1.08, cycles_per_step
    # f16 / bf16: half the operations per MFMA, the same 32 cycles each.
    halves = (torch.randn(1 << 20, device="cuda") / 64)
    for type_flag, buf in ((abi.MMT4D_TYPE_F16F16F32, halves.half()), (abi.MMT4D_TYPE_BF16BF16F32, halves.bfloat16())):
        raw = buf.view(torch.int8)
        rc, tflops, mhz = _probe(lib, raw, 1, type_flag=type_flag)
        assert rc == 0
        assert 250.0 < tflops < 2516.0
        cycles_per_step = mhz * 1e6 / (tflops * 1e12 / (cus * 4 * 32 * 32768.0))
        assert 1024.0 <= cycles_per_step < 1024.0 * 1.08, cycles_per_step


def test_probe_rejects_bad_arguments():
    lib = library.load()
    buf = torch.zeros(2 << 20, dtype=torch.int8, device="cuda")
    invalid = 1  # hipErrorInvalidValue
    s8 = abi.MMT4D_TYPE_S8S8S32
    assert library.load_bench_probe().uk_bench_probe_matrix_pipe(s8, None, 2 << 20, 0, 64, None, None) == invalid
    assert library.load_bench_probe().uk_bench_probe_matrix_pipe(s8, buf.data_ptr(), 1 << 20, 0, 64, None, None) == invalid
    assert library.load_bench_probe().uk_bench_probe_matrix_pipe(s8, buf.data_ptr(), 2 << 20, 0, 63, None, None) == invalid
    assert library.load_bench_probe().uk_bench_probe_matrix_pipe(s8, buf.data_ptr(), 2 << 20, 0, 0, None, None) == invalid
    assert library.load_bench_probe().uk_bench_probe_matrix_pipe(abi.MMT4D_TYPE_S8S4S32, buf.data_ptr(), 2 << 20, 0, 64, None, None) == invalid
    # Output pointers are optional.
    assert library.load_bench_probe().uk_bench_probe_matrix_pipe(s8, buf.data_ptr(), 2 << 20, 1, 64, None, None) == 0
