"""The allocation-free mmt4d entry point (iree_uk_mi355x_mmt4d_noalloc_p, no
counterpart in the reference) against iree_uk_mmt4d_p on the same host
operands, through the C ABI: bit-exact for integers, identical bits for floats
(both run the same kernel), also against the oracle. Two calls in a row share
the device's static staging memory; the second is smaller, so stale bytes of
the first would show. Sizes beyond the stated maximum are rejected through the
failure handler without launching."""
import ctypes as C

import numpy as np
import pytest
import torch

from iree_amd import abi, library, synth

pytestmark = pytest.mark.gpu


def _params(lhs, rhs, out, M, N, K, M0, N0, K0, flags, lhs_stride=None, out_stride=None):
    p = abi.Mmt4dParams()
    p.lhs_buffer, p.rhs_buffer, p.out_buffer = lhs.ctypes.data, rhs.ctypes.data, out.ctypes.data
    p.lhs_stride0 = K * M0 * K0 if lhs_stride is None else lhs_stride
    p.rhs_stride0 = K * N0 * K0
    p.out_stride0 = N * M0 * N0 if out_stride is None else out_stride
    p.M, p.N, p.K, p.M0, p.N0, p.K0, p.flags = M, N, K, M0, N0, K0, flags
    return p


def _case(seed, M, N, K, M0, N0, K0, flags, gap=0):
    """Host operands; `gap` extra elements between lhs rows and between out rows."""
    ls, os_ = K * M0 * K0 + gap, N * M0 * N0 + gap
    if flags & 0xFF == abi.MMT4D_TYPE_S8S8S32:
        lhs = synth.uniform_int8(seed, 0, M * ls)
        rhs = synth.uniform_int8(seed, 1, N * K * N0 * K0)
        init = (synth.bits64(seed, 2, M * os_) & np.uint64(0xFFFFF)).astype(np.int32)
    else:
        lhs = synth.f16_bits(synth.normal_f32(seed, 0, M * ls, 1.0 / 8))
        rhs = synth.f16_bits(synth.normal_f32(seed, 1, N * K * N0 * K0, 1.0 / 8))
        init = synth.normal_f32(seed, 2, M * os_)
    return lhs, rhs, init, ls, os_


CASES = [
    # (M, N, K, M0, N0, K0, flags, gap): the first is the larger one.
    (48, 40, 64, 8, 8, 4, abi.MMT4D_TYPE_S8S8S32 | abi.MMT4D_ACCUMULATE, 32),
    (5, 3, 7, 8, 8, 4, abi.MMT4D_TYPE_S8S8S32, 0),
    (12, 9, 20, 16, 16, 16, abi.MMT4D_TYPE_F16F16F32 | abi.MMT4D_ACCUMULATE, 16),
    (1, 2, 3, 16, 16, 16, abi.MMT4D_TYPE_F16F16F32, 0),
]


def test_noalloc_matches_allocating_entry_point_twice_in_a_row(oracle_lib):
    assert torch.cuda.is_available()
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    for seed, (M, N, K, M0, N0, K0, flags, gap) in enumerate(CASES):
        lhs, rhs, init, ls, os_ = _case(100 + seed, M, N, K, M0, N0, K0, flags, gap)
        got, want, ref = init.copy(), init.copy(), init.copy()
        lib.iree_uk_mi355x_mmt4d_noalloc_p(C.byref(_params(lhs, rhs, got, M, N, K, M0, N0, K0, flags, ls, os_)))
        kernel = lib.iree_uk_mi355x_last_kernel()
        lib.iree_uk_mmt4d_p(C.byref(_params(lhs, rhs, want, M, N, K, M0, N0, K0, flags, ls, os_)))
        assert kernel == lib.iree_uk_mi355x_last_kernel() and kernel != b""
        # Same kernel on the same bytes: identical bits, gaps between rows included.
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (M, N, K)
        oracle_lib.oracle_mmt4d(C.byref(_params(lhs, rhs, ref, M, N, K, M0, N0, K0,
                                                flags | abi.MMT4D_ALLOW_GENERIC_FALLBACK, ls, os_)))
        if flags & 0xFF == abi.MMT4D_TYPE_S8S8S32:
            assert np.array_equal(got, ref), (M, N, K)
        else:
            rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
            assert np.all(np.abs(got - ref) <= 1e-3 * np.maximum(np.abs(ref), rms)), (M, N, K)


def test_noalloc_takes_device_operands_without_staging():
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    M, N, K, M0, N0, K0 = 64, 64, 128, 8, 8, 4   # 2 MiB of int32 output: would not matter, nothing is staged
    lhs, rhs, init, _, _ = _case(7, M, N, K, M0, N0, K0, abi.MMT4D_TYPE_S8S8S32)
    d_l, d_r = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
    d_a, d_b = torch.from_numpy(init).cuda(), torch.from_numpy(init).cuda()

    def dev_params(out):
        p = abi.Mmt4dParams()
        p.lhs_buffer, p.rhs_buffer, p.out_buffer = d_l.data_ptr(), d_r.data_ptr(), out.data_ptr()
        p.lhs_stride0, p.rhs_stride0, p.out_stride0 = K * M0 * K0, K * N0 * K0, N * M0 * N0
        p.M, p.N, p.K, p.M0, p.N0, p.K0, p.flags = M, N, K, M0, N0, K0, abi.MMT4D_TYPE_S8S8S32
        return p

    lib.iree_uk_mi355x_mmt4d_noalloc_p(C.byref(dev_params(d_a)))
    lib.iree_uk_mmt4d_p(C.byref(dev_params(d_b)))
    assert torch.equal(d_a, d_b)


def test_noalloc_rejects_operands_beyond_its_static_memory():
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    limit = 16 * 1024 * 1024
    # lhs 4 MiB + rhs 4 MiB + out 16 MiB of host memory: more than the array holds.
    M = N = 256
    K, M0, N0, K0 = 64, 8, 8, 4
    assert M * K * M0 * K0 + N * K * N0 * K0 + 4 * M * N * M0 * N0 > limit
    lhs = np.zeros(M * K * M0 * K0, np.int8)
    rhs = np.zeros(N * K * N0 * K0, np.int8)
    out = np.full(M * N * M0 * N0, 77, np.int32)
    seen = []
    cb = library.FAIL_HANDLER(lambda f, l, fn, cond: seen.append(cond.decode()))
    lib.iree_uk_mi355x_set_fail_handler(cb)
    try:
        lib.iree_uk_mi355x_mmt4d_noalloc_p(C.byref(_params(lhs, rhs, out, M, N, K, M0, N0, K0,
                                                           abi.MMT4D_TYPE_S8S8S32)))
    finally:
        lib.iree_uk_mi355x_set_fail_handler(library.FAIL_HANDLER(0))
    assert len(seen) == 1 and "IREE_UK_MI355X_NOALLOC_MAX_STAGED_BYTES" in seen[0], seen
    assert lib.iree_uk_mi355x_last_kernel() == b""
    assert np.all(out == 77)
    # The same shapes still run on the allocating entry point.
    lib.iree_uk_mmt4d_p(C.byref(_params(lhs, rhs, out, M, N, K, M0, N0, K0, abi.MMT4D_TYPE_S8S8S32)))
    assert np.all(out == 0)


def _run_in_thread(fn):
    import threading
    box = {}

    def body():
        try:
            box["value"] = fn()
        except BaseException as e:   # re-raised in the caller
            box["error"] = e
    t = threading.Thread(target=body)
    t.start()
    t.join()
    if "error" in box:
        raise box["error"]
    return box.get("value")


def test_noalloc_call_leaves_free_device_memory_unchanged():
    """The property the entry point exists for: no hipMalloc / hipFree. A fresh host thread owns no staging
    buffers, so its first call with host operands is where the allocating entry point must allocate
    (seen below as a drop in free device memory, which shows that the measure can see it) and where this one
    must not."""
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    M, N, K, M0, N0, K0 = 96, 64, 512, 8, 8, 4     # lhs 1.5 MiB, rhs 1 MiB, out 1.5 MiB of host memory
    flags = abi.MMT4D_TYPE_S8S8S32
    lhs, rhs, init, _, _ = _case(11, M, N, K, M0, N0, K0, flags)
    torch.cuda.synchronize()

    def measure(entry):
        def body():
            assert lib.iree_uk_mi355x_init(0) == 0
            out = init.copy()
            free_before, _ = torch.cuda.mem_get_info()
            entry(C.byref(_params(lhs, rhs, out, M, N, K, M0, N0, K0, flags)))
            free_after, _ = torch.cuda.mem_get_info()
            return free_before - free_after, out
        return _run_in_thread(body)

    used_noalloc, got = measure(lib.iree_uk_mi355x_mmt4d_noalloc_p)
    used_alloc, want = measure(lib.iree_uk_mmt4d_p)
    assert np.array_equal(got, want)
    assert used_noalloc == 0, used_noalloc
    assert used_alloc >= lhs.nbytes + rhs.nbytes + init.nbytes, used_alloc


def test_noalloc_overlapping_calls_are_correct_or_cleanly_refused():
    """Two host threads call the entry point with host operands at the same time, on one device: they share
    its static staging memory, which only one call may use at a time. Every call must either produce the
    result of the allocating entry point or be refused through the failure handler with its output
    untouched ("static staging memory busy"); the microkernels are to be callable from many threads
    (the reference's README.md:26)."""
    import threading
    lib = library.load()
    assert lib.iree_uk_mi355x_init(0) == 0
    lib.iree_uk_mi355x_set_stream(None, 0)
    M, N, K, M0, N0, K0 = 64, 48, 512, 8, 8, 4
    flags = abi.MMT4D_TYPE_S8S8S32 | abi.MMT4D_ACCUMULATE
    cases = []
    for seed in (31, 32):
        lhs, rhs, init, _, _ = _case(seed, M, N, K, M0, N0, K0, flags)
        want = init.copy()
        lib.iree_uk_mmt4d_p(C.byref(_params(lhs, rhs, want, M, N, K, M0, N0, K0, flags)))
        cases.append((lhs, rhs, init, want))

    refused = {}    # thread id -> messages
    cb = library.FAIL_HANDLER(lambda f, l, fn, cond: refused.setdefault(threading.get_ident(), []).append(cond.decode()))
    lib.iree_uk_mi355x_set_fail_handler(cb)
    outcomes = {0: [0, 0], 1: [0, 0]}   # worker -> [done, refused]
    errors = []
    start = threading.Barrier(2)

    def worker(w):
        try:
            assert lib.iree_uk_mi355x_init(0) == 0
            lhs, rhs, init, want = cases[w]
            mine = refused.setdefault(threading.get_ident(), [])
            start.wait()
            for _ in range(60):
                out = init.copy()
                before = len(mine)
                lib.iree_uk_mi355x_mmt4d_noalloc_p(C.byref(_params(lhs, rhs, out, M, N, K, M0, N0, K0, flags)))
                if len(mine) > before:
                    assert len(mine) == before + 1 and "static staging memory busy" in mine[-1], mine[-1]
                    assert np.array_equal(out, init), "a refused call wrote its output"
                    outcomes[w][1] += 1
                else:
                    assert np.array_equal(out, want), "an accepted call gave a wrong result"
                    outcomes[w][0] += 1
        except BaseException as e:
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(w,)) for w in (0, 1)]
    try:
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    finally:
        lib.iree_uk_mi355x_set_fail_handler(library.FAIL_HANDLER(0))
    if errors:
        raise errors[0]
    assert outcomes[0][0] > 0 and outcomes[1][0] > 0, outcomes
    assert sum(outcomes[0]) == 60 and sum(outcomes[1]) == 60, outcomes
    # Afterwards the memory is free again.
    out = cases[0][2].copy()
    lib.iree_uk_mi355x_mmt4d_noalloc_p(C.byref(_params(cases[0][0], cases[0][1], out, M, N, K, M0, N0, K0, flags)))
    assert np.array_equal(out, cases[0][3])
