// Third measuring stick of the benchmark's helper library (libuk_bench_probe.so, not part of the microkernel
// library): where the time of one launch of the 256x256 int8 mmt4d kernel goes. The kernel is the library's own
// source (mmt4d_mfma_kernels.h) compiled once more with its timeline readings switched on: wavefront 0 of every
// workgroup reads the constant-rate 100 MHz counter at its start, when its main loop begins and ends, when its
// last MFMA has been issued and when its stores have been acknowledged. With `staggered_tail` = 0 the variant
// that stores everything after the loop runs, for comparison.
#define UK_KERNEL_TIMELINE
#define UK_MFMA_KERNEL_BODIES
#include "../mmt4d_mfma_kernels.h"

#define UK_API extern "C" __attribute__((visibility("default")))

namespace {

bool fill_args(uk::MfmaArgs* m, const void* lhs, const void* rhs, void* out, long long M, long long N, long long K,
               int M0, int N0, int K0) {
  const int log2_t = M0 == 8 ? 3 : (M0 == 16 ? 4 : -1);
  if (log2_t < 0 || N0 != M0 || !(K0 == 4 || K0 == 16 || K0 == 32 || K0 == 64)) return false;
  if ((K * K0) % 64 || K * K0 < 512 || ((M * M0 + 255) / 256) * ((N * N0 + 255) / 256) > 256) return false;
  m->lhs = (const uint8_t*)lhs; m->rhs = (const uint8_t*)rhs; m->out = (uint8_t*)out;
  m->lhs_stride_bytes = K * M0 * K0; m->rhs_stride_bytes = K * N0 * K0; m->out_stride0 = N * M0 * N0;
  m->M = (int32_t)M; m->N = (int32_t)N; m->K = (int32_t)K;
  m->log2_M0 = m->log2_N0 = log2_t;
  m->lhs_rb = m->rhs_rb = K0;
  m->log2_lhs_rb = m->log2_rhs_rb = K0 == 4 ? 2 : (K0 == 16 ? 4 : (K0 == 32 ? 5 : 6));
  m->chunks = (int32_t)(K * K0 / 64);
  m->tile_rows = m->tile_cols = 0;
  m->accumulate = 0;
  return true;
}

hipError_t launch(const uk::MfmaArgs& m, int K0, bool staggered_tail, hipStream_t stream) {
  return K0 == 4 ? uk::launch_direct<uk::kI8, false, false, 4, 4, 4, 4>(m, stream, staggered_tail)
                 : uk::launch_direct<uk::kI8, false, false, 16, 4, 4, 4>(m, stream, staggered_tail);
}

}  // namespace

// s8s8s32 problem of M x N x K tiles (M0 = N0 in {8, 16}; K0 = 4 or K0 in {16, 32, 64}), tight strides, device
// pointers, K in whole 64-byte chunks and at least 8 of them, no more than 256 block tiles.
// One launch of the instrumented kernel on `stream`, nothing else (for timing it from outside).
UK_API int uk_bench_probe_mmt4d_launch(const void* lhs, const void* rhs, void* out, long long M, long long N,
                                       long long K, int M0, int N0, int K0, int staggered_tail, void* stream) {
  uk::MfmaArgs m;
  if (!fill_args(&m, lhs, rhs, out, M, N, K, M0, N0, K0)) return (int)hipErrorInvalidValue;
  return (int)launch(m, K0, staggered_tail != 0, (hipStream_t)stream);
}

// Runs `warmup` launches back to back and then `repeats` groups of five; after each group it synchronises and
// reads the last launch's readings. Writes, averaged over the groups, for each of the `*tiles` workgroups five
// times in ns relative to the earliest start: start, loop begin, loop end, last MFMA, stores acknowledged
// (readings[5*w+i]).
UK_API int uk_bench_probe_mmt4d_timeline(const void* lhs, const void* rhs, void* out, long long M, long long N,
                                         long long K, int M0, int N0, int K0, int staggered_tail, int warmup,
                                         int repeats, double* readings, int* tiles) {
  uk::MfmaArgs m;
  if (!fill_args(&m, lhs, rhs, out, M, N, K, M0, N0, K0) || repeats < 1) return (int)hipErrorInvalidValue;
  const int n = (int)(((M * M0 + 255) / 256) * ((N * N0 + 255) / 256));
  for (int i = 0; i < 5 * n; ++i) readings[i] = 0;
  hipError_t e = hipSuccess;
  for (int i = 0; i < warmup && e == hipSuccess; ++i) e = launch(m, K0, staggered_tail != 0, nullptr);
  static unsigned long long raw[256 * 8];
  for (int r = 0; r < repeats && e == hipSuccess; ++r) {
    for (int i = 0; i < 5 && e == hipSuccess; ++i) e = launch(m, K0, staggered_tail != 0, nullptr);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipMemcpyFromSymbol(raw, HIP_SYMBOL(uk::uk_timeline), sizeof raw);
    if (e != hipSuccess) break;
    unsigned long long first = ~0ull;
    for (int w = 0; w < n; ++w) first = raw[8 * w] < first ? raw[8 * w] : first;
    for (int w = 0; w < n; ++w)
      for (int i = 0; i < 5; ++i) readings[5 * w + i] += 10.0 * (double)(raw[8 * w + i] - first) / repeats;
  }
  if (e != hipSuccess) return (int)e;
  *tiles = n;
  return 0;
}
