// A second measuring stick for the benchmark, in the same helper library as the
// matrix-pipe probe (libuk_bench_probe.so, not part of the microkernel library):
// what the device streams to and from HBM with nothing else to do. Three plain
// kernels over a flat buffer, 16 bytes per lane and access, non-temporal like
// the pack / unpack kernels' accesses: read only (summed, the sum written by
// nobody unless it is a value that does not occur), write only, and copy. A
// persistent grid walks the buffer in blocks of 256 threads x UNROLL vectors.
// pack, unpack and the matrix-vector kernels are reported next to these rates:
// the part's published 8 TB/s is not what any kernel reaches.
#include <hip/hip_runtime.h>

#include <cstdint>

#define UK_API extern "C" __attribute__((visibility("default")))

namespace {

typedef int v4i32 __attribute__((ext_vector_type(4)));

// Workgroup -> the block of 256 x UNROLL vectors it starts with. Consecutive workgroup ids run on different
// XCDs (id 8 s + x on XCD x); with xcd_group > 1 each XCD takes xcd_group consecutive blocks at a time, as
// the pack / unpack kernels deal their blocks (what does not fill eight whole groups goes one by one).
__device__ __forceinline__ long long first_block(int xcd_group) {
  const unsigned id = blockIdx.x;
  if (xcd_group <= 1) return id;
  const unsigned xcd = id & 7, slot = id >> 3, group = (unsigned)xcd_group;
  const unsigned grouped_slots = (gridDim.x >> 3) / group * group;
  if (slot >= grouped_slots) return id;
  const unsigned g = slot / group;
  return (long long)(g * 8 + xcd) * group + (slot - g * group);
}

template <int MODE, int UNROLL, bool STREAMING>
__global__ __launch_bounds__(256) void stream_kernel(v4i32* __restrict__ dst, const v4i32* __restrict__ src,
                                                     long long vectors, int xcd_group, int* sink) {
  const long long per_pass = (long long)gridDim.x * 256 * UNROLL;
  v4i32 sum = {0, 0, 0, 0};
  for (long long base = first_block(xcd_group) * 256 * UNROLL; base < vectors; base += per_pass) {
    v4i32 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const long long i = base + u * 256 + threadIdx.x;
      v[u] = v4i32{1, 2, 3, 4};
      if (MODE != 1 && i < vectors) v[u] = STREAMING ? __builtin_nontemporal_load(src + i) : src[i];
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const long long i = base + u * 256 + threadIdx.x;
      if (MODE == 0) {
        sum += v[u];
      } else if (i < vectors) {
        if (STREAMING) __builtin_nontemporal_store(v[u], dst + i); else dst[i] = v[u];
      }
    }
  }
  if (MODE == 0 && (sum.x ^ sum.y ^ sum.z ^ sum.w) == 0x5EEDBEEF) *sink = sum.x;
}

template <int MODE, int UNROLL, bool STREAMING>
int launch(void* dst, const void* src, long long vectors, int grid_blocks, int xcd_group, int resident, void* sink,
           hipStream_t s) {
  const long long one_pass = (vectors + 256 * UNROLL - 1) / (256 * UNROLL);
  const unsigned grid = (unsigned)(grid_blocks > 0 && grid_blocks < one_pass ? grid_blocks : one_pass);
  // Workgroup memory the kernel never touches, asked for only to hold the workgroups per compute unit down.
  const unsigned lds = resident > 0 ? (unsigned)(160 * 1024 / resident < 65536 ? 160 * 1024 / resident : 65536) : 0u;
  hipLaunchKernelGGL((stream_kernel<MODE, UNROLL, STREAMING>), dim3(grid), dim3(256), lds, s, (v4i32*)dst,
                     (const v4i32*)src, vectors, xcd_group, (int*)sink);
  return (int)hipGetLastError();
}

template <int MODE>
int launch_mode(int unroll, int streaming, void* dst, const void* src, long long vectors, int grid_blocks,
                int xcd_group, int resident, void* sink, hipStream_t s) {
  if (unroll == 1) return streaming ? launch<MODE, 1, true>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s)
                                    : launch<MODE, 1, false>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
  if (unroll == 2) return streaming ? launch<MODE, 2, true>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s)
                                    : launch<MODE, 2, false>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
  if (unroll == 4) return streaming ? launch<MODE, 4, true>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s)
                                    : launch<MODE, 4, false>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
  if (unroll == 8) return streaming ? launch<MODE, 8, true>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s)
                                    : launch<MODE, 8, false>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
  if (unroll == 16) return streaming ? launch<MODE, 16, true>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s)
                                     : launch<MODE, 16, false>(dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
  return (int)hipErrorInvalidValue;
}

}  // namespace

// mode 0: read `bytes` from src; 1: write `bytes` to dst; 2: copy src -> dst. `bytes` a multiple of 16, buffers
// 16-byte aligned. `grid_blocks` workgroups of 256 threads (0: one pass over the buffer, i.e. not persistent),
// `unroll` (1, 2, 4, 8 or 16) vectors in flight per thread, `streaming` != 0: non-temporal accesses, `xcd_group` > 1:
// blocks dealt to the XCDs in groups of that many, `resident` > 0: at most that many workgroups per compute unit.
// Enqueues one launch on `stream` and returns the HIP status; the caller times it and keeps the best variant.
UK_API int uk_bench_probe_hbm_stream(int mode, void* dst, const void* src, long long bytes, int grid_blocks,
                                     int unroll, int streaming, int xcd_group, int resident, void* sink, void* stream) {
  if (bytes <= 0 || bytes % 16) return (int)hipErrorInvalidValue;
  const long long vectors = bytes / 16;
  hipStream_t s = (hipStream_t)stream;
  switch (mode) {
    case 0: return launch_mode<0>(unroll, streaming, dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
    case 1: return launch_mode<1>(unroll, streaming, dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
    case 2: return launch_mode<2>(unroll, streaming, dst, src, vectors, grid_blocks, xcd_group, resident, sink, s);
    default: return (int)hipErrorInvalidValue;
  }
}
