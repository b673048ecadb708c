// MFMA mmt4d for gfx950: s8s8s32, s8s4s32, f16f16f32 and bf16bf16f32.
//
// One workgroup of 256 threads (4 wavefronts in a 2x2 arrangement) computes a
// block of (32*AM) lhs rows x (32*BN) rhs rows of the logical matrix; each
// wavefront owns a (16*AM) x (16*BN) sub-block as AM x BN accumulator
// fragments of one 16x16 MFMA each. The K dimension is walked in chunks of 64
// BYTES per operand row (64 int8 or 32 f16/bf16 values = one MFMA K-block).
//
// Data flow per chunk: global -> registers (issued one chunk ahead) -> LDS,
// stored fragment-major so that a wavefront fetches one 16-row x 64-byte MFMA
// operand with a single conflict-free 128-bit LDS read per lane -> MFMA.
//
// Operand layouts. An mmt4d operand row (one i0 of one tile) is not contiguous
// in memory: its K0 values of consecutive k are M0*K0 elements apart
// (mmt4d_tile_generic.c:70-71). With RB = bytes of one (k, i0) row piece:
//   RB multiple of 16: a lane's 16 operand bytes are contiguous in memory and
//     K is consumed in its natural order;
//   RB == 4 (the 8x8x4 int8 tiles): a lane's 16 bytes are gathered from 4
//     consecutive k steps. That permutes K inside a chunk, identically for
//     lhs and rhs, which leaves every integer sum unchanged.
// The int4 rhs of s8s4s32 is widened in registers on its way to LDS: nibble n
// becomes the int8 value 16*n (sign in bit 7, no sign-extension step), the
// accumulators therefore hold 16x the result and are shifted right by 4 at
// the end, which is exact while 16*128*8*depth < 2^31.
//
// The MFMA is issued with the rhs fragment as its row operand and the lhs
// fragment as its column operand, so a lane ends up with 4 consecutive j0 of
// one output row: one 128-bit store per fragment into the [M0][N0] tile.
#include "uk_internal.h"

namespace uk {
namespace {

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf16 __attribute__((ext_vector_type(8)));

enum Kind { kI8 = 0, kF16 = 1, kBF16 = 2 };

struct MfmaArgs {
  const uint8_t* lhs;
  const uint8_t* rhs;
  uint8_t* out;
  int64_t lhs_stride_bytes;  // between consecutive lhs tiles rows (i)
  int64_t rhs_stride_bytes;
  int64_t out_stride0;       // elements
  int32_t M, N, K;           // tile counts
  int32_t log2_M0, log2_N0;
  int32_t lhs_rb, rhs_rb;    // bytes of one (k, i0) row piece
  int32_t log2_lhs_rb, log2_rhs_rb;
  int32_t chunks;            // ceil(K * lhs_rb / 64)
  int32_t tile_rows, tile_cols;  // grid of block tiles
  int32_t accumulate;
};

template <int KIND>
struct AccType { typedef v4i32 type; };
template <> struct AccType<kF16> { typedef v4f32 type; };
template <> struct AccType<kBF16> { typedef v4f32 type; };

template <int KIND>
__device__ __forceinline__ typename AccType<KIND>::type mfma(uint4 row_operand, uint4 col_operand,
                                                             typename AccType<KIND>::type acc) {
  if constexpr (KIND == kI8) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i32, row_operand),
                                                 __builtin_bit_cast(v4i32, col_operand), acc, 0, 0, 0);
  } else if constexpr (KIND == kF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, row_operand),
                                                  __builtin_bit_cast(v8f16, col_operand), acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf16, row_operand),
                                                   __builtin_bit_cast(v8bf16, col_operand), acc, 0, 0, 0);
  }
}

// 16 int4 values (two dwords, element 2b in the low nibble of byte b) to 16
// int8 values equal to 16x the signed nibbles, in element order.
__device__ __forceinline__ uint4 widen_i4_times16(uint2 w) {
  const uint32_t lo0 = (w.x << 4) & 0xF0F0F0F0u, hi0 = w.x & 0xF0F0F0F0u;
  const uint32_t lo1 = (w.y << 4) & 0xF0F0F0F0u, hi1 = w.y & 0xF0F0F0F0u;
  uint4 r;
  r.x = (lo0 & 0xFFu) | ((hi0 & 0xFFu) << 8) | ((lo0 & 0xFF00u) << 8) | ((hi0 & 0xFF00u) << 16);
  r.y = ((lo0 >> 16) & 0xFFu) | (((hi0 >> 16) & 0xFFu) << 8) | ((lo0 >> 8) & 0xFF0000u) |
        (hi0 & 0xFF000000u);
  r.z = (lo1 & 0xFFu) | ((hi1 & 0xFFu) << 8) | ((lo1 & 0xFF00u) << 8) | ((hi1 & 0xFF00u) << 16);
  r.w = ((lo1 >> 16) & 0xFFu) | (((hi1 >> 16) & 0xFFu) << 8) | ((lo1 >> 8) & 0xFF0000u) |
        (hi1 & 0xFF000000u);
  return r;
}

// One 16-byte operand piece: row `row_base` (address of its k = 0 piece), 16-byte
// column `c` (0..3) of chunk `kc`. G is the contiguous run in memory: 16 (vector
// load), 4 (gather 4 k steps) or, for I4, 8 bytes of nibbles widened to 16.
// `kstep` is the distance in bytes between consecutive k of the same row.
template <int G, bool I4>
__device__ __forceinline__ uint4 load_piece(const uint8_t* row_base, int64_t kstep, int32_t rb,
                                            int32_t log2_rb, int32_t K, int kc, int c) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if constexpr (I4) {
    const int32_t row_byte = 32 * kc + 8 * c;  // in bytes of packed nibbles
    const int32_t k1 = row_byte >> log2_rb;
    if (k1 < K) {
      const uint2 w = *(const uint2*)(row_base + (int64_t)k1 * kstep + (row_byte & (rb - 1)));
      v = widen_i4_times16(w);
    }
  } else if constexpr (G == 16) {
    const int32_t row_byte = 64 * kc + 16 * c;
    const int32_t k1 = row_byte >> log2_rb;
    if (k1 < K) v = *(const uint4*)(row_base + (int64_t)k1 * kstep + (row_byte & (rb - 1)));
  } else {  // G == 4: rb == 4
    const int32_t k1 = 16 * kc + 4 * c;
    const uint8_t* p = row_base + (int64_t)k1 * kstep;
    if (k1 + 0 < K) v.x = *(const uint32_t*)(p);
    if (k1 + 1 < K) v.y = *(const uint32_t*)(p + kstep);
    if (k1 + 2 < K) v.z = *(const uint32_t*)(p + 2 * kstep);
    if (k1 + 3 < K) v.w = *(const uint32_t*)(p + 3 * kstep);
  }
  return v;
}

template <int KIND, bool RHS_I4, int G, int AM, int BN>
__global__ __launch_bounds__(256) void mmt4d_mfma_kernel(const MfmaArgs a) {
  typedef typename AccType<KIND>::type acc_t;
  constexpr int BLOCK_ROWS = 32 * AM;  // lhs rows per workgroup
  constexpr int BLOCK_COLS = 32 * BN;  // rhs rows per workgroup
  constexpr int A_PIECES = BLOCK_ROWS * 4;  // 16-byte pieces per chunk
  constexpr int B_PIECES = BLOCK_COLS * 4;
  constexpr int A_PER_THREAD = (A_PIECES + 255) / 256;
  constexpr int B_PER_THREAD = (B_PIECES + 255) / 256;
  __shared__ uint4 lds_a[2][A_PIECES];
  __shared__ uint4 lds_b[2][B_PIECES];

  // Workgroup -> block tile. Consecutive workgroup ids go to different XCDs
  // (8 of them, each with its own L2), so ids are first regrouped so that one
  // XCD works on a contiguous range of tiles, then that range is walked in
  // bands of 4 tile rows so that neighbours share lhs and rhs panels.
  const int total_tiles = a.tile_rows * a.tile_cols;
  const int per_xcd = (total_tiles + 7) >> 3;
  const int linear = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (linear >= total_tiles) return;
  constexpr int BAND = 4;
  const int band = linear / (BAND * a.tile_cols);
  const int band_first = band * BAND;
  const int band_rows = min(a.tile_rows - band_first, BAND);
  const int in_band = linear - band * BAND * a.tile_cols;
  const int tile_row = band_first + in_band % band_rows;
  const int tile_col = in_band / band_rows;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;

  const int32_t M0 = 1 << a.log2_M0, N0 = 1 << a.log2_N0;
  const int64_t total_rows = (int64_t)a.M << a.log2_M0;
  const int64_t total_cols = (int64_t)a.N << a.log2_N0;
  const int64_t lhs_kstep = (int64_t)a.lhs_rb << a.log2_M0;
  const int64_t rhs_kstep = (int64_t)a.rhs_rb << a.log2_N0;

  // Rows this thread copies. Piece p = tid + 256*s lands at LDS slot p, which
  // is fragment (p >> 6), 16-byte column (p >> 4) & 3, row p & 15 of the
  // fragment. Rows past the end of the matrix are redirected to its last row:
  // their products are computed and never stored.
  const uint8_t* a_row[A_PER_THREAD];
  const uint8_t* b_row[B_PER_THREAD];
#pragma unroll
  for (int s = 0; s < A_PER_THREAD; ++s) {
    const int p = tid + 256 * s;
    int64_t row = (int64_t)tile_row * BLOCK_ROWS + (p >> 6) * 16 + (p & 15);
    row = min(row, total_rows - 1);
    a_row[s] = a.lhs + (row >> a.log2_M0) * a.lhs_stride_bytes + (row & (M0 - 1)) * a.lhs_rb;
  }
#pragma unroll
  for (int s = 0; s < B_PER_THREAD; ++s) {
    const int p = tid + 256 * s;
    int64_t row = (int64_t)tile_col * BLOCK_COLS + (p >> 6) * 16 + (p & 15);
    row = min(row, total_cols - 1);
    b_row[s] = a.rhs + (row >> a.log2_N0) * a.rhs_stride_bytes + (row & (N0 - 1)) * a.rhs_rb;
  }

  acc_t acc[AM][BN];
#pragma unroll
  for (int i = 0; i < AM; ++i)
#pragma unroll
    for (int j = 0; j < BN; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

  uint4 a_next[A_PER_THREAD], b_next[B_PER_THREAD];
  auto fetch = [&](int kc) {
#pragma unroll
    for (int s = 0; s < A_PER_THREAD; ++s) {
      const int p = tid + 256 * s;
      if (A_PIECES % 256 == 0 || p < A_PIECES)
        a_next[s] = load_piece<G, false>(a_row[s], lhs_kstep, a.lhs_rb, a.log2_lhs_rb, a.K, kc,
                                         (p >> 4) & 3);
    }
#pragma unroll
    for (int s = 0; s < B_PER_THREAD; ++s) {
      const int p = tid + 256 * s;
      if (B_PIECES % 256 == 0 || p < B_PIECES)
        b_next[s] = load_piece<G, RHS_I4>(b_row[s], rhs_kstep, a.rhs_rb, a.log2_rhs_rb, a.K, kc,
                                          (p >> 4) & 3);
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int s = 0; s < A_PER_THREAD; ++s) {
      const int p = tid + 256 * s;
      if (A_PIECES % 256 == 0 || p < A_PIECES) lds_a[stage][p] = a_next[s];
    }
#pragma unroll
    for (int s = 0; s < B_PER_THREAD; ++s) {
      const int p = tid + 256 * s;
      if (B_PIECES % 256 == 0 || p < B_PIECES) lds_b[stage][p] = b_next[s];
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();

  for (int kc = 0; kc < a.chunks; ++kc) {
    const int stage = kc & 1;
    if (kc + 1 < a.chunks) fetch(kc + 1);

    const uint4* frag_a = &lds_a[stage][(wave_m * AM) * 64 + lane];
    const uint4* frag_b = &lds_b[stage][(wave_n * BN) * 64 + lane];
    uint4 bf[BN];
#pragma unroll
    for (int j = 0; j < BN; ++j) bf[j] = frag_b[j * 64];
#pragma unroll
    for (int i = 0; i < AM; ++i) {
      const uint4 af = frag_a[i * 64];
#pragma unroll
      for (int j = 0; j < BN; ++j) acc[i][j] = mfma<KIND>(bf[j], af, acc[i][j]);
    }

    if (kc + 1 < a.chunks) stash(stage ^ 1);
    __syncthreads();
  }

  // Epilogue. Lane l holds, for fragment (i, j): lhs row 16*i + (l & 15) and
  // rhs rows 16*j + 4*(l >> 4) + {0,1,2,3} of the wavefront's sub-block.
  const int64_t row0 = (int64_t)tile_row * BLOCK_ROWS + wave_m * (16 * AM) + (lane & 15);
  const int64_t col0 = (int64_t)tile_col * BLOCK_COLS + wave_n * (16 * BN) + 4 * (lane >> 4);
  const int64_t tile_elems = (int64_t)M0 * N0;
#pragma unroll
  for (int i = 0; i < AM; ++i) {
    const int64_t row = row0 + 16 * i;
    if (row >= total_rows) continue;
    acc_t* out_row = (acc_t*)nullptr;
    const int64_t row_off = (row >> a.log2_M0) * a.out_stride0 + ((row & (M0 - 1)) << a.log2_N0);
#pragma unroll
    for (int j = 0; j < BN; ++j) {
      const int64_t col = col0 + 16 * j;
      if (col >= total_cols) continue;
      out_row = (acc_t*)(a.out + 4 * (row_off + (col >> a.log2_N0) * tile_elems + (col & (N0 - 1))));
      acc_t v = acc[i][j];
      if constexpr (RHS_I4) v = v >> 4;
      if (a.accumulate) v += *out_row;
      *out_row = v;
    }
  }
}

int log2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int l = 0;
  while ((1ll << l) < v) ++l;
  return l;
}

struct Plan {
  int kind;
  bool rhs_i4;
  int gather;  // 16 or 4
  MfmaArgs args;
};

// Fills `plan` if the problem is covered. With `probe_only` only type and tile
// shape are looked at.
bool make_plan(const Mmt4dArgs& a, bool probe_only, Plan* plan) {
  int kind, elem_bytes;
  bool i4 = false;
  switch (a.flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: kind = kI8; elem_bytes = 1; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: kind = kI8; elem_bytes = 1; i4 = true; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: kind = kF16; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: kind = kBF16; elem_bytes = 2; break;
    default: return false;
  }
  const int lm0 = log2_exact(a.M0), ln0 = log2_exact(a.N0);
  if (lm0 < 0 || ln0 < 0 || a.M0 > 16 || a.N0 > 16 || a.N0 < 4) return false;
  const int lhs_rb = a.K0 * elem_bytes;
  const int rhs_rb = i4 ? a.K0 / 2 : lhs_rb;
  const int llrb = log2_exact(lhs_rb), lrrb = log2_exact(rhs_rb);
  if (llrb < 0 || lrrb < 0) return false;
  int gather;
  if (i4) {
    if (lhs_rb < 16 || rhs_rb < 8) return false;
    gather = 16;
  } else if (lhs_rb >= 16) {
    gather = 16;
  } else if (lhs_rb == 4) {
    gather = 4;
  } else {
    return false;
  }
  plan->kind = kind;
  plan->rhs_i4 = i4;
  plan->gather = gather;
  if (probe_only) return true;

  // Alignment of every vector access the kernel makes.
  const int lhs_align = gather == 16 ? 16 : 4;
  const int rhs_align = i4 ? 8 : lhs_align;
  const int64_t lhs_stride_bytes = a.lhs_stride0 * elem_bytes;
  const int64_t rhs_stride_bytes = i4 ? a.rhs_stride0 / 2 : a.rhs_stride0 * elem_bytes;
  if (((uintptr_t)a.lhs % lhs_align) || (a.M > 1 && lhs_stride_bytes % lhs_align)) return false;
  if (((uintptr_t)a.rhs % rhs_align) || (a.N > 1 && rhs_stride_bytes % rhs_align)) return false;
  if (((uintptr_t)a.out % 16) || (a.M > 1 && a.out_stride0 % 4)) return false;
  // 16x-scaled int4 accumulation must not overflow int32.
  if (i4 && (int64_t)a.K * a.K0 >= 131072) return false;
  // K == 0 (zero fill) is left to the generic kernel.
  if (a.K == 0) return false;

  MfmaArgs& m = plan->args;
  m.lhs = a.lhs; m.rhs = a.rhs; m.out = a.out;
  m.lhs_stride_bytes = lhs_stride_bytes;
  m.rhs_stride_bytes = rhs_stride_bytes;
  m.out_stride0 = a.out_stride0;
  m.M = (int32_t)a.M; m.N = (int32_t)a.N; m.K = (int32_t)a.K;
  m.log2_M0 = lm0; m.log2_N0 = ln0;
  m.lhs_rb = lhs_rb; m.rhs_rb = rhs_rb;
  m.log2_lhs_rb = llrb; m.log2_rhs_rb = lrrb;
  m.chunks = (int32_t)(((int64_t)a.K * lhs_rb + 63) / 64);
  m.accumulate = (a.flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) ? 1 : 0;
  return true;
}

template <int KIND, bool RHS_I4, int G, int AM, int BN>
hipError_t launch_tile(MfmaArgs m, hipStream_t stream) {
  const int64_t rows = (int64_t)m.M << m.log2_M0, cols = (int64_t)m.N << m.log2_N0;
  m.tile_rows = (int32_t)((rows + 32 * AM - 1) / (32 * AM));
  m.tile_cols = (int32_t)((cols + 32 * BN - 1) / (32 * BN));
  const int64_t tiles = (int64_t)m.tile_rows * m.tile_cols;
  const unsigned grid = (unsigned)(((tiles + 7) / 8) * 8);
  hipLaunchKernelGGL((mmt4d_mfma_kernel<KIND, RHS_I4, G, AM, BN>), dim3(grid), dim3(256), 0, stream, m);
  return hipGetLastError();
}

// Picks the largest block tile that still gives every compute unit work.
template <int KIND, bool RHS_I4, int G>
hipError_t launch_variant(const MfmaArgs& m, hipStream_t stream, const char** name) {
  const int64_t rows = (int64_t)m.M << m.log2_M0, cols = (int64_t)m.N << m.log2_N0;
  auto tiles = [&](int br, int bc) { return ((rows + br - 1) / br) * ((cols + bc - 1) / bc); };
  if (tiles(256, 256) >= 200) {
    *name = "mmt4d_mfma_256x256";
    return launch_tile<KIND, RHS_I4, G, 8, 8>(m, stream);
  }
  if (tiles(128, 128) >= 200 || (rows > 64 && cols > 64)) {
    *name = "mmt4d_mfma_128x128";
    return launch_tile<KIND, RHS_I4, G, 4, 4>(m, stream);
  }
  *name = "mmt4d_mfma_64x64";
  return launch_tile<KIND, RHS_I4, G, 2, 2>(m, stream);
}

hipError_t launch_mfma(const Mmt4dArgs& a, hipStream_t stream, const char** name) {
  Plan plan;
  if (!make_plan(a, false, &plan)) return hipErrorInvalidValue;
  const MfmaArgs& m = plan.args;
  if (plan.rhs_i4) return launch_variant<kI8, true, 16>(m, stream, name);
  if (plan.kind == kI8)
    return plan.gather == 16 ? launch_variant<kI8, false, 16>(m, stream, name)
                             : launch_variant<kI8, false, 4>(m, stream, name);
  if (plan.kind == kF16)
    return plan.gather == 16 ? launch_variant<kF16, false, 16>(m, stream, name)
                             : launch_variant<kF16, false, 4>(m, stream, name);
  return plan.gather == 16 ? launch_variant<kBF16, false, 16>(m, stream, name)
                           : launch_variant<kBF16, false, 4>(m, stream, name);
}

Mmt4dLauncher select_common(const Mmt4dArgs& a, bool probe_only, uint32_t type_a, uint32_t type_b) {
  const uint32_t t = a.flags & IREE_UK_FLAG_MMT4D_TYPE_MASK;
  if (t != type_a && t != type_b) return nullptr;
  Plan plan;
  return make_plan(a, probe_only, &plan) ? launch_mfma : nullptr;
}

}  // namespace

Mmt4dLauncher select_mmt4d_i8_mfma(const Mmt4dArgs& a, bool probe_only) {
  return select_common(a, probe_only, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32);
}
Mmt4dLauncher select_mmt4d_f16_mfma(const Mmt4dArgs& a, bool probe_only) {
  return select_common(a, probe_only, IREE_UK_FLAG_MMT4D_TYPE_F16F16F32,
                       IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32);
}
Mmt4dLauncher select_mmt4d_s8s4_mfma(const Mmt4dArgs& a, bool probe_only) {
  return select_common(a, probe_only, IREE_UK_FLAG_MMT4D_TYPE_S8S4S32, IREE_UK_FLAG_MMT4D_TYPE_S8S4S32);
}

}  // namespace uk
