// MFMA mmt4d for gfx950: s8s8s32, s8s4s32, f16f16f32 and bf16bf16f32.
//
// One workgroup of 256 threads (4 wavefronts in a 2x2 arrangement) computes a
// block of (64*AM) lhs rows x (64*BN) rhs rows of the logical matrix; each
// wavefront owns a (32*AM) x (32*BN) sub-block as AM x BN accumulator
// fragments of one 32x32 MFMA each (v_mfma_i32_32x32x32_i8,
// v_mfma_f32_32x32x16_f16/bf16: a single wavefront per SIMD keeps the matrix
// pipe busy with these, which it cannot with the 16x16 shapes). The K dimension
// is walked in chunks of 64 BYTES per operand row (64 int8 or 32 f16/bf16
// values = two MFMA K-steps).
//
// Two kernels share this tiling and the epilogue:
//   mmt4d_mfma_direct_kernel (the fast path): operands go global memory ->
//     LDS directly, 16 contiguous bytes per lane, through a ring of LDS stages
//     filled several chunks ahead; needs 16-byte aligned operand rows and at
//     least one full chunk of K (a K that ends inside a chunk is handled by
//     overlapping the last chunk with the one before it).
//   mmt4d_mfma_kernel (everything else the plan admits: 4-byte aligned
//     operands, narrow tiles, less than a chunk of K, an int4 rhs whose K ends
//     inside a chunk): global -> registers (issued two chunks
//     ahead) -> LDS -> registers (read one chunk ahead) -> MFMA.
// In both, LDS holds the operands fragment-major, so that a wavefront fetches
// a 32-row x 32-byte MFMA operand with conflict-free reads that are linear in
// the lane number.
//
// Operand layouts. An mmt4d operand row (one i0 of one tile) is not contiguous
// in memory: its K0 values of consecutive k are M0*K0 elements apart
// (mmt4d_tile_generic.c:70-71). With RB = bytes of one (k, i0) row piece:
//   RB multiple of 16: a lane's 16 operand bytes are contiguous in memory;
//   RB == 4 (the 8x8x4 int8 tiles): a lane's 16 bytes come from 4 different k
//     steps. K is permuted inside a chunk, identically for lhs and rhs, which
//     leaves every integer sum unchanged (and reorders a float sum).
// The int4 rhs of s8s4s32 is widened in registers: nibble n becomes the int8
// value 16*n (sign in bit 7, no sign-extension step), the accumulators
// therefore hold 16x the result and are shifted right by 4 at the end, which
// is exact while 16*128*8*depth < 2^31.
//
// The MFMA is issued with the rhs fragment as its row operand and the lhs
// fragment as its column operand, so a lane ends up with 4 consecutive j0 of
// one output row: one 128-bit store per fragment into the [M0][N0] tile.
#ifndef IREE_AMD_CSRC_MMT4D_MFMA_KERNELS_H_
#define IREE_AMD_CSRC_MMT4D_MFMA_KERNELS_H_

#include <type_traits>

#include "uk_device.h"
#include "uk_internal.h"

namespace uk {

enum MfmaKind { kI8 = 0, kF16 = 1, kBF16 = 2, kF32 = 3 };

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

// One entry per translation unit of kernel instantiations (they are split by
// type so that they compile side by side). `gather` is 16 or 4 (bytes of one
// contiguous row piece that a lane's 16 operand bytes are made of); `narrow`:
// the output is the 16-bit type of the operands (one rounding at the end).
hipError_t launch_mfma_i8(const MfmaArgs& m, int gather, bool rhs_i4, hipStream_t stream, const char** name);
hipError_t launch_mfma_f16(const MfmaArgs& m, int gather, bool narrow, hipStream_t stream, const char** name);
hipError_t launch_mfma_bf16(const MfmaArgs& m, int gather, bool narrow, hipStream_t stream, const char** name);
hipError_t launch_mfma_f32(const MfmaArgs& m, int gather, hipStream_t stream, const char** name);
hipError_t launch_mfma_f16_narrow(const MfmaArgs& m, int gather, hipStream_t stream, const char** name);
hipError_t launch_mfma_bf16_narrow(const MfmaArgs& m, int gather, hipStream_t stream, const char** name);

// Whether the direct-to-LDS kernel covers the problem with row pieces of
// `gather` bytes (2 and 8 have no other MFMA kernel).
bool mfma_direct_covers(const MfmaArgs& m, int gather, bool rhs_i4);

#ifdef UK_MFMA_KERNEL_BODIES
namespace {

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v16i32 __attribute__((ext_vector_type(16)));
typedef float v16f32 __attribute__((ext_vector_type(16)));
typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf16 __attribute__((ext_vector_type(8)));

template <int KIND>
struct AccType { typedef v16i32 type; typedef int scalar; };
template <> struct AccType<kF16> { typedef v16f32 type; typedef float scalar; };
template <> struct AccType<kBF16> { typedef v16f32 type; typedef float scalar; };
template <> struct AccType<kF32> { typedef v16f32 type; typedef float scalar; };

// MFMAs that one pair of 16-byte operand fragments feeds: f32 has only the
// 32x32x2 shape (one float per lane), so its 4 floats take 4 instructions.
template <int KIND> struct SubSteps { static constexpr int value = KIND == kF32 ? 4 : 1; };

// Sub-step `sub` (< SubSteps<KIND>::value) of the product of two 16-byte
// operand fragments.
template <int KIND>
__device__ __forceinline__ typename AccType<KIND>::type mfma(uint4 row_operand, uint4 col_operand,
                                                             typename AccType<KIND>::type acc, int sub = 0) {
  if constexpr (KIND == kI8) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(v4i32, row_operand),
                                                 __builtin_bit_cast(v4i32, col_operand), acc, 0, 0, 0);
  } else if constexpr (KIND == kF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8f16, row_operand),
                                                  __builtin_bit_cast(v8f16, col_operand), acc, 0, 0, 0);
  } else if constexpr (KIND == kBF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf16, row_operand),
                                                   __builtin_bit_cast(v8bf16, col_operand), acc, 0, 0, 0);
  } else {
    const uint32_t r = sub == 0 ? row_operand.x : sub == 1 ? row_operand.y : sub == 2 ? row_operand.z : row_operand.w;
    const uint32_t c = sub == 0 ? col_operand.x : sub == 1 ? col_operand.y : sub == 2 ? col_operand.z : col_operand.w;
    return __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(r), __uint_as_float(c), acc, 0, 0, 0);
  }
}

// All sub-steps of one fragment pair.
template <int KIND>
__device__ __forceinline__ typename AccType<KIND>::type mfma_all(uint4 row_operand, uint4 col_operand,
                                                                 typename AccType<KIND>::type acc) {
#pragma unroll
  for (int sub = 0; sub < SubSteps<KIND>::value; ++sub) acc = mfma<KIND>(row_operand, col_operand, acc, sub);
  return acc;
}

// 16 int4 values (two dwords, element 2b in the low nibble of byte b) to 16
// int8 values equal to 16x the signed nibbles, in element order: the even and
// the odd elements of a dword are isolated in the high nibbles of two dwords,
// whose bytes are then interleaved.
__device__ __forceinline__ uint4 widen_i4_times16(uint2 w) {
  const uint32_t even0 = (w.x << 4) & 0xF0F0F0F0u, odd0 = w.x & 0xF0F0F0F0u;
  const uint32_t even1 = (w.y << 4) & 0xF0F0F0F0u, odd1 = w.y & 0xF0F0F0F0u;
  uint4 r;
  r.x = __builtin_amdgcn_perm(odd0, even0, 0x05010400u);
  r.y = __builtin_amdgcn_perm(odd0, even0, 0x07030602u);
  r.z = __builtin_amdgcn_perm(odd1, even1, 0x05010400u);
  r.w = __builtin_amdgcn_perm(odd1, even1, 0x07030602u);
  return r;
}

// k step (relative to its chunk's first) that the 16-byte column `c` of an
// operand row starts at.
template <int G, bool I4>
__device__ __forceinline__ int32_t piece_kstep(int c, int32_t log2_rb) {
  if constexpr (I4) return (8 * c) >> log2_rb;
  if constexpr (G == 16) return (16 * c) >> log2_rb;
  return 4 * c;
}

// One 16-byte operand piece for LDS. `p` points at the piece's first byte for
// the current chunk. G is the contiguous run in memory: 16 (one vector load),
// 4 (gather one dword from each of 4 consecutive k steps, `kstep` bytes apart)
// or, for I4, 8 bytes of nibbles widened to 16. With CHECKED, parts whose k
// step `k1 (+d)` is not below K read as zero.
template <int G, bool I4, bool CHECKED>
__device__ __forceinline__ uint4 load_piece(const uint8_t* p, int64_t kstep, int32_t k1, int32_t K) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if constexpr (I4) {
    if (!CHECKED || k1 < K) v = widen_i4_times16(*(const uint2*)p);
  } else if constexpr (G == 16) {
    if (!CHECKED || k1 < K) v = *(const uint4*)p;
  } else {
    if (!CHECKED || k1 + 0 < K) v.x = *(const uint32_t*)(p);
    if (!CHECKED || k1 + 1 < K) v.y = *(const uint32_t*)(p + kstep);
    if (!CHECKED || k1 + 2 < K) v.z = *(const uint32_t*)(p + 2 * kstep);
    if (!CHECKED || k1 + 3 < K) v.w = *(const uint32_t*)(p + 3 * kstep);
  }
  return v;
}

// Workgroup -> block tile. Consecutive workgroup ids go to different XCDs (8 of
// them, each with its own L2), so ids are first regrouped so that one XCD works
// on a contiguous range of tiles, then that range is walked in bands of 4 tile
// rows so that neighbours share lhs and rhs panels. False: nothing to do.
__device__ __forceinline__ bool locate_block(const MfmaArgs& a, int* tile_row, int* tile_col) {
  const int total_tiles = a.tile_rows * a.tile_cols;
  const int per_xcd = (total_tiles + 7) >> 3;
  const int linear = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (linear >= total_tiles) return false;
  constexpr int BAND = 4;
  const int band = linear / (BAND * a.tile_cols);
  const int band_first = band * BAND;
  const int band_rows = min(a.tile_rows - band_first, BAND);
  const int in_band = linear - band * BAND * a.tile_cols;
  *tile_row = band_first + in_band % band_rows;
  *tile_col = in_band / band_rows;
  return true;
}

// Writes one wavefront's accumulators. Lane l holds, for fragment (i, j): lhs
// row 32*i + (l & 31) and, in accumulator registers 4*q .. 4*q+3, rhs rows
// 32*j + 8*q + 4*(l >> 5) + {0..3} of the wavefront's sub-block, which starts at
// (wave_row, wave_col) of the logical matrix: four consecutive j0 of one output
// row, one 128-bit store (64-bit for a NARROW, i.e. 16-bit, output, rounded to
// nearest even the way common.h:701-770 does). When accumulating, a fragment's
// loads are issued before its first add, so their latencies overlap.
//
// PAIR_A / PAIR_B: the fragments of that operand were fed in interleaved pairs
// (2-byte row pieces, see the direct-to-LDS kernel): lane row r of fragments
// 2p and 2p + 1 is row 64*p + 2*r resp. 64*p + 2*r + 1 of the sub-block. For
// the columns this means that accumulators e and e + 1 of fragment 2p and of
// fragment 2p + 1 together are four consecutive j0, so two fragments are
// written at a time.
template <int KIND, bool RHS_I4, bool NARROW, int AM, int BN, bool PAIR_A = false, bool PAIR_B = false>
__device__ __forceinline__ void store_block(const MfmaArgs& a, typename AccType<KIND>::type (&acc)[AM][BN],
                                            int64_t wave_row, int64_t wave_col, int lane) {
  typedef typename AccType<KIND>::scalar scalar_t;
  typedef scalar_t quad_t __attribute__((ext_vector_type(4)));
  typedef typename std::conditional<NARROW, uint2, quad_t>::type stored_t;
  constexpr int OUT_BYTES = NARROW ? 2 : 4;
  constexpr int EBITS = KIND == kF16 ? 5 : 8;
  static_assert(!NARROW || KIND == kF16 || KIND == kBF16, "16-bit outputs are floats");
  const int32_t M0 = 1 << a.log2_M0, N0 = 1 << a.log2_N0;
  const int64_t total_rows = (int64_t)a.M << a.log2_M0;
  const int64_t total_cols = (int64_t)a.N << a.log2_N0;
  static_assert((!PAIR_A || AM % 2 == 0) && (!PAIR_B || BN % 2 == 0), "pairs of fragments");
  constexpr int JS = PAIR_B ? 2 : 1;  // rhs fragments written together
  // Byte offset of quad (j, q) from the sub-block's first column tile (the same
  // for every row, and small) and whether the quad lies inside the matrix.
  const int64_t first_col_tile = wave_col >> a.log2_N0;
  uint8_t* wave_out = a.out + OUT_BYTES * (first_col_tile << (a.log2_M0 + a.log2_N0));
  uint32_t col_off[BN][4];
  uint32_t col_inside = 0;
#pragma unroll
  for (int j = 0; j < BN; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int64_t col = PAIR_B ? wave_col + 8 * (lane >> 5) + 64 * (j >> 1) + 16 * q + 4 * (j & 1)
                                 : wave_col + 4 * (lane >> 5) + 32 * j + 8 * q;
      col_off[j][q] = (uint32_t)(OUT_BYTES * ((((col >> a.log2_N0) - first_col_tile) << (a.log2_M0 + a.log2_N0)) +
                                              (col & (N0 - 1))));
      if (col < total_cols) col_inside |= 1u << (4 * j + q);
    }
  auto to_float = [](stored_t w) -> quad_t {
    if constexpr (NARROW) {
      return quad_t{widen16<EBITS>((uint16_t)w.x), widen16<EBITS>((uint16_t)(w.x >> 16)),
                    widen16<EBITS>((uint16_t)w.y), widen16<EBITS>((uint16_t)(w.y >> 16))};
    } else {
      return w;
    }
  };
  auto to_stored = [](quad_t v) -> stored_t {
    if constexpr (NARROW) {
      return make_uint2((uint32_t)narrow16<EBITS>(v.x) | ((uint32_t)narrow16<EBITS>(v.y) << 16),
                        (uint32_t)narrow16<EBITS>(v.z) | ((uint32_t)narrow16<EBITS>(v.w) << 16));
    } else {
      return v;
    }
  };
  // With paired lhs fragments, fragments 2p and 2p + 1 hold the even and the odd
  // rows of the same 64: they are written together, so that the stores which
  // make up a cache line of the output (two rows of a 16-wide int32 tile, say)
  // follow each other directly. Written a fragment at a time, each line was
  // sent to memory in pieces (2.6x the output size in write traffic).
  constexpr int IS = PAIR_A ? 2 : 1;  // lhs fragments written together
#pragma unroll
  for (int i0 = 0; i0 < AM; i0 += IS) {
    bool row_inside[IS];
    uint8_t* row_out[IS];
#pragma unroll
    for (int t = 0; t < IS; ++t) {
      const int i = i0 + t;
      const int64_t this_row =
          wave_row + (PAIR_A ? 64 * (i >> 1) + 2 * (lane & 31) + (i & 1) : 32 * i + (lane & 31));
      const int64_t row = min(this_row, total_rows - 1);
      row_inside[t] = this_row < total_rows;
      row_out[t] = wave_out + OUT_BYTES * ((row >> a.log2_M0) * a.out_stride0 + ((row & (M0 - 1)) << a.log2_N0));
    }
#pragma unroll
    for (int j0 = 0; j0 < BN; j0 += JS) {
      // Pin the fragment(s) where they are until their turn: left alone, the
      // compiler moves all 256 accumulators to ordinary registers right after
      // the main loop, and there are not that many.
      typename AccType<KIND>::type frag[IS][JS];
#pragma unroll
      for (int t = 0; t < IS; ++t)
#pragma unroll
        for (int s = 0; s < JS; ++s) {
          frag[t][s] = acc[i0 + t][j0 + s];
          asm volatile("" : "+a"(frag[t][s]));
        }
      quad_t v[IS][JS][4];
#pragma unroll
      for (int t = 0; t < IS; ++t)
#pragma unroll
        for (int s = 0; s < JS; ++s)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if constexpr (PAIR_B) {
              v[t][s][q] = quad_t{frag[t][0][4 * q + 2 * s], frag[t][1][4 * q + 2 * s], frag[t][0][4 * q + 2 * s + 1],
                                  frag[t][1][4 * q + 2 * s + 1]};
            } else {
              v[t][s][q] = quad_t{frag[t][s][4 * q], frag[t][s][4 * q + 1], frag[t][s][4 * q + 2], frag[t][s][4 * q + 3]};
            }
            if constexpr (RHS_I4) v[t][s][q] = v[t][s][q] >> 4;
          }
      if (a.accumulate) {
        quad_t old[IS][JS][4];
#pragma unroll
        for (int t = 0; t < IS; ++t)
#pragma unroll
          for (int s = 0; s < JS; ++s)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              old[t][s][q] = quad_t{0, 0, 0, 0};
              if (row_inside[t] && (col_inside >> (4 * (j0 + s) + q) & 1))
                old[t][s][q] = to_float(*(const stored_t*)(row_out[t] + col_off[j0 + s][q]));
            }
#pragma unroll
        for (int t = 0; t < IS; ++t)
#pragma unroll
          for (int s = 0; s < JS; ++s)
#pragma unroll
            for (int q = 0; q < 4; ++q) v[t][s][q] += old[t][s][q];
      }
      // Store order: the pieces of one row right after each other (with paired
      // rhs fragments v[.][0][q] and v[.][1][q] are the two halves of 32
      // contiguous bytes), then the neighbouring row of the other lhs fragment.
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int t = 0; t < IS; ++t)
#pragma unroll
          for (int s = 0; s < JS; ++s)
            if (row_inside[t] && (col_inside >> (4 * (j0 + s) + q) & 1))
              *(stored_t*)(row_out[t] + col_off[j0 + s][q]) = to_stored(v[t][s][q]);
      // Keep the fragments apart: hoisting all address arithmetic and
      // accumulator reads to the top costs more registers than there are.
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

template <int KIND, bool RHS_I4, bool NARROW, int G, int AM, int BN, int MIN_BLOCKS, bool TAIL>
__global__ __launch_bounds__(256, MIN_BLOCKS) void mmt4d_mfma_kernel(const MfmaArgs a) {
  typedef typename AccType<KIND>::type acc_t;
  constexpr int BLOCK_ROWS = 64 * AM;  // lhs rows per workgroup
  constexpr int BLOCK_COLS = 64 * BN;  // rhs rows per workgroup
  constexpr int A_PIECES = BLOCK_ROWS * 4;  // 16-byte pieces per chunk
  constexpr int B_PIECES = BLOCK_COLS * 4;
  constexpr int A_PER_THREAD = (A_PIECES + 255) / 256;
  constexpr int B_PER_THREAD = (B_PIECES + 255) / 256;
  static_assert(A_PIECES % 256 == 0 && B_PIECES % 256 == 0, "block tile too small");
  __shared__ uint4 lds_a[2][A_PIECES];
  __shared__ uint4 lds_b[2][B_PIECES];

  int tile_row, tile_col;
  if (!locate_block(a, &tile_row, &tile_col)) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;

  const int32_t M0 = 1 << a.log2_M0, N0 = 1 << a.log2_N0;
  const int64_t total_rows = (int64_t)a.M << a.log2_M0;
  const int64_t total_cols = (int64_t)a.N << a.log2_N0;
  const int64_t lhs_kstep = (int64_t)a.lhs_rb << a.log2_M0;
  const int64_t rhs_kstep = (int64_t)a.rhs_rb << a.log2_N0;
  // k steps covered by one chunk (64 bytes of an lhs row).
  const int32_t ksteps_per_chunk = 64 >> a.log2_lhs_rb;

  // Workgroup-uniform bases and 32-bit per-piece offsets from them. Piece
  // p = tid + 256*s lands at LDS slot p: fragment (p >> 7), 16-byte column
  // (p >> 5) & 3, row p & 31 of the fragment (column c is K-step c >> 1, lane
  // half c & 1 of the MFMA operand). Rows past the end of the matrix
  // are redirected to its last row: their products are computed, never stored.
  const int64_t first_row = (int64_t)tile_row * BLOCK_ROWS;
  const int64_t first_col = (int64_t)tile_col * BLOCK_COLS;
  const uint8_t* lhs_base = a.lhs + (first_row >> a.log2_M0) * a.lhs_stride_bytes;
  const uint8_t* rhs_base = a.rhs + (first_col >> a.log2_N0) * a.rhs_stride_bytes;
  uint32_t a_off[A_PER_THREAD], b_off[B_PER_THREAD];
#pragma unroll
  for (int s = 0; s < A_PER_THREAD; ++s) {
    const int p = tid + 256 * s;
    const int c = (p >> 5) & 3;
    const int64_t row = min(first_row + (p >> 7) * 32 + (p & 31), total_rows - 1);
    const int64_t tile = (row >> a.log2_M0) - (first_row >> a.log2_M0);
    const int32_t col_byte = G == 16 ? 16 * c : 0;
    const int32_t k1 = piece_kstep<G, false>(c, a.log2_lhs_rb);
    a_off[s] = (uint32_t)(tile * a.lhs_stride_bytes + (row & (M0 - 1)) * a.lhs_rb +
                          k1 * lhs_kstep + (col_byte & (a.lhs_rb - 1)));
  }
#pragma unroll
  for (int s = 0; s < B_PER_THREAD; ++s) {
    const int p = tid + 256 * s;
    const int c = (p >> 5) & 3;
    const int64_t row = min(first_col + (p >> 7) * 32 + (p & 31), total_cols - 1);
    const int64_t tile = (row >> a.log2_N0) - (first_col >> a.log2_N0);
    const int32_t col_byte = RHS_I4 ? 8 * c : (G == 16 ? 16 * c : 0);
    const int32_t k1 = piece_kstep<G, RHS_I4>(c, a.log2_rhs_rb);
    b_off[s] = (uint32_t)(tile * a.rhs_stride_bytes + (row & (N0 - 1)) * a.rhs_rb +
                          k1 * rhs_kstep + (col_byte & (a.rhs_rb - 1)));
  }

  acc_t acc[AM][BN];
#pragma unroll
  for (int i = 0; i < AM; ++i)
#pragma unroll
    for (int j = 0; j < BN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  // Global -> register prefetch of one chunk, two chunks deep: while chunk kc
  // is multiplied, chunk kc + 1 moves from registers to LDS and chunks kc + 2
  // and kc + 3 are in flight from memory (a load takes longer than one chunk
  // of MFMAs, so a single chunk of lookahead would stall every iteration).
  uint4 a_pre[2][A_PER_THREAD], b_pre[2][B_PER_THREAD];
  auto fetch = [&](int kc, uint4* a_next, uint4* b_next) {
    const int32_t k1_0 = kc * ksteps_per_chunk;
    const uint8_t* la = lhs_base + (int64_t)k1_0 * lhs_kstep;
    const uint8_t* lb = rhs_base + (int64_t)k1_0 * rhs_kstep;
#pragma unroll
    for (int s = 0; s < A_PER_THREAD; ++s)
      a_next[s] = load_piece<G, false, false>(la + a_off[s], lhs_kstep, 0, 0);
#pragma unroll
    for (int s = 0; s < B_PER_THREAD; ++s)
      b_next[s] = load_piece<G, RHS_I4, false>(lb + b_off[s], rhs_kstep, 0, 0);
  };
  // Same for a chunk that K ends inside of: missing k steps read as zero.
  auto fetch_checked = [&](int kc, uint4* a_next, uint4* b_next) {
    const int32_t k1_0 = kc * ksteps_per_chunk;
    const uint8_t* la = lhs_base + (int64_t)k1_0 * lhs_kstep;
    const uint8_t* lb = rhs_base + (int64_t)k1_0 * rhs_kstep;
#pragma unroll
    for (int s = 0; s < A_PER_THREAD; ++s)
      a_next[s] = load_piece<G, false, true>(
          la + a_off[s], lhs_kstep,
          k1_0 + piece_kstep<G, false>(((tid + 256 * s) >> 5) & 3, a.log2_lhs_rb), a.K);
#pragma unroll
    for (int s = 0; s < B_PER_THREAD; ++s)
      b_next[s] = load_piece<G, RHS_I4, true>(
          lb + b_off[s], rhs_kstep,
          k1_0 + piece_kstep<G, RHS_I4>(((tid + 256 * s) >> 5) & 3, a.log2_rhs_rb), a.K);
  };
  auto stash = [&](int stage, const uint4* a_next, const uint4* b_next) {
#pragma unroll
    for (int s = 0; s < A_PER_THREAD; ++s) lds_a[stage][tid + 256 * s] = a_next[s];
#pragma unroll
    for (int s = 0; s < B_PER_THREAD; ++s) lds_b[stage][tid + 256 * s] = b_next[s];
  };

  // Fragment registers, double buffered: while the MFMAs of chunk kc run from
  // one set, the fragments of chunk kc + 1 are read from LDS into the other.
  // The loop is unrolled by two so the sets swap roles without copies, and its
  // body is branch-free (the prefetch index is clamped instead) so that LDS
  // reads, global loads and MFMAs can be scheduled against each other.
  uint4 pa[AM][2], pb[BN][2], qa[AM][2], qb[BN][2];
  auto read_frags = [&](int stage, uint4 (*fa)[2], uint4 (*fb)[2]) {
    const uint4* frag_a = &lds_a[stage][(wave_m * AM) * 128 + lane];
    const uint4* frag_b = &lds_b[stage][(wave_n * BN) * 128 + lane];
    // K-step 0 first: it is what the next step's first MFMAs consume.
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
      for (int j = 0; j < BN; ++j) fb[j][kk] = frag_b[j * 128 + kk * 64];
#pragma unroll
      for (int i = 0; i < AM; ++i) fa[i][kk] = frag_a[i * 128 + kk * 64];
    }
  };
  auto multiply = [&](const uint4 (*fa)[2], const uint4 (*fb)[2], int kk) {
#pragma unroll
    for (int i = 0; i < AM; ++i)
#pragma unroll
      for (int j = 0; j < BN; ++j) acc[i][j] = mfma_all<KIND>(fb[j][kk], fa[i][kk], acc[i][j]);
  };
  // Chunks that lie entirely inside K run through the pipeline; a trailing
  // partial chunk is handled after it, unpipelined.
  const int full_chunks = a.K / ksteps_per_chunk;
  const int last_chunk = full_chunks - 1;
  // One pipeline step for chunk kc, whose fragments are in `cur`:
  //   registers(kc + 1) -> LDS stage, first half of the MFMAs (covers the LDS
  //   write latency), barrier, global loads of chunk kc + 3 into the register
  //   set just freed, LDS reads of the fragments of chunk kc + 1, second half
  //   of the MFMAs (covers the LDS read latency). Prefetch indices are clamped
  //   to the last full chunk, so the body is branch-free.
  auto step = [&](int kc, int stage, const uint4 (*cur_a)[2], const uint4 (*cur_b)[2],
                  uint4 (*nxt_a)[2], uint4 (*nxt_b)[2]) {
    // A wavefront issues in order, so memory instructions only overlap with
    // the matrix pipe if they sit between MFMAs in program order: the two
    // halves below are interleaved one MFMA at a time with the LDS writes and
    // global loads (first half) and with the LDS reads (second half).
    constexpr int MFMAS = AM * BN;  // per half
    constexpr int WRITES = A_PER_THREAD + B_PER_THREAD;
    constexpr int LOADS = (G == 4 ? 4 : 1) * A_PER_THREAD + ((G == 4 && !RHS_I4) ? 4 : 1) * B_PER_THREAD;
    constexpr int READS = 2 * (AM + BN);
    stash(stage, a_pre[stage], b_pre[stage]);
    fetch(min(kc + 3, last_chunk), a_pre[stage], b_pre[stage]);
    multiply(cur_a, cur_b, 0);
#pragma unroll
    for (int m = 0; m < MFMAS; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      if (m < WRITES) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one LDS write
      constexpr int LOADS_PER = (LOADS + MFMAS - 1) / MFMAS;
      if (m * LOADS_PER < LOADS) {
        __builtin_amdgcn_sched_group_barrier(0x002, 2 * LOADS_PER, 0);  // address arithmetic
        __builtin_amdgcn_sched_group_barrier(0x020, LOADS_PER, 0);      // global loads
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_frags(stage, nxt_a, nxt_b);
    multiply(cur_a, cur_b, 1);
#pragma unroll
    for (int m = 0; m < MFMAS; ++m) {
      constexpr int READS_PER = (READS + MFMAS - 1) / MFMAS;
      if (m * READS_PER < READS) __builtin_amdgcn_sched_group_barrier(0x100, READS_PER, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  if (full_chunks > 0) {
    // Chunk c travels through register set c & 1 and LDS stage c & 1.
    fetch(0, a_pre[0], b_pre[0]);
    fetch(min(1, last_chunk), a_pre[1], b_pre[1]);
    stash(0, a_pre[0], b_pre[0]);
    fetch(min(2, last_chunk), a_pre[0], b_pre[0]);
    __syncthreads();
    read_frags(0, pa, pb);
    int kc = 0;
    for (; kc + 1 < full_chunks; kc += 2) {
      step(kc, 1, pa, pb, qa, qb);
      step(kc + 1, 0, qa, qb, pa, pb);
    }
    if (kc < full_chunks) {
      multiply(pa, pb, 0);
      multiply(pa, pb, 1);
    }
  }
  if constexpr (TAIL) {
    fetch_checked(full_chunks, a_pre[0], b_pre[0]);
    __syncthreads();  // every wavefront is done reading LDS stage 0
    stash(0, a_pre[0], b_pre[0]);
    __syncthreads();
    read_frags(0, pa, pb);
    multiply(pa, pb, 0);
    multiply(pa, pb, 1);
  }

  store_block<KIND, RHS_I4, NARROW, AM, BN>(a, acc, first_row + wave_m * (32 * AM),
                                            first_col + wave_n * (32 * BN), lane);
}

// ---------------------------------------------------------------------------
// Direct-to-LDS variant: the same block tiling, but operand pieces travel
// global memory -> LDS without passing through registers
// (global_load_lds_dwordx4: lane l of a wavefront writes its 16 bytes at
// M0 + 16*l), through a ring of 4 LDS stages filled three chunks ahead of the
// MFMAs. It needs no register prefetch buffers, no LDS writes and no
// data-dependent waits other than one counter wait per chunk. It covers the
// int8/f16/bf16 rhs (no nibble widening on the way) and K that ends on a chunk
// boundary; everything else uses the kernel above.
//
// Every load moves 16 contiguous bytes per lane, also for the 4-byte row
// pieces of e.g. the 8x8x4 int8 tiles (G == 4), where 16 contiguous bytes are
// 4 consecutive rows of one k step: there the transposition to "one row, 16
// bytes of K" happens on the way out of LDS, with four 32-bit reads per
// fragment instead of one 128-bit read, and the loads are arranged so that
// those reads are linear in the lane number (conflict-free).
//
// The loads are issued from inline assembly: the compiler cannot see that they
// write LDS, so it does not serialise the LDS reads against them; ordering is
// enforced by hand with s_waitcnt vmcnt + a workgroup barrier once per chunk.
extern __shared__ uint4 ring[];

// Measuring aid, compiled in only by the benchmark's probe library (csrc/bench/probe_mmt4d_timeline.hip):
// wavefront 0 of each of the first 256 workgroups leaves five readings of the constant-rate 100 MHz
// counter (start, main loop begins, main loop ends, last MFMA issued, stores acknowledged).
#ifdef UK_KERNEL_TIMELINE
#define UK_TIMELINE(...) __VA_ARGS__
__device__ unsigned long long uk_timeline[256 * 8];
#else
#define UK_TIMELINE(...)
#endif

// One wavefront-wide load of 64 x 16 bytes to LDS byte offset `lds_off`
// (wavefront-uniform) from `base` (uniform) + per-lane byte offset `voff`.
__device__ __forceinline__ void load_to_lds(uint32_t lds_off, uint32_t voff, const uint8_t* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_off), "v"(voff), "s"(base)
               : "memory");
}

// 8 bytes per lane from LDS, transposed within each group of 16 lanes
// (ds_read_b64_tr_b8): the 16 lanes' 8-byte chunks are taken as 8 rows of 16
// bytes (chunks 2j and 2j + 1 make row j), and lane i of the group receives
// byte i of every row. With a k-major operand ("16 matrix rows at k, then the
// same rows at k + 1, ...") lane i thus gets 8 consecutive k of matrix row i.
__device__ __forceinline__ uint2 lds_read_transposed(const uint8_t* p) {
  typedef int v2i32 __attribute__((ext_vector_type(2)));
  const v2i32 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i32*)(p));
  return make_uint2((uint32_t)v.x, (uint32_t)v.y);
}

// A wavefront-uniform pointer, said to be so: the loads above take their base from scalar registers, and whether
// the compiler keeps a uniform 64-bit address computation on the scalar unit depends on what else uses its inputs.
__device__ __forceinline__ const uint8_t* uniform_pointer(const uint8_t* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const uint8_t*)(((uint64_t)hi << 32) | lo);
}

template <int N>
__device__ __forceinline__ void wait_loads_but() {
  static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// (The 256x256 tile needs all 512 registers of a lane for one wavefront; said
// explicitly, because left to its occupancy heuristics the compiler may keep
// the accumulators in scratch memory instead.)
// STAGGER: 0 = every accumulator stored after the last MFMA; 1 = staggered tail (see below); 2 = the same for
// an accumulating call, the destination read in the tail; 3 = accumulating call with the destination read and
// added during the main loop (needs enough steps), tail as in 1.
template <int KIND, bool RHS_I4, bool NARROW, int G, int AM, int BN, int STAGES, int STAGGER = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, AM * BN >= 16 ? 1 : (AM * BN >= 4 ? 2 : 4))))
void mmt4d_mfma_direct_kernel(const MfmaArgs a) {
  typedef typename AccType<KIND>::type acc_t;
  static_assert(!RHS_I4 || (G == 16 && BN >= 2), "int4 rhs: 16-byte pieces, at least one fragment per wavefront");
  constexpr int BLOCK_ROWS = 64 * AM, BLOCK_COLS = 64 * BN;
  // 16-byte pieces per chunk: 64 bytes of K per row, 32 bytes for an int4 rhs.
  constexpr int A_PIECES = BLOCK_ROWS * 4, B_PIECES = BLOCK_COLS * (RHS_I4 ? 2 : 4);
  constexpr int STAGE_PIECES = A_PIECES + B_PIECES;
  constexpr int AHEAD = STAGES - 1;  // chunks in flight ahead of the one being multiplied
  static_assert(STAGES >= 4, "ring depth");
  // 2-byte row pieces: an operand with an even number of fragments per
  // wavefront is fed in interleaved pairs of fragments (see the layouts below).
  constexpr bool PAIR_A = G == 2 && AM % 2 == 0, PAIR_B = G == 2 && BN % 2 == 0;
  // Load instructions per wavefront and chunk (64 lanes x 16 bytes each), each
  // with its own per-lane offset.
  constexpr int A_LOADS = A_PIECES / 256, B_LOADS = B_PIECES / 256;
  constexpr int LOADS = A_LOADS + B_LOADS;
  static_assert(A_PIECES % 256 == 0 && B_PIECES % 256 == 0, "block tile too small");
  static_assert((AHEAD - 1) * LOADS <= 63, "the loads in flight must fit the 6-bit counter");

  UK_TIMELINE(const unsigned long long tl_start = __builtin_amdgcn_s_memrealtime(); unsigned long long tl_loop = 0,
              tl_loop_end = 0;)
  int tile_row, tile_col;
  if (!locate_block(a, &tile_row, &tile_col)) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 1, wave_n = wave & 1;

  const int64_t total_rows = (int64_t)a.M << a.log2_M0;
  const int64_t total_cols = (int64_t)a.N << a.log2_N0;
  const int64_t lhs_kstep = (int64_t)a.lhs_rb << a.log2_M0;
  const int64_t rhs_kstep = (int64_t)a.rhs_rb << a.log2_N0;
  const int32_t ksteps_per_chunk = 64 >> a.log2_lhs_rb;
  const int64_t lhs_chunk_bytes = ksteps_per_chunk * lhs_kstep;
  const int64_t rhs_chunk_bytes = ksteps_per_chunk * rhs_kstep;

  const int64_t first_row = (int64_t)tile_row * BLOCK_ROWS;
  const int64_t first_col = (int64_t)tile_col * BLOCK_COLS;
  const uint8_t* lhs_base = uniform_pointer(a.lhs + (first_row >> a.log2_M0) * a.lhs_stride_bytes);
  const uint8_t* rhs_base = uniform_pointer(a.rhs + (first_col >> a.log2_N0) * a.rhs_stride_bytes);

  // Load t of wavefront w fills the 16-byte LDS slots 64*m .. 64*m + 63 of its
  // operand, m = 4*t + w, lane l the slot 64*m + l.
  //   G == 16: slot p holds fragment p >> 7, rows 16*((p >> 6) & 1) + (p & 15),
  //     16-byte column c = (p >> 4) & 3 (K-step c >> 1, lane half c & 1 of the
  //     MFMA operand): one load covers 16 rows x 64 bytes, which for 64-byte row
  //     pieces is 1 KiB of contiguous memory (with "32 rows x 32 bytes" every
  //     cache line was touched by two loads: 7 % slower). Lane 32*h + r reads
  //     slot 128*f + 64*(r >> 4) + 16*(2*kk + h) + (r & 15), one 128-bit read;
  //     every group of 16 lanes reads 256 contiguous bytes: no bank conflicts.
  //     (With an int4 rhs the lhs keeps the older arrangement: slot p holds row
  //     p & 31, column slot (p >> 5) & 3, read at slot 128*f + 64*kk + lane.)
  //   G == 2, 4, 8 (bytes of a row piece; R = 16 / G rows share 16 contiguous
  //     bytes, a chunk is 64 / G k steps): slot 64*m + l holds rows R*g ..
  //     R*g + R - 1 (g = l % (2*G)) of fragment m >> 1 at k step
  //     (32/G)*(m & 1) + (16/G)*h + d of the chunk (h = (l / (2*G)) & 1,
  //     d = l / (4*G)). The G-byte element number 64*((2*f + kk)*(16/G) + d) +
  //     32*h + r of the operand is then row r of fragment f at that k step: the
  //     MFMA operand of lane 32*h + r for K-step kk is elements d = 0 .. 16/G - 1,
  //     each read linear in the lane number (4-byte pieces: two paired dword
  //     reads; 8-byte: two 64-bit reads; 2-byte: eight reads of the dword the
  //     element shares with its neighbour row, and a byte permute that picks
  //     the lane's half). K is permuted inside a chunk, identically for lhs
  //     and rhs.
  //   G == 2, fragments in pairs (an even number of them per wavefront): 16-bit
  //     reads deliver half of what the LDS can, so a lane reads dwords, i.e. two
  //     adjacent rows of one k step, and gives the low half to fragment 2p, the
  //     high half to fragment 2p + 1: row r of those fragments is row 2*r resp.
  //     2*r + 1 of the pair's 64 rows (the epilogue undoes it). Slot 64*m + l
  //     holds rows 8*g .. 8*g + 7 (g = l & 7) of pair m >> 2 at k step
  //     16*kk + 8*h + 4*(m & 1) + (l >> 4) of the chunk (kk = (m >> 1) & 1,
  //     h = (l >> 3) & 1), the same k steps per (K-step, lane half) as in the
  //     unpaired layout, so the two can be mixed between lhs and rhs. Dword
  //     64*d + 32*h + r of a (pair, K-step) is then rows 2*r, 2*r + 1 at the
  //     lane's d-th k step: eight dword reads linear in the lane number (four
  //     two-address instructions) and eight byte permutes per two fragments.
  //     (Tried: lanes arranged so that four consecutive ones load four
  //     consecutive k steps of one row group, i.e. one cache line instead of
  //     two for M0 = 16 or four for M0 = 8, with an xor spreading the row groups
  //     over the banks. The reads then need eight separate addresses: 8x8x2
  //     int8 tiles went from 114 to 100 us per 4096^3, 16x16x2 from 83 to 89.)
  //   int4 rhs: slot 64*f + 32*h + r holds nibbles 32*h .. 32*h + 31 of row r of
  //     fragment f: lane 32*h + r reads that slot once per chunk and widens its
  //     first 8 bytes for K-step 0, its last 8 for K-step 1. The lhs columns are
  //     assigned to match: (K-step kk, lane half h) gets 16-byte column kk + 2*h.
  // Rows past the end of the matrix are redirected to its last row (group):
  // their products are computed, never stored.
  auto row_offset = [&](int64_t row, int64_t last, int64_t first, int log2_t0, int64_t stride_bytes,
                        int32_t rb) -> int64_t {
    row = min(row, last);
    const int64_t tile = (row >> log2_t0) - (first >> log2_t0);
    return tile * stride_bytes + (row & ((1 << log2_t0) - 1)) * rb;
  };
  //   G == 16, lhs tiles one row tall (a row-major matrix: a row's 64 bytes of a
  //     chunk are contiguous, consecutive rows a whole row pitch apart): with the
  //     arrangement above four consecutive lanes would load from four cache
  //     lines. Here lane l of a load takes row l >> 2 of the load's 16 and the
  //     16-byte column (l & 3) ^ ((l >> 4) & 3), so four consecutive lanes cover
  //     one row's 64 bytes; lane 32*h + r reads slot 128*f + 64*(r >> 4) + 4*r' +
  //     ((2*kk + h) ^ ((r' >> 2) & 3)), r' = r & 15: the xor spreads the sixteen
  //     rows of a group of lanes over all banks. The slot for K-step 1 is the one
  //     for K-step 0 with bit 1 flipped, a per-lane distance (lhs_kk1_step).
  constexpr bool ROWS16 = G == 16 && !RHS_I4;
  const bool lhs_row_major = ROWS16 && a.log2_M0 == 0;
  uint32_t a_off[A_LOADS], b_off[B_LOADS];
  if constexpr (G == 16) {
#pragma unroll
    for (int t = 0; t < A_LOADS; ++t) {
      const int p = tid + 256 * t;
      int c = RHS_I4 ? ((p >> 6) & 1) + 2 * ((p >> 5) & 1) : (p >> 4) & 3;
      int row = RHS_I4 ? (p >> 7) * 32 + (p & 31) : (p >> 7) * 32 + 16 * ((p >> 6) & 1) + (p & 15);
      if (lhs_row_major) {
        c = (p & 3) ^ ((p >> 4) & 3);
        row = (p >> 7) * 32 + 16 * ((p >> 6) & 1) + ((p >> 2) & 15);
      }
      a_off[t] = (uint32_t)(row_offset(first_row + row, total_rows - 1, first_row,
                                       a.log2_M0, a.lhs_stride_bytes, a.lhs_rb) +
                            ((16 * c) >> a.log2_lhs_rb) * lhs_kstep + ((16 * c) & (a.lhs_rb - 1)));
    }
#pragma unroll
    for (int t = 0; t < B_LOADS; ++t) {
      const int p = tid + 256 * t;
      const int c = RHS_I4 ? (p >> 5) & 1 : (p >> 4) & 3;
      const int row = RHS_I4 ? (p >> 6) * 32 + (p & 31) : (p >> 7) * 32 + 16 * ((p >> 6) & 1) + (p & 15);
      b_off[t] = (uint32_t)(row_offset(first_col + row, total_cols - 1, first_col, a.log2_N0,
                                       a.rhs_stride_bytes, a.rhs_rb) +
                            ((16 * c) >> a.log2_rhs_rb) * rhs_kstep + ((16 * c) & (a.rhs_rb - 1)));
    }
  } else if constexpr (G == 1) {
    // One-byte row pieces (K0 = 1 int8: the operand is k-major, M0 bytes per k
    // step). A load brings one group of 16 rows x 64 k steps = 1 KiB, group
    // m = 4*t + w of the operand (fragment m >> 1), into slots 64*m .. 64*m + 63:
    // 16-row tiles: lane l the 16 rows at k step l; 8-row tiles: lane l the 8
    // rows of tile l & 1 of the group at k steps 2*(l >> 1) and + 1. Either
    // way a k step's 16 rows lie within 32 bytes of LDS and the transposing
    // read (lds_read_transposed) hands lane (r, h) 8 consecutive k of row r; two
    // of them make a K-step's 16 bytes, in ascending k like every layout here.
    auto piece_of = [&](int log2_t0, int t, int* row, int* k1) {
      const int group = 4 * t + wave;
      *row = 16 * group + (log2_t0 == 4 ? 0 : 8 * (lane & 1));
      *k1 = log2_t0 == 4 ? lane : 2 * (lane >> 1);
    };
#pragma unroll
    for (int t = 0; t < A_LOADS; ++t) {
      int row, k1;
      piece_of(a.log2_M0, t, &row, &k1);
      a_off[t] = (uint32_t)(row_offset(first_row + row, total_rows - (1 << a.log2_M0), first_row, a.log2_M0,
                                       a.lhs_stride_bytes, a.lhs_rb) + k1 * lhs_kstep);
    }
#pragma unroll
    for (int t = 0; t < B_LOADS; ++t) {
      int row, k1;
      piece_of(a.log2_N0, t, &row, &k1);
      b_off[t] = (uint32_t)(row_offset(first_col + row, total_cols - (1 << a.log2_N0), first_col, a.log2_N0,
                                       a.rhs_stride_bytes, a.rhs_rb) + k1 * rhs_kstep);
    }
  } else {
    constexpr int R = 16 / G;  // rows per 16-byte piece
    // Row group and k step of the chunk of this lane's piece in load t (the
    // wavefront's share of the k steps included).
    auto piece_of = [&](bool paired, int t, int* row, int* k1) {
      if (paired) {
        *row = 64 * t + 8 * (lane & 7);
        *k1 = 16 * (wave >> 1) + 8 * ((lane >> 3) & 1) + 4 * (wave & 1) + (lane >> 4);
      } else {
        *row = 32 * (2 * t + (wave >> 1)) + R * (lane % (2 * G));
        *k1 = (32 / G) * (wave & 1) + (16 / G) * ((lane / (2 * G)) & 1) + lane / (4 * G);
      }
    };
#pragma unroll
    for (int t = 0; t < A_LOADS; ++t) {
      int row, k1;
      piece_of(PAIR_A, t, &row, &k1);
      a_off[t] = (uint32_t)(row_offset(first_row + row, total_rows - R, first_row, a.log2_M0, a.lhs_stride_bytes,
                                       a.lhs_rb) + k1 * lhs_kstep);
    }
#pragma unroll
    for (int t = 0; t < B_LOADS; ++t) {
      int row, k1;
      piece_of(PAIR_B, t, &row, &k1);
      b_off[t] = (uint32_t)(row_offset(first_col + row, total_cols - R, first_col, a.log2_N0, a.rhs_stride_bytes,
                                       a.rhs_rb) + k1 * rhs_kstep);
    }
  }

  acc_t acc[AM][BN];
#pragma unroll
  for (int i = 0; i < AM; ++i)
#pragma unroll
    for (int j = 0; j < BN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  // K may end inside the last chunk (not with an int4 rhs). That chunk is then
  // loaded from where a full chunk ends at K, so it overlaps the chunk before
  // it and every load stays inside the operands, and the overlap, i.e. the
  // first `cut_bytes` of its 64 bytes per row, is zeroed in the fragments of
  // both operands (0 * 0 adds nothing, whatever the data).
  const int chunks = a.chunks;
  const int last_chunk = chunks - 1;
  const int32_t cut_bytes = RHS_I4 ? 0 : (int32_t)((64 - (((int64_t)a.K << a.log2_lhs_rb) & 63)) & 63);
  const int64_t lhs_last_base = a.K * lhs_kstep - lhs_chunk_bytes;
  const int64_t rhs_last_base = a.K * rhs_kstep - rhs_chunk_bytes;
  const int64_t lhs_last_advance = lhs_last_base - (last_chunk - 1) * lhs_chunk_bytes;
  const int64_t rhs_last_advance = rhs_last_base - (last_chunk - 1) * rhs_chunk_bytes;

  // Load number `n` (compile-time after unrolling) of the chunk whose operand
  // bases are la / lb, into the stage at LDS byte offset `stage_off`.
  auto issue_load = [&](int n, uint32_t stage_off, const uint8_t* la, const uint8_t* lb) {
    const bool is_a = n < A_LOADS;
    const int t = is_a ? n : n - A_LOADS;
    load_to_lds(stage_off + (is_a ? 0 : A_PIECES * 16) + (256 * t + 64 * wave) * 16,
                is_a ? a_off[t] : b_off[t], is_a ? la : lb);
  };
  auto issue_chunk = [&](int kc) {
    const int idx = min(kc, last_chunk);
    const uint32_t stage_off = (uint32_t)(kc % STAGES) * (STAGE_PIECES * 16);
    const uint8_t* la = lhs_base + (idx == last_chunk ? lhs_last_base : idx * lhs_chunk_bytes);
    const uint8_t* lb = rhs_base + (idx == last_chunk ? rhs_last_base : idx * rhs_chunk_bytes);
#pragma unroll
    for (int n = 0; n < LOADS; ++n) issue_load(n, stage_off, la, lb);
  };

  uint4 pa[AM][2], pb[BN][2], qa[AM][2], qb[BN][2];
  // G < 16: dword `part` (0..3) of a lane's operand for one (fragment, K-step),
  // whose first element is at `first` (already including the lane's offset):
  // the elements are 64*G bytes apart.
  auto gather_dword = [](const uint8_t* first, int part) -> uint32_t {
    if constexpr (G == 2) {
      const uint32_t lo = *(const uint16_t*)(first + (2 * part) * 128);
      const uint32_t hi = *(const uint16_t*)(first + (2 * part + 1) * 128);
      return lo | (hi << 16);
    } else if constexpr (G == 4) {
      return *(const uint32_t*)(first + part * 256);
    } else {
      return *(const uint32_t*)(first + (part >> 1) * 512 + 4 * (part & 1));
    }
  };
  // G == 1: byte offset of lane (r, h)'s transposing reads inside a fragment's
  // 2 KiB (two 16-row groups of 1 KiB, k-major): group r >> 4, k steps from 16*h,
  // and the lane's chunk c = r & 15 of the 16 that one read transposes: the 8
  // rows 8*(c & 1) .. + 7 at k step c >> 1.
  auto transposed_lane_offset = [&](int log2_t0) -> int32_t {
    const int c = lane & 15;
    const int chunk = log2_t0 == 4 ? 8 * c : 32 * (c >> 2) + 16 * (c & 1) + 8 * ((c >> 1) & 1);
    return 1024 * ((lane & 31) >> 4) + 256 * (lane >> 5) + chunk;
  };
  // Fragment f of an operand at 16-byte slot `operand` of the ring, K-step kk.
  auto read_frag = [&](int operand, int f, int kk) -> uint4 {
    if (RHS_I4 && operand >= A_PIECES) {
      const uint4 raw = ring[operand + 64 * f + lane];
      return widen_i4_times16(kk ? make_uint2(raw.z, raw.w) : make_uint2(raw.x, raw.y));
    }
    if constexpr (G == 16) {
      if (!RHS_I4 && operand == 0 && lhs_row_major)
        return ring[128 * f + 64 * ((lane & 31) >> 4) + 4 * (lane & 15) + ((2 * kk + (lane >> 5)) ^ ((lane >> 2) & 3))];
      if (!RHS_I4) return ring[operand + 128 * f + 32 * kk + 64 * ((lane & 31) >> 4) + 16 * (lane >> 5) + (lane & 15)];
      return ring[operand + 128 * f + 64 * kk + lane];
    } else if constexpr (G == 1) {
      const uint8_t* first = (const uint8_t*)(ring + operand) + 2048 * f + 512 * kk +
                             transposed_lane_offset(operand >= A_PIECES ? a.log2_N0 : a.log2_M0);
      const uint2 lo = lds_read_transposed(first), hi = lds_read_transposed(first + 128);
      return make_uint4(lo.x, lo.y, hi.x, hi.y);
    } else {
      const uint8_t* first = (const uint8_t*)(ring + operand) + 1024 * (2 * f + kk) + G * lane;
      return make_uint4(gather_dword(first, 0), gather_dword(first, 1), gather_dword(first, 2), gather_dword(first, 3));
    }
  };
  // Paired fragments: dwords 2*part and 2*part + 1 of the lane's eight for
  // (pair, K-step), split into dword `part` of the even and of the odd fragment.
  auto set_dword = [](uint4& v, int part, uint32_t w) {
    if (part == 0) v.x = w; else if (part == 1) v.y = w; else if (part == 2) v.z = w; else v.w = w;
  };
  auto read_pair_part = [](const uint8_t* first, int part) -> uint2 {
    return make_uint2(*(const uint32_t*)(first + 512 * part), *(const uint32_t*)(first + 512 * part + 256));
  };
  auto split_pair_part = [&](uint2 w, int part, uint4& even, uint4& odd) {
    set_dword(even, part, __builtin_amdgcn_perm(w.y, w.x, 0x05040100u));
    set_dword(odd, part, __builtin_amdgcn_perm(w.y, w.x, 0x07060302u));
  };
  const int frag_a0 = wave_m * AM, frag_b0 = wave_n * BN;

  // Loop-carried, wavefront-uniform state: where the next chunk to load comes
  // from and goes to, and the stage the next fragments are read from. Kept as
  // running values (a few scalar adds per step) rather than recomputed from the
  // chunk number (64-bit multiplies on the scalar unit, in front of the step's
  // first MFMA).
  constexpr uint32_t STAGE_BYTES = STAGE_PIECES * 16, RING_BYTES = STAGES * STAGE_BYTES;
  const uint8_t* load_a = lhs_base + (AHEAD >= last_chunk ? lhs_last_base : AHEAD * lhs_chunk_bytes);
  const uint8_t* load_b = rhs_base + (AHEAD >= last_chunk ? rhs_last_base : AHEAD * rhs_chunk_bytes);
  int load_chunk = AHEAD;
  uint32_t load_stage_off = AHEAD * STAGE_BYTES % RING_BYTES;
  uint32_t read_stage_off = STAGE_BYTES;
  const uint32_t frag_a_off = (uint32_t)((wave_m * AM) * 128) * 16;
  const uint32_t frag_b_off = (uint32_t)(A_PIECES + (wave_n * BN) * (RHS_I4 ? 64 : 128)) * 16;
  // Lane 32*h + r's byte offset into a fragment, and the slots from one K-step
  // of a fragment to the next (see the layouts above).
  const uint8_t* ring_bytes =
      (const uint8_t*)ring + (ROWS16 ? 16 * (64 * ((lane & 31) >> 4) + 16 * (lane >> 5) + (lane & 15))
                                     : (G == 1 ? 0 : (G == 16 ? 16 : G) * lane));
  // G == 2: lanes address dwords, not 16-bit elements. Paired: dword number
  // lane; unpaired: the dword that holds the lane's element (two lanes share
  // it), from which `own_half` then picks the low or the high half. (16-bit
  // reads that fill the halves of a register one after the other made these
  // tiles 1.8x slower than the 4-byte ones: the second read of a register has
  // to wait for the first.)
  // (G == 1: the per-operand lane offset of the transposing reads instead.)
  // (Row-major lhs: the distance from the rhs lane slot, which ring_bytes holds, to the lhs one for K-step 0.)
  const int32_t lhs_rm_slot0 = 4 * (lane & 15) + ((lane >> 5) ^ ((lane >> 2) & 3));
  const int32_t pair_a_lane =
      G == 1 ? transposed_lane_offset(a.log2_M0)
             : (G == 2 ? (PAIR_A ? 2 * lane : -2 * (lane & 1))
                       : (lhs_row_major ? 16 * (lhs_rm_slot0 - (16 * (lane >> 5) + (lane & 15))) : 0));
  // Bytes from an lhs fragment's K-step 0 to its K-step 1 in this lane's reads.
  const int32_t lhs_kk1_step = lhs_row_major ? 16 * ((lhs_rm_slot0 ^ 2) - lhs_rm_slot0) : 16 * (ROWS16 ? 32 : 64);
  const int32_t pair_b_lane =
      G == 1 ? transposed_lane_offset(a.log2_N0) : (G != 2 ? 0 : (PAIR_B ? 2 * lane : -2 * (lane & 1)));
  const uint32_t own_half = (lane & 1) ? 0x07060302u : 0x05040100u;
  constexpr int KK16 = ROWS16 ? 32 : 64;

  // One pipeline step for the chunk whose fragments are in `cur`:
  //   a few MFMAs first (they only need registers, and keep the matrix pipe
  //   fed across the barrier); wait until this wavefront's loads of the next
  //   chunk have landed; barrier (now everyone's have, and everyone is done
  //   reading the stage of the previous chunk); then the remaining MFMAs with,
  //   between them, the loads of the chunk three ahead into the stage just
  //   freed and the LDS reads of the next chunk's fragments.
  // A wavefront issues in order and a memory instruction takes several cycles
  // to issue, so more than one or two of them between two MFMAs lets the
  // matrix pipe run dry: they are dealt out one (half) fragment and at most one
  // load per MFMA. The reads end a quarter of the step before its end, so that
  // the last of them has returned when the next step starts; fragments are
  // read in the order the next step consumes them.
  // (`held_loads_behind`: the eight loads of destination values that variant 3 issues at the start of a phase
  // are younger than the chunk this step waits for, and may stay in flight with it.)
  // `between_mfmas(m)`: extra work placed behind MFMA m of the step (variant 3 adds destination values there).
  auto step_with = [&](const uint4 (*cur_a)[2], const uint4 (*cur_b)[2], uint4 (*nxt_a)[2], uint4 (*nxt_b)[2],
                       bool held_loads_behind, auto between_mfmas) {
    constexpr int SUB = SubSteps<KIND>::value;
    constexpr int MFMAS = 2 * AM * BN * SUB;
    // Units a fragment's LDS reads are dealt out in: a 128-bit read; two pairs of
    // dwords; two 64-bit reads; four pairs of dwords holding 16-bit elements.
    constexpr int PARTS = G == 16 ? 1 : (G == 2 ? 4 : 2);
    // Read units, in the order the next step consumes them: per K-step the rhs
    // fragments, then the lhs fragments. An int4 rhs fragment is read once, raw,
    // for both K-steps (first), and widened after the last read has been issued.
    constexpr int B_UNITS = RHS_I4 ? BN : 0;
    constexpr int UNITS_A = AM * (PAIR_A ? 2 : PARTS), UNITS_B = BN * (PAIR_B ? 2 : PARTS);  // per K-step
    constexpr int READS = RHS_I4 ? BN + 2 * AM : 2 * (UNITS_A + UNITS_B);
    constexpr int LEAD = MFMAS >= 16 ? 4 : (MFMAS >= 8 ? 2 : 0);   // MFMAs ahead of the barrier
    // MFMAs after the last read. (On the 128x64 tile 2-byte pieces get one, so that their reads are not split
    // right behind their issue: 128 x 14336 x 4096 int8 16x16x2 27 -> 24 us, f16 16x16x1 49 -> 42 us; on the
    // 64x64 tile it changed nothing.)
    constexpr int TAIL_FREE = MFMAS >= 8 ? MFMAS / 4 : ((RHS_I4 || (G == 2 && MFMAS >= 4)) ? 1 : 0);
    constexpr int SLOTS = MFMAS - LEAD - TAIL_FREE;                // MFMAs that carry memory work
    static_assert(SLOTS >= 1, "no room for the memory instructions");
    static_assert(!RHS_I4 || TAIL_FREE >= 1, "nowhere to widen");
    // Paired fragments: the dwords of a read unit are split this many MFMAs
    // after the read was issued (a wavefront issues in order: splitting right
    // away would stall it, MFMAs included, for the LDS latency of every unit).
    // (3 MFMAs: int8 16x16x2 at 4096^3 86 us; 5: 81 us; 8, all there are on the 256x256 tile: 79 us.)
    constexpr int SPLIT_DELAY = TAIL_FREE;
    uint2 raw_pair[G == 2 ? READS : 1];
    // Where read unit u of the next step's fragments goes.
    auto unit_of = [&](int u, bool* is_b, bool* paired, int* kk, int* y) {
      *kk = u / (UNITS_A + UNITS_B);
      const int x = u % (UNITS_A + UNITS_B);
      *is_b = x < UNITS_B;
      *paired = *is_b ? PAIR_B : PAIR_A;
      *y = *is_b ? x : x - UNITS_B;
    };
    auto split_units_of = [&](int read_slot) {
      if constexpr (G == 2) {
        if (read_slot < 0 || read_slot >= SLOTS) return;
#pragma unroll
        for (int u = read_slot * READS / SLOTS; u < (read_slot + 1) * READS / SLOTS; ++u) {
          bool is_b, paired;
          int kk, y;
          unit_of(u, &is_b, &paired, &kk, &y);
          uint4(*nxt)[2] = is_b ? nxt_b : nxt_a;
          if (paired) {
            split_pair_part(raw_pair[u], y % 4, nxt[2 * (y / 4)][kk], nxt[2 * (y / 4) + 1][kk]);
          } else {
            set_dword(nxt[y / 4][kk], y % 4, __builtin_amdgcn_perm(raw_pair[u].y, raw_pair[u].x, own_half));
          }
        }
      }
    };
    auto multiply = [&](int m) {
      const int kk = m / (AM * BN * SUB), sub = (m / (AM * BN)) % SUB, i = (m % (AM * BN)) / BN, j = m % BN;
      acc[i][j] = mfma<KIND>(cur_b[j][kk], cur_a[i][kk], acc[i][j], sub);
    };
#pragma unroll
    for (int m = 0; m < LEAD; ++m) {
      multiply(m);
      between_mfmas(m);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (STAGGER == 3) {
      if (held_loads_behind) wait_loads_but<LOADS*(AHEAD - 2) + 8>(); else wait_loads_but<LOADS*(AHEAD - 2)>();
    } else {
      wait_loads_but<LOADS*(AHEAD - 2)>();
    }
    __builtin_amdgcn_s_barrier();
    // The fragments read during this step are those of chunk load_chunk - AHEAD + 1.
    // (The variants with the staggered tail are launched for K in whole chunks only: nothing to cut there, and the
    // masking, which the compiler makes unconditional, 64 instructions per step, is left out.)
    const bool cut_next = STAGGER == 0 && cut_bytes != 0 && load_chunk - AHEAD + 1 == last_chunk;
    const uint8_t* read_a = ring_bytes + read_stage_off + frag_a_off + pair_a_lane;
    const uint8_t* read_a_kk1 = read_a + lhs_kk1_step;  // (used where the lhs has 16-byte pieces)
    const uint8_t* read_b = ring_bytes + read_stage_off + frag_b_off + pair_b_lane;
    uint4 raw_b[RHS_I4 ? BN : 1];
#pragma unroll
    for (int m = LEAD; m < MFMAS; ++m) {
      const int slot = m - LEAD;
      if (slot < SLOTS) {
#pragma unroll
        for (int n = slot * LOADS / SLOTS; n < (slot + 1) * LOADS / SLOTS; ++n)
          issue_load(n, load_stage_off, load_a, load_b);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = slot * READS / SLOTS; u < (slot + 1) * READS / SLOTS; ++u) {
          if constexpr (RHS_I4) {
            if (u < B_UNITS) {
              raw_b[u] = *(const uint4*)(read_b + (64 * u) * 16);
            } else {
              const int kk = (u - B_UNITS) / AM, i = (u - B_UNITS) % AM;
              nxt_a[i][kk] = *(const uint4*)((kk ? read_a_kk1 : read_a) + 128 * i * 16);
            }
          } else {
            bool is_b, paired;
            int kk, y;
            unit_of(u, &is_b, &paired, &kk, &y);
            const uint8_t* src = is_b ? read_b : read_a;
            uint4(*nxt)[2] = is_b ? nxt_b : nxt_a;
            if (paired) {
              raw_pair[u] = read_pair_part(src + 4096 * (y / 4) + 2048 * kk, y % 4);
              continue;
            }
            const int frag = y / PARTS, part = y % PARTS;
            uint4& dst = nxt[frag][kk];
            if constexpr (G == 16) {
              if (is_b) dst = *(const uint4*)(src + (128 * frag + KK16 * kk) * 16);
              else dst = *(const uint4*)((kk ? read_a_kk1 : read_a) + 128 * frag * 16);
            } else {
              const uint8_t* first = src + 1024 * (2 * frag + kk);
              if constexpr (G == 1) {
                // One transposing read: 8 consecutive k of the lane's row.
                const uint2 w = lds_read_transposed(src + 2048 * frag + 512 * kk + 128 * part);
                if (part == 0) { dst.x = w.x; dst.y = w.y; } else { dst.z = w.x; dst.w = w.y; }
              } else if constexpr (G == 2) {
                // Elements 2*part and 2*part + 1 of the lane's eight, 128 bytes apart, each with its neighbour.
                raw_pair[u] = make_uint2(*(const uint32_t*)(first + 256 * part), *(const uint32_t*)(first + 256 * part + 128));
                (void)dst;
              } else if constexpr (G == 8) {
                // One 64-bit read (two dword reads of adjacent addresses, which
                // is what the compiler makes of 4-byte aligned accesses, collide
                // on the banks: lanes are 8 bytes apart).
                const uint2 w = *(const uint2*)(first + part * 512);
                if (part == 0) { dst.x = w.x; dst.y = w.y; } else { dst.z = w.x; dst.w = w.y; }
              } else {
                if (part == 0) { dst.x = gather_dword(first, 0); dst.y = gather_dword(first, 1); }
                else { dst.z = gather_dword(first, 2); dst.w = gather_dword(first, 3); }
              }
            }
          }
        }
      } else if constexpr (RHS_I4) {
        // Widening, dealt out over the MFMAs that carry no memory work.
        const int tail = slot - SLOTS;
#pragma unroll
        for (int w = tail * 2 * BN / TAIL_FREE; w < (tail + 1) * 2 * BN / TAIL_FREE; ++w) {
          const int kk = w / BN, j = w % BN;
          nxt_b[j][kk] = widen_i4_times16(kk ? make_uint2(raw_b[j].z, raw_b[j].w) : make_uint2(raw_b[j].x, raw_b[j].y));
        }
      }
      split_units_of(slot - SPLIT_DELAY);
      multiply(m);
      between_mfmas(m);
      if (m == MFMAS - 1) {
        // Advance the running state (clamped at the last chunk: the loads
        // issued beyond it are redundant, their stages are never read).
        const bool more = load_chunk < last_chunk, to_last = load_chunk + 1 == last_chunk;
        load_a += more ? (to_last ? lhs_last_advance : lhs_chunk_bytes) : 0;
        load_b += more ? (to_last ? rhs_last_advance : rhs_chunk_bytes) : 0;
        ++load_chunk;
        load_stage_off = load_stage_off + STAGE_BYTES == RING_BYTES ? 0 : load_stage_off + STAGE_BYTES;
        read_stage_off = read_stage_off + STAGE_BYTES == RING_BYTES ? 0 : read_stage_off + STAGE_BYTES;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!RHS_I4) {
      if (cut_next) {
        // Lane half h of K-step kk holds bytes 32*kk + 16*h .. + 15 of the chunk's
        // 64 bytes per row, in ascending order of k in every layout above.
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const int cut = min(max(cut_bytes - 32 * kk - 16 * (lane >> 5), 0), 16);
          uint32_t keep[4];
#pragma unroll
          for (int w = 0; w < 4; ++w)
            keep[w] = cut >= 4 * w + 4 ? 0u : (cut <= 4 * w ? 0xFFFFFFFFu : 0xFFFFFFFFu << (8 * (cut - 4 * w)));
#pragma unroll
          for (int i = 0; i < AM; ++i) {
            nxt_a[i][kk].x &= keep[0]; nxt_a[i][kk].y &= keep[1]; nxt_a[i][kk].z &= keep[2]; nxt_a[i][kk].w &= keep[3];
          }
#pragma unroll
          for (int j = 0; j < BN; ++j) {
            nxt_b[j][kk].x &= keep[0]; nxt_b[j][kk].y &= keep[1]; nxt_b[j][kk].z &= keep[2]; nxt_b[j][kk].w &= keep[3];
          }
        }
      }
    }
  };
  auto step = [&](const uint4 (*cur_a)[2], const uint4 (*cur_b)[2], uint4 (*nxt_a)[2], uint4 (*nxt_b)[2],
                  bool held_loads_behind = false) {
    step_with(cur_a, cur_b, nxt_a, nxt_b, held_loads_behind, [](int) {});
  };

  // The last AHEAD chunks, for the 256x256 tile. At the end of the loop above
  // every accumulator becomes final at the same moment, and the whole tile (256
  // KiB per workgroup, the whole output of the launch in one burst) is stored
  // with the matrix pipe idle. Here the loop stops AHEAD chunks early, when
  // their operands are all in the workgroup already (one chunk's fragments in
  // registers, the others in the ring), and those chunks are multiplied in
  // another order: first the register chunk as usual, during which the loads
  // still in flight are awaited and the ring chunks' rhs fragments and the first
  // row's lhs fragments are read; then fragment by fragment, two fragments of a
  // row at a time, each pair running through the ring chunks and being stored
  // while the next pair is multiplied (one 128-bit store per MFMA, the first
  // behind the pair's last MFMA by a few instructions so that it does not wait
  // for it). Only the last pair's stores come after the last MFMA. The stores of
  // the launch are thereby spread over the last two and a half steps.
  // K in whole chunks, unpaired fragment layouts.
  constexpr bool TAILED = STAGGER != 0;
  static_assert(!TAILED || (AM == 4 && BN == 4 && !RHS_I4 && !PAIR_A && !PAIR_B && KIND != kF32), "staggered tail");
  // Output addressing of this wavefront's fragments, as in store_block: the byte offset of quad (j, q) from the
  // sub-block's first column tile, whether it lies inside the matrix, and the pointer of a fragment row's line.
  typedef typename AccType<KIND>::scalar out_scalar_t;
  typedef out_scalar_t out_quad_t __attribute__((ext_vector_type(4)));
  typedef typename std::conditional<NARROW, uint2, out_quad_t>::type out_stored_t;
  constexpr int OUT_BYTES = NARROW ? 2 : 4;
  struct OutAddressing {
    uint8_t* wave_out;
    uint32_t col_off[BN][4];
    uint32_t col_inside;
  };
  auto out_addressing = [&]() -> OutAddressing {
    OutAddressing o;
    const int32_t N0 = 1 << a.log2_N0;
    const int64_t wave_col = first_col + wave_n * (32 * BN);
    const int64_t first_col_tile = wave_col >> a.log2_N0;
    o.wave_out = a.out + OUT_BYTES * (first_col_tile << (a.log2_M0 + a.log2_N0));
    o.col_inside = 0;
#pragma unroll
    for (int j = 0; j < BN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = wave_col + 4 * (lane >> 5) + 32 * j + 8 * q;
        o.col_off[j][q] = (uint32_t)(OUT_BYTES * ((((col >> a.log2_N0) - first_col_tile) << (a.log2_M0 + a.log2_N0)) +
                                                  (col & (N0 - 1))));
        if (col < total_cols) o.col_inside |= 1u << (4 * j + q);
      }
    return o;
  };
  auto out_row_pointer = [&](const OutAddressing& o, int i, bool* inside) -> uint8_t* {
    const int32_t M0 = 1 << a.log2_M0;
    const int64_t this_row = first_row + wave_m * (32 * AM) + 32 * i + (lane & 31);
    const int64_t row = min(this_row, total_rows - 1);
    *inside = this_row < total_rows;
    return o.wave_out + OUT_BYTES * ((row >> a.log2_M0) * a.out_stride0 + ((row & (M0 - 1)) << a.log2_N0));
  };
  constexpr int OUT_EBITS = KIND == kF16 ? 5 : 8;
  auto out_to_float = [](out_stored_t w) -> out_quad_t {
    if constexpr (NARROW) {
      return out_quad_t{widen16<OUT_EBITS>((uint16_t)w.x), widen16<OUT_EBITS>((uint16_t)(w.x >> 16)),
                        widen16<OUT_EBITS>((uint16_t)w.y), widen16<OUT_EBITS>((uint16_t)(w.y >> 16))};
    } else {
      return w;
    }
  };
  auto out_to_stored = [](out_quad_t v) -> out_stored_t {
    if constexpr (NARROW) {
      return make_uint2((uint32_t)narrow16<OUT_EBITS>(v.x) | ((uint32_t)narrow16<OUT_EBITS>(v.y) << 16),
                        (uint32_t)narrow16<OUT_EBITS>(v.z) | ((uint32_t)narrow16<OUT_EBITS>(v.w) << 16));
    } else {
      return v;
    }
  };

  auto tail = [&](auto cur_a, auto cur_b) {  // (generic: only instantiated where it is called)
    constexpr int JR = AHEAD - 1;            // chunks in the ring
    constexpr int PAIR_MFMAS = 4 * JR;       // two fragments x JR chunks x two K-steps
    static_assert(PAIR_MFMAS >= 8, "a quad of the previous pair is stored with each MFMA");
    const OutAddressing o = out_addressing();

    // Fragment f of an operand, K-step kk, from the stage whose per-lane bases are given.
    auto read_fragment = [&](const uint8_t* base_a, const uint8_t* base_a_kk1, const uint8_t* base_b, bool is_b, int f,
                             int kk) -> uint4 {
      const uint8_t* src = is_b ? base_b : base_a;
      if constexpr (G == 16) {
        if (is_b) return *(const uint4*)(src + (128 * f + KK16 * kk) * 16);
        return *(const uint4*)((kk ? base_a_kk1 : base_a) + 128 * f * 16);
      } else if constexpr (G == 1) {
        const uint2 lo = lds_read_transposed(src + 2048 * f + 512 * kk);
        const uint2 hi = lds_read_transposed(src + 2048 * f + 512 * kk + 128);
        return make_uint4(lo.x, lo.y, hi.x, hi.y);
      } else if constexpr (G == 8) {
        const uint8_t* first = src + 1024 * (2 * f + kk);
        const uint2 lo = *(const uint2*)first, hi = *(const uint2*)(first + 512);
        return make_uint4(lo.x, lo.y, hi.x, hi.y);
      } else {
        const uint8_t* first = src + 1024 * (2 * f + kk);
        return make_uint4(gather_dword(first, 0), gather_dword(first, 1), gather_dword(first, 2), gather_dword(first, 3));
      }
    };
    // Per-lane bases of the ring chunks' stages.
    const uint8_t* base_a[JR];
    const uint8_t* base_a_kk1[JR];
    const uint8_t* base_b[JR];
    {
      uint32_t stage_off = read_stage_off;
#pragma unroll
      for (int c = 0; c < JR; ++c) {
        base_a[c] = ring_bytes + stage_off + frag_a_off + pair_a_lane;
        base_a_kk1[c] = base_a[c] + lhs_kk1_step;
        base_b[c] = ring_bytes + stage_off + frag_b_off + pair_b_lane;
        stage_off = stage_off + STAGE_BYTES == RING_BYTES ? 0 : stage_off + STAGE_BYTES;
      }
    }
    uint4 tb[BN][JR][2], ta[2][JR][2];
    // The reads of the register phase, in the order the first pair needs them: per chunk and K-step the first
    // lhs row and the first two rhs fragments, then the other two rhs fragments.
    constexpr int EARLY_READS = 2 * JR * (1 + BN);
    auto early_read = [&](int n) {
      const int half = n / (2 * JR * 3);  // 0: lhs row 0 and rhs 0, 1; 1: rhs 2, 3
      if (half == 0) {
        const int c = n / 6, kk = (n / 3) % 2, what = n % 3;
        if (what == 0) ta[0][c][kk] = read_fragment(base_a[c], base_a_kk1[c], base_b[c], false, 0, kk);
        else tb[what - 1][c][kk] = read_fragment(base_a[c], base_a_kk1[c], base_b[c], true, what - 1, kk);
      } else {
        const int m = n - 2 * JR * 3, c = m / 4, kk = (m / 2) % 2, j = 2 + m % 2;
        tb[j][c][kk] = read_fragment(base_a[c], base_a_kk1[c], base_b[c], true, j, kk);
      }
    };

    // Register phase: the chunk whose fragments are in `cur`, in the usual order.
    constexpr int REG_MFMAS = 2 * AM * BN;
    constexpr int WAIT_AT = REG_MFMAS - 20 > 4 ? 12 : 4;  // MFMAs ahead of the wait for the ring chunks' loads
#pragma unroll
    for (int m = 0; m < REG_MFMAS; ++m) {
      if (m == WAIT_AT) {
        wait_loads_but<0>();
        __builtin_amdgcn_s_barrier();
      }
      if (m >= WAIT_AT) {
        constexpr int SLOTS = REG_MFMAS - WAIT_AT;
#pragma unroll
        for (int n = (m - WAIT_AT) * EARLY_READS / SLOTS; n < (m - WAIT_AT + 1) * EARLY_READS / SLOTS; ++n) early_read(n);
      }
      const int kk = m / (AM * BN), i = (m % (AM * BN)) / BN, j = m % BN;
      acc[i][j] = mfma<KIND>(cur_b[j][kk], cur_a[i][kk], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }

    // Fragment phase. (The accumulators are pinned where they are, here and again before each pair is stored:
    // left alone, the compiler moves them to ordinary registers ahead of the stores, and there are not that many.)
#pragma unroll
    for (int i = 0; i < AM; ++i)
#pragma unroll
      for (int j = 0; j < BN; ++j) asm volatile("" : "+a"(acc[i][j]));
    uint8_t* prev_row = nullptr;
    bool prev_row_inside = false;
    // Quad n (fragment n / 4 of the pair, quad n % 4) of pair (i, jp). An accumulating call adds what the
    // destination held, loaded while the pair was multiplied (one quad per MFMA, each into the register the
    // previous pair's quad of the same number has just been added from).
    constexpr bool ACCUMULATING = STAGGER == 2;
    out_quad_t old[2][4];
    auto store_quad = [&](int i, int jp, int n, uint8_t* row_out, bool row_inside) {
      const int t = n / 4, q = n % 4, j = 2 * jp + t;
      out_quad_t v = out_quad_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
      if constexpr (ACCUMULATING) v += old[t][q];
      if (row_inside && (o.col_inside >> (4 * j + q) & 1)) *(out_stored_t*)(row_out + o.col_off[j][q]) = out_to_stored(v);
    };
    auto load_old = [&](int jp, int n, const uint8_t* row_out, bool row_inside) {
      const int t = n / 4, q = n % 4, j = 2 * jp + t;
      old[t][q] = out_quad_t{0, 0, 0, 0};
      if (row_inside && (o.col_inside >> (4 * j + q) & 1))
        old[t][q] = out_to_float(*(const out_stored_t*)(row_out + o.col_off[j][q]));
    };
#pragma unroll
    for (int i = 0; i < AM; ++i) {
      bool row_inside;
      uint8_t* row_out = out_row_pointer(o, i, &row_inside);
#pragma unroll
      for (int jp = 0; jp < BN / 2; ++jp) {
        const int pair = i * (BN / 2) + jp;
#pragma unroll
        for (int m = 0; m < PAIR_MFMAS; ++m) {
          // The previous pair's quads, from the third MFMA on (its last MFMA has left the pipe by then).
          constexpr int STORE_FROM = PAIR_MFMAS >= 10 ? 2 : 0;
          const int n = m - STORE_FROM;
          if (n >= 0 && n < 8) {
            if (pair > 0) {
              const int pi = (pair - 1) / (BN / 2), pjp = (pair - 1) % (BN / 2);
              if (n == 0) asm volatile("" : "+a"(acc[pi][2 * pjp]), "+a"(acc[pi][2 * pjp + 1]));
              store_quad(pi, pjp, n, pi == i ? row_out : prev_row, pi == i ? row_inside : prev_row_inside);
            }
            if constexpr (ACCUMULATING) load_old(jp, n, row_out, row_inside);
          }
          // The next row's lhs fragments, read under this row's second pair.
          if (jp == BN / 2 - 1 && i + 1 < AM && m < 2 * JR)
            ta[(i + 1) & 1][m / 2][m % 2] = read_fragment(base_a[m / 2], base_a_kk1[m / 2], base_b[m / 2], false, i + 1, m % 2);
          const int c = m / 4, kk = (m / 2) % 2, t = m % 2, j = 2 * jp + t;
          acc[i][j] = mfma<KIND>(tb[j][c][kk], ta[i & 1][c][kk], acc[i][j]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      prev_row = row_out;
      prev_row_inside = row_inside;
    }
    // The last pair's quads.
    UK_TIMELINE(const unsigned long long tl_last_mfma = __builtin_amdgcn_s_memrealtime();)
    asm volatile("" : "+a"(acc[AM - 1][BN - 2]), "+a"(acc[AM - 1][BN - 1]));
#pragma unroll
    for (int n = 0; n < 8; ++n) store_quad(AM - 1, BN / 2 - 1, n, prev_row, prev_row_inside);
    UK_TIMELINE(asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (lane == 0 && wave == 0 && blockIdx.x < 256) {
                  unsigned long long* t = uk_timeline + blockIdx.x * 8;
                  t[0] = tl_start; t[1] = tl_loop; t[2] = tl_loop_end; t[3] = tl_last_mfma;
                  t[4] = __builtin_amdgcn_s_memrealtime();
                })
  };

#pragma unroll
  for (int c = 0; c < AHEAD; ++c) issue_chunk(c);
  wait_loads_but<(AHEAD - 1) * LOADS>();
  __syncthreads();
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
    for (int j = 0; j < BN; ++j) {
      if constexpr (PAIR_B) {
        if (j % 2 == 0) {
#pragma unroll
          for (int part = 0; part < 4; ++part)
            split_pair_part(
                read_pair_part((const uint8_t*)(ring + A_PIECES) + 2048 * (frag_b0 + j) + 2048 * kk + 4 * lane, part),
                part, pb[j][kk], pb[j + 1][kk]);
        }
      } else {
        pb[j][kk] = read_frag(A_PIECES, frag_b0 + j, kk);
      }
    }
#pragma unroll
    for (int i = 0; i < AM; ++i) {
      if constexpr (PAIR_A) {
        if (i % 2 == 0) {
#pragma unroll
          for (int part = 0; part < 4; ++part)
            split_pair_part(read_pair_part((const uint8_t*)ring + 2048 * (frag_a0 + i) + 2048 * kk + 4 * lane, part),
                            part, pa[i][kk], pa[i + 1][kk]);
        }
      } else {
        pa[i][kk] = read_frag(0, frag_a0 + i, kk);
      }
    }
  }
  UK_TIMELINE(tl_loop = __builtin_amdgcn_s_memrealtime();)
  int kc = 0;
  if constexpr (TAILED) {
    // (The host launches this variant only for K in whole chunks, at least 2 * STAGES of them.)
    // An odd step first, so that the loop always ends with the next chunk's fragments in (pa, pb).
    const int main_steps = chunks - AHEAD;
    if (main_steps & 1) {
      step(pa, pb, qa, qb);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
        for (int i = 0; i < AM; ++i) pa[i][kk] = qa[i][kk];
#pragma unroll
        for (int j = 0; j < BN; ++j) pb[j][kk] = qb[j][kk];
      }
      kc = 1;
    }
    if constexpr (STAGGER == 3) {
      // An accumulating call: what the destination held is added to the accumulators on the way, so that the
      // tail only stores (read in the tail, the 256 KiB per workgroup come from HBM on top of the stores, with
      // three chunks of MFMAs to hide under). One phase per pair of fragments: its eight quads are loaded, an even
      // number of steps runs, and in the last of them the values are added, each fragment's behind its first
      // MFMA of that step, two registers per MFMA, done before its second. The loads are issued from assembly,
      // like those of the ring, so that the compiler does not wait for them (its waits would be for every load
      // in flight, the ring's youngest included): after three steps they have landed, because loads return in
      // order and the third step waits for a chunk that was requested after them. A lane outside the matrix loads
      // from the start of the destination; what it adds is never stored.
      static_assert(SubSteps<KIND>::value == 1, "one MFMA per fragment and K-step");
      const OutAddressing o = out_addressing();
      constexpr int PAIRS = AM * (BN / 2);
      // The workgroups of a launch run in step; were all of them to load a pair at the same moment, the 16 MiB
      // would take longer to arrive than the two steps the ring can wait. Each therefore starts its phases a
      // different number of steps into the loop (one phase's worth of steps is set aside for that).
      const int per_phase = ((main_steps - kc) / (PAIRS + 1)) & ~1;  // (the host sees to it that this is at least 4)
      for (int lead = 2 * ((int)((blockIdx.x >> 3) & 7) * (per_phase / 2) >> 3); lead > 0; lead -= 2, kc += 2) {
        step(pa, pb, qa, qb);
        step(qa, qb, pa, pb);
      }
#pragma unroll
      for (int pair = 0; pair < PAIRS; ++pair) {
        const int i = pair / (BN / 2), jp = pair % (BN / 2);
        bool row_inside;
        const uint8_t* row_out = out_row_pointer(o, i, &row_inside);
        out_stored_t held[8];
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          const int j = 2 * jp + n / 4, q = n % 4;
          const uint8_t* from = row_inside && (o.col_inside >> (4 * j + q) & 1) ? row_out + o.col_off[j][q] : a.out;
          if constexpr (NARROW) asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(held[n]) : "v"(from) : "memory");
          else asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(held[n]) : "v"(from) : "memory");
        }
        int held_loads_behind = 1;
        for (int s = 0; s + 2 < per_phase; s += 2, kc += 2) {
          asm volatile("" : "+s"(held_loads_behind));  // (one copy of the loop body, not a peeled first pass)
          step(pa, pb, qa, qb, held_loads_behind != 0);
          step(qa, qb, pa, pb, held_loads_behind != 0);
          held_loads_behind = 0;
        }
        step(pa, pb, qa, qb);
        out_quad_t was[8];
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          asm volatile("" : "+v"(held[n]));
          was[n] = out_to_float(held[n]);
        }
        step_with(qa, qb, pa, pb, false, [&](int m) {
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const int j = 2 * jp + t, slot = m - (i * BN + j + 2);
            if (slot < 0 || slot >= 8) continue;
#pragma unroll
            for (int r = 2 * slot; r < 2 * slot + 2; ++r) acc[i][j][r] += was[4 * t + r / 4][r % 4];
          }
        });
        kc += 2;
      }
    }
    for (; kc + 1 < main_steps; kc += 2) {
      step(pa, pb, qa, qb);
      step(qa, qb, pa, pb);
    }
    UK_TIMELINE(tl_loop_end = __builtin_amdgcn_s_memrealtime();)
    tail(pa, pb);
    return;
  }
  for (; kc + 1 < chunks; kc += 2) {
    step(pa, pb, qa, qb);
    step(qa, qb, pa, pb);
  }
  if (kc < chunks) step(pa, pb, qa, qb);
  // No load may still be writing LDS when the workgroup's allocation is freed.
  wait_loads_but<0>();
  UK_TIMELINE(tl_loop_end = __builtin_amdgcn_s_memrealtime();)

  store_block<KIND, RHS_I4, NARROW, AM, BN, PAIR_A, PAIR_B>(a, acc, first_row + wave_m * (32 * AM),
                                                            first_col + wave_n * (32 * BN), lane);
  UK_TIMELINE(asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
              if (lane == 0 && wave == 0 && blockIdx.x < 256) {
                unsigned long long* t = uk_timeline + blockIdx.x * 8;
                t[0] = tl_start; t[1] = tl_loop; t[2] = tl_loop_end; t[3] = tl_loop_end;
                t[4] = __builtin_amdgcn_s_memrealtime();
              })
}

// (Overloads on scalars rather than a bit cast of a vector element.)
__device__ __forceinline__ uint32_t value_bits(int32_t v) { return (uint32_t)v; }
__device__ __forceinline__ uint32_t value_bits(float v) { return __float_as_uint(v); }
__device__ __forceinline__ void set_from_bits(int32_t& v, uint32_t bits) { v = (int32_t)bits; }
__device__ __forceinline__ void set_from_bits(float& v, uint32_t bits) { v = __uint_as_float(bits); }

// ---------------------------------------------------------------------------
// Block tiles whose four wavefronts split K instead of the tile, for problems
// with few block tiles: few rhs rows against a long K (say 128 x 4096 x 14336,
// 128 tiles of 64x64), or at most 128 lhs rows (one tile row of 128x64). There
// the kernel above is bound by the latency of one pipeline step (counter wait,
// barrier, LDS reads; about 140 ns) per 64 bytes of K per workgroup, and with
// few tiles half the compute units have no workgroup at all. Here every
// wavefront multiplies the whole tile ((32*AMF) x 64, AMF x 2 fragments) over
// its quarter of the step's K bytes, so a workgroup streams more per step, and
// the four partial tiles are summed through LDS at the end, in wavefront order
// (deterministic). Row pieces of 16 bytes or more, int8 / f16 / bf16.
//   AMF == 2: 64x64 tile, 256 bytes of K per row and step (two MFMA K-steps per
//     wavefront), ring of 4 stages of 32 KiB. 128 x 4096 x 14336 bf16 62 -> 41 us.
//   AMF == 4: 128x64 tile, 128 bytes of K per row and step (one K-step per
//     wavefront), ring of 6 stages of 24 KiB.
// What bounds them is what a compute unit's load path moves (64 bytes per
// cycle at best; a stage takes about 500 resp. 400 cycles).
//
// LDS stage: per operand four slices (one per wavefront's share of K, 16*COLS
// bytes per row, COLS = 2 * K-steps per wavefront) of fragments in the layout
// of the kernel above (G == 16) with COLS 16-byte columns: slot p of a
// fragment holds rows 16*(p / (16*COLS)) + (p & 15), column (p >> 4) & (COLS-1).
// A load fills 64 consecutive slots of one slice.
template <int KIND, bool NARROW, int AMF>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, AMF == 2 ? 2 : 1)))
void mmt4d_mfma_split_k_kernel(const MfmaArgs a) {
  typedef typename AccType<KIND>::type acc_t;
  static_assert(KIND != kF32, "one MFMA per fragment pair");
  static_assert(AMF == 2 || AMF == 4, "64 or 128 lhs rows");
  constexpr int KKW = AMF == 2 ? 2 : 1;       // MFMA K-steps per wavefront and step
  constexpr int COLS = 2 * KKW;               // 16-byte columns of a slice
  constexpr int CHUNK_BYTES = 4 * 16 * COLS;  // of K per row and step
  constexpr int STAGES = AMF == 2 ? 4 : 6, AHEAD = STAGES - 1;  // (a fifth stage of the 64x64 tile changed nothing)
  constexpr int FRAG_SLOTS = 32 * COLS;
  constexpr int A_SLICE = AMF * FRAG_SLOTS, B_SLICE = 2 * FRAG_SLOTS;  // slots per slice
  constexpr int A_PIECES = 4 * A_SLICE, B_PIECES = 4 * B_SLICE;
  constexpr uint32_t STAGE_BYTES = (A_PIECES + B_PIECES) * 16, RING_BYTES = STAGES * STAGE_BYTES;
  constexpr int A_LOADS = A_PIECES / 256, B_LOADS = B_PIECES / 256, LOADS = A_LOADS + B_LOADS;  // per wavefront
  constexpr int READS = KKW * (AMF + 2);      // 128-bit LDS reads per wavefront and step
  constexpr int MFMAS = KKW * AMF * 2;
  static_assert(MFMAS == 8 && LOADS <= 8 && READS <= 8, "the step below deals memory work over four of eight MFMAs");

  int tile_row, tile_col;
  if (!locate_block(a, &tile_row, &tile_col)) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int64_t total_rows = (int64_t)a.M << a.log2_M0;
  const int64_t total_cols = (int64_t)a.N << a.log2_N0;
  const int64_t lhs_kstep = (int64_t)a.lhs_rb << a.log2_M0;
  const int64_t rhs_kstep = (int64_t)a.rhs_rb << a.log2_N0;
  const int64_t lhs_chunk_bytes = (CHUNK_BYTES >> a.log2_lhs_rb) * lhs_kstep;
  const int64_t rhs_chunk_bytes = (CHUNK_BYTES >> a.log2_rhs_rb) * rhs_kstep;
  const int64_t first_row = (int64_t)tile_row * (32 * AMF), first_col = (int64_t)tile_col * 64;
  const uint8_t* lhs_base = a.lhs + (first_row >> a.log2_M0) * a.lhs_stride_bytes;
  const uint8_t* rhs_base = a.rhs + (first_col >> a.log2_N0) * a.rhs_stride_bytes;

  // Rows past the end of the matrix are redirected to its last row: computed, never stored.
  auto piece_offset = [&](int64_t row, int64_t last, int64_t first, int log2_t0, int64_t stride_bytes, int32_t rb,
                          int log2_rb, int64_t kstep, int byte_in_chunk) -> uint32_t {
    row = min(row, last);
    const int64_t tile = (row >> log2_t0) - (first >> log2_t0);
    return (uint32_t)(tile * stride_bytes + (row & ((1 << log2_t0) - 1)) * rb + (byte_in_chunk >> log2_rb) * kstep +
                      (byte_in_chunk & (rb - 1)));
  };
  // Load t of wavefront w is group 4*t + w of its operand's groups of 64 slots, slice by slice.
  auto group_of = [&](int t, int slice_slots, int* slice, int* row, int* byte_in_chunk) {
    const int group = 4 * t + wave, per_slice = slice_slots / 64;
    *slice = group / per_slice;
    const int p = 64 * (group % per_slice) + lane;  // slot within the slice
    *row = 32 * (p / FRAG_SLOTS) + 16 * ((p / (16 * COLS)) & 1) + (p & 15);
    *byte_in_chunk = 16 * COLS * *slice + 16 * ((p >> 4) & (COLS - 1));
  };
  uint32_t a_off[A_LOADS], b_off[B_LOADS], a_lds[A_LOADS], b_lds[B_LOADS];
#pragma unroll
  for (int t = 0; t < A_LOADS; ++t) {
    int slice, row, byte_in_chunk;
    group_of(t, A_SLICE, &slice, &row, &byte_in_chunk);
    a_off[t] = piece_offset(first_row + row, total_rows - 1, first_row, a.log2_M0, a.lhs_stride_bytes, a.lhs_rb,
                            a.log2_lhs_rb, lhs_kstep, byte_in_chunk);
    a_lds[t] = (uint32_t)(64 * (4 * t + wave)) * 16;
  }
#pragma unroll
  for (int t = 0; t < B_LOADS; ++t) {
    int slice, row, byte_in_chunk;
    group_of(t, B_SLICE, &slice, &row, &byte_in_chunk);
    b_off[t] = piece_offset(first_col + row, total_cols - 1, first_col, a.log2_N0, a.rhs_stride_bytes, a.rhs_rb,
                            a.log2_rhs_rb, rhs_kstep, byte_in_chunk);
    b_lds[t] = (uint32_t)(A_PIECES + 64 * (4 * t + wave)) * 16;
  }

  acc_t acc[AMF][2];
#pragma unroll
  for (int i = 0; i < AMF; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  const int chunks = (int)(((int64_t)a.K << a.log2_lhs_rb) / CHUNK_BYTES);  // K is whole steps
  const int last_chunk = chunks - 1;

  auto issue_load = [&](int n, uint32_t stage_off, const uint8_t* la, const uint8_t* lb) {
    if (n < A_LOADS) load_to_lds(stage_off + a_lds[n], a_off[n], la);
    else load_to_lds(stage_off + b_lds[n - A_LOADS], b_off[n - A_LOADS], lb);
  };
  // This wavefront's operand registers for one chunk: fragment f, K-step kk.
  uint4 pa[AMF][KKW], pb[2][KKW], qa[AMF][KKW], qb[2][KKW];
  // Lane 32*h + r reads slot 16*COLS*(r >> 4) + 16*(2*kk + h) + (r & 15) of a fragment.
  const uint8_t* lane_a = (const uint8_t*)ring +
                          16 * (A_SLICE * wave + 16 * COLS * ((lane & 31) >> 4) + 16 * (lane >> 5) + (lane & 15));
  const uint8_t* lane_b = lane_a + 16 * (A_PIECES + (B_SLICE - A_SLICE) * wave);
  // Read number u of a step, in the order the next step consumes them: per K-step the rhs fragments, then the lhs.
  auto read_unit = [&](int u, const uint8_t* stage, uint4 (*fa)[KKW], uint4 (*fb)[KKW]) {
    const int kk = u / (AMF + 2), e = u % (AMF + 2);
    if (e < 2) fb[e][kk] = *(const uint4*)(stage + (lane_b - (const uint8_t*)ring) + (FRAG_SLOTS * e + 32 * kk) * 16);
    else fa[e - 2][kk] = *(const uint4*)(stage + (lane_a - (const uint8_t*)ring) + (FRAG_SLOTS * (e - 2) + 32 * kk) * 16);
  };

  const uint8_t* load_a = lhs_base + min(AHEAD, last_chunk) * lhs_chunk_bytes;
  const uint8_t* load_b = rhs_base + min(AHEAD, last_chunk) * rhs_chunk_bytes;
  int load_chunk = AHEAD;
  uint32_t load_stage_off = AHEAD * STAGE_BYTES % RING_BYTES;
  uint32_t read_stage_off = STAGE_BYTES;

  // One step, as in the kernel above: two MFMAs ahead of the wait and the barrier, then the loads of the chunk
  // AHEAD ahead and the LDS reads of the next chunk dealt out over four MFMAs, two MFMAs without memory work.
  auto step = [&](const uint4 (*cur_a)[KKW], const uint4 (*cur_b)[KKW], uint4 (*nxt_a)[KKW], uint4 (*nxt_b)[KKW]) {
    auto multiply = [&](int m) {
      const int kk = m / (AMF * 2), i = (m % (AMF * 2)) >> 1, j = m & 1;
      acc[i][j] = mfma<KIND>(cur_b[j][kk], cur_a[i][kk], acc[i][j]);
    };
    multiply(0);
    multiply(1);
    __builtin_amdgcn_sched_barrier(0);
    wait_loads_but<LOADS*(AHEAD - 2)>();
    __builtin_amdgcn_s_barrier();
    const uint8_t* stage = (const uint8_t*)ring + read_stage_off;
#pragma unroll
    for (int m = 2; m < 8; ++m) {
      const int slot = m - 2;
      if (slot < 4) {
#pragma unroll
        for (int n = slot * LOADS / 4; n < (slot + 1) * LOADS / 4; ++n) issue_load(n, load_stage_off, load_a, load_b);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = slot * READS / 4; u < (slot + 1) * READS / 4; ++u) read_unit(u, stage, nxt_a, nxt_b);
      }
      multiply(m);
      if (m == 7) {
        const bool more = load_chunk < last_chunk;
        load_a += more ? lhs_chunk_bytes : 0;
        load_b += more ? rhs_chunk_bytes : 0;
        ++load_chunk;
        load_stage_off = load_stage_off + STAGE_BYTES == RING_BYTES ? 0 : load_stage_off + STAGE_BYTES;
        read_stage_off = read_stage_off + STAGE_BYTES == RING_BYTES ? 0 : read_stage_off + STAGE_BYTES;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

#pragma unroll
  for (int c = 0; c < AHEAD; ++c) {
    const int idx = min(c, last_chunk);
#pragma unroll
    for (int n = 0; n < LOADS; ++n)
      issue_load(n, (uint32_t)c * STAGE_BYTES, lhs_base + idx * lhs_chunk_bytes, rhs_base + idx * rhs_chunk_bytes);
  }
  wait_loads_but<(AHEAD - 1) * LOADS>();
  __syncthreads();
#pragma unroll
  for (int u = 0; u < READS; ++u) read_unit(u, (const uint8_t*)ring, pa, pb);
  int kc = 0;
  for (; kc + 1 < chunks; kc += 2) {
    step(pa, pb, qa, qb);
    step(qa, qb, pa, pb);
  }
  if (kc < chunks) step(pa, pb, qa, qb);
  wait_loads_but<0>();
  __syncthreads();  // nobody reads operands from the ring any more

  // The four partial tiles, summed in wavefront order. Wavefront w ends up with the fragments
  // (OWN*(w >> 1) + o, w & 1), o < OWN: a block of (32*OWN) x 32 outputs. partial[((f*4 + w)*16 + v)][lane] is
  // accumulator register v of wavefront w's fragment f = 2*i + j.
  constexpr int OWN = AMF / 2;
  uint32_t* partial = (uint32_t*)ring;
#pragma unroll
  for (int f = 0; f < 2 * AMF; ++f) {
    const int i = f >> 1, j = f & 1;
    if (2 * (i / OWN) + j != wave) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const typename AccType<KIND>::scalar value = acc[i][j][v];
        partial[((f * 4 + wave) * 16 + v) * 64 + lane] = value_bits(value);
      }
    }
  }
  __syncthreads();
  acc_t total[OWN][1];
#pragma unroll
  for (int o = 0; o < OWN; ++o) {
    // (the wavefront's own partial, selected without indexing the accumulator array by a run-time value)
    acc_t own = acc[o][0];
#pragma unroll
    for (int w = 1; w < 4; ++w)
      if (wave == w) own = acc[OWN * (w >> 1) + o][w & 1];
    const int f = 2 * (OWN * (wave >> 1) + o) + (wave & 1);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      acc_t part;
      if (w == wave) {
        part = own;
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          typename AccType<KIND>::scalar value;
          set_from_bits(value, partial[((f * 4 + w) * 16 + v) * 64 + lane]);
          part[v] = value;
        }
      }
      if (w == 0) total[o][0] = part; else total[o][0] += part;
    }
  }
  store_block<KIND, false, NARROW, OWN, 1>(a, total, first_row + 32 * OWN * (wave >> 1), first_col + 32 * (wave & 1), lane);
}

// Whether the direct-to-LDS kernel covers the problem: every lane can load 16
// contiguous bytes (4-byte row pieces 4 rows at a time, an int4 rhs in pieces
// of 32 nibbles), and K is long enough.
template <bool RHS_I4, int G>
bool direct_covers(const MfmaArgs& m) {
  // K ending inside a chunk: not with an int4 rhs, and one full chunk at least.
  const int64_t row_bytes = (int64_t)m.K * m.lhs_rb;
  if (row_bytes % 64 != 0 && (RHS_I4 || row_bytes < 64)) return false;
  if (RHS_I4) return m.rhs_rb >= 16 && (uintptr_t)m.rhs % 16 == 0 && m.rhs_stride_bytes % 16 == 0;
  if (G == 16) return true;
  // One-byte pieces: tiles of 8 or 16 rows (a 16-byte piece is one or two k steps of a whole tile).
  if (G == 1)
    return m.log2_M0 >= 3 && m.log2_N0 >= 3 && (uintptr_t)m.lhs % 16 == 0 && (uintptr_t)m.rhs % 16 == 0 &&
           m.lhs_stride_bytes % 16 == 0 && m.rhs_stride_bytes % 16 == 0;
  // 16 / G rows of one k step make up a lane's 16 bytes: tiles at least that tall.
  return (G << m.log2_M0) >= 16 && (G << m.log2_N0) >= 16 && (uintptr_t)m.lhs % 16 == 0 &&
         (uintptr_t)m.rhs % 16 == 0 && m.lhs_stride_bytes % 16 == 0 && m.rhs_stride_bytes % 16 == 0;
}

void set_tile_grid(MfmaArgs* m, int block_rows, int block_cols, unsigned* grid) {
  const int64_t rows = (int64_t)m->M << m->log2_M0, cols = (int64_t)m->N << m->log2_N0;
  m->tile_rows = (int32_t)((rows + block_rows - 1) / block_rows);
  m->tile_cols = (int32_t)((cols + block_cols - 1) / block_cols);
  const int64_t tiles = (int64_t)m->tile_rows * m->tile_cols;
  *grid = (unsigned)(((tiles + 7) / 8) * 8);
}

// Direct-to-LDS kernel on (64*AM) x (64*BN) block tiles with a ring of STAGES stages.
template <int KIND, bool RHS_I4, bool NARROW, int G, int AM, int BN, int STAGES>
hipError_t launch_direct(MfmaArgs m, hipStream_t stream, bool staggered_tail = true) {
  unsigned grid;
  set_tile_grid(&m, 64 * AM, 64 * BN, &grid);
  constexpr int stage_pieces = 256 * AM + (RHS_I4 ? 128 : 256) * BN;
  constexpr size_t lds_bytes = (size_t)STAGES * 16 * stage_pieces;
  static_assert(lds_bytes <= 160 * 1024, "ring does not fit the LDS");
  void (*kernel)(const MfmaArgs) = mmt4d_mfma_direct_kernel<KIND, RHS_I4, NARROW, G, AM, BN, STAGES>;
  // The 256x256 tile with the staggered tail: K in whole chunks, enough of them.
  if constexpr (AM == 4 && BN == 4 && !RHS_I4 && G != 2 && KIND != kF32) {
    if (staggered_tail && ((int64_t)m.K * m.lhs_rb) % 64 == 0 && m.chunks >= 2 * STAGES) {
      // (Accumulating: read the destination during the loop where every one of the eight phases gets four steps.)
      if (m.accumulate && m.chunks >= STAGES + 9 * 4) kernel = mmt4d_mfma_direct_kernel<KIND, RHS_I4, NARROW, G, AM, BN, STAGES, 3>;
      else if (m.accumulate) kernel = mmt4d_mfma_direct_kernel<KIND, RHS_I4, NARROW, G, AM, BN, STAGES, 2>;
      else kernel = mmt4d_mfma_direct_kernel<KIND, RHS_I4, NARROW, G, AM, BN, STAGES, 1>;
    }
  }
  // Above 64 KiB of dynamic LDS the limit has to be raised (per device, so it
  // is simply done on every launch: it only sets a field).
  if (lds_bytes > 65536) {
    const hipError_t attr =
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr != hipSuccess) return attr;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds_bytes, stream, m);
  return hipGetLastError();
}

// The tiles with K split over the wavefronts. Returns the number of 32-row lhs fragments of the tile to use (2:
// few 64x64 tiles and a long K; 4: at most 128 lhs rows, one row of 128x64 tiles), or 0 for the ordinary kernels.
inline int split_k_tile(const MfmaArgs& m, bool int8) {
  const int64_t rows = (int64_t)m.M << m.log2_M0, cols = (int64_t)m.N << m.log2_N0;
  const int64_t row_bytes = (int64_t)m.K * m.lhs_rb;
  if (((rows + 63) / 64) * ((cols + 63) / 64) <= 128 && row_bytes % 256 == 0 && row_bytes >= 4096) return 2;
  // (bf16 128 x 14336 x 4096 27 -> 25 us, 96 rows 27 -> 23 us, 128 x 8192 x 8192 40 -> 36 us. Not with less K per
  // row, where the prologue and the summing of the partial tiles cost what the steps gain; not for int8, which does
  // twice the MFMA work per byte: 128 x 14336 x 8192 29 -> 31 us; not with more tiles than compute units, where
  // 128x128 tiles win: bf16 128 x 28672 x 4096 41 -> 49 us.)
  if (!int8 && rows > 64 && rows <= 128 && cols <= 256 * 64 && row_bytes % 128 == 0 && row_bytes >= 8192) return 4;
  return 0;
}

template <int KIND, bool NARROW, int AMF>
hipError_t launch_split_k(MfmaArgs m, hipStream_t stream) {
  unsigned grid;
  set_tile_grid(&m, 32 * AMF, 64, &grid);
  constexpr int lds_bytes = AMF == 2 ? 4 * 32768 : 6 * 24576;
  auto kernel = mmt4d_mfma_split_k_kernel<KIND, NARROW, AMF>;
  const hipError_t attr = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds_bytes, stream, m);
  return hipGetLastError();
}

// Register-staged kernel (any K, any alignment the plan admits).
template <int KIND, bool RHS_I4, bool NARROW, int G, int AM, int BN, int MIN_BLOCKS>
hipError_t launch_staged(MfmaArgs m, hipStream_t stream) {
  // 2- and 8-byte row pieces exist on the direct path only; the plan does not
  // admit problems that would need this kernel for them.
  if constexpr (G != 16 && G != 4) return hipErrorInvalidValue;
  else {
  unsigned grid;
  set_tile_grid(&m, 64 * AM, 64 * BN, &grid);
  // K ending inside a chunk needs the kernel variant with the zero-filling tail step.
  const bool tail = ((int64_t)m.K * m.lhs_rb) % 64 != 0;
  if (tail) {
    hipLaunchKernelGGL((mmt4d_mfma_kernel<KIND, RHS_I4, NARROW, G, AM, BN, MIN_BLOCKS, true>), dim3(grid),
                       dim3(256), 0, stream, m);
  } else {
    hipLaunchKernelGGL((mmt4d_mfma_kernel<KIND, RHS_I4, NARROW, G, AM, BN, MIN_BLOCKS, false>), dim3(grid),
                       dim3(256), 0, stream, m);
  }
  return hipGetLastError();
  }
}

// Picks the block tile. Larger tiles move fewer operand bytes per multiply
// through L2 -> LDS and run the matrix pipe longer between barriers, smaller
// ones spread a problem over more compute units. The estimate is
//   (workgroups per compute unit, rounded up) x (tile area) / (tile efficiency),
// with the efficiencies measured at saturation on bf16 16x16x8 operands
// (TFLOP/s at 2048 x 14336 x 4096: 256x256 1003, 256x128 905, 128x128 851,
// 128x64 607, 64x64 529). It reproduces the measured best tile on every shape
// tried (128 .. 4096 rows against 14336 columns, 1024^2 .. 4096^2 squares).
struct TileChoice {
  int am, bn;
  float efficiency;
  bool direct_only;  // no register-staged instantiation of this shape
};

template <bool RHS_I4>
int choose_tile(const MfmaArgs& m, bool direct, const TileChoice** chosen) {
  static const TileChoice kTiles[] = {
      {4, 4, 1003.f, false}, {4, 2, 905.f, true}, {2, 2, 851.f, false}, {2, 1, 607.f, true}, {1, 1, 529.f, false},
      {1, 2, 600.f, true}};
  const int64_t rows = (int64_t)m.M << m.log2_M0, cols = (int64_t)m.N << m.log2_N0;
  int best = -1;
  double best_cost = 0;
  for (int i = 0; i < (int)(sizeof kTiles / sizeof kTiles[0]); ++i) {
    const TileChoice& t = kTiles[i];
    if (t.direct_only && !direct) continue;
    if (RHS_I4 && t.bn < 2 && t.direct_only) continue;  // the int4 direct path needs a rhs fragment per wavefront
    if (!RHS_I4 && t.am == 1 && t.bn == 2) continue;    // 64x128 exists for the int4 rhs only (in place of 128x64)
    // The int4 64x64 tile exists only register-staged, at less than half the
    // rate of the direct 64x128 one on the same problem.
    if (RHS_I4 && direct && t.am == 1 && t.bn == 1) continue;
    const int64_t br = 64 * t.am, bc = 64 * t.bn;
    const int64_t workgroups = ((rows + br - 1) / br) * ((cols + bc - 1) / bc);
    const double cost = (double)((workgroups + 255) / 256) * (double)(br * bc) / t.efficiency;
    if (best < 0 || cost < best_cost) {
      best = i;
      best_cost = cost;
    }
  }
  *chosen = &kTiles[best];
  return best;
}

template <int KIND, bool RHS_I4, int G, bool NARROW>
hipError_t launch_variant(const MfmaArgs& m, hipStream_t stream, const char** name) {
  const bool direct = direct_covers<RHS_I4, G>(m);
  if constexpr (G == 16 && !RHS_I4 && KIND != kF32) {
    const int split = direct ? split_k_tile(m, KIND == kI8) : 0;
    if (split == 2) {
      *name = "mmt4d_mfma_64x64_split_k";
      return launch_split_k<KIND, NARROW, 2>(m, stream);
    }
    if (split == 4) {
      *name = "mmt4d_mfma_128x64_split_k";
      return launch_split_k<KIND, NARROW, 4>(m, stream);
    }
  }
  const TileChoice* tile;
  switch (choose_tile<RHS_I4>(m, direct, &tile)) {
    case 0:
      *name = "mmt4d_mfma_256x256";
#ifndef UK_STAGES_256
#define UK_STAGES_256 4
#endif
      if (direct) return launch_direct<KIND, RHS_I4, NARROW, G, 4, 4, UK_STAGES_256>(m, stream);
      return launch_staged<KIND, RHS_I4, NARROW, G, 4, 4, 1>(m, stream);
    case 1:
      *name = "mmt4d_mfma_256x128";
      return launch_direct<KIND, RHS_I4, NARROW, G, 4, 2, 4>(m, stream);
    case 2:
      *name = "mmt4d_mfma_128x128";
      if (direct) return launch_direct<KIND, RHS_I4, NARROW, G, 2, 2, 4>(m, stream);
      return launch_staged<KIND, RHS_I4, NARROW, G, 2, 2, 2>(m, stream);
    case 5:
      *name = "mmt4d_mfma_64x128";
      if constexpr (RHS_I4) return launch_direct<KIND, RHS_I4, NARROW, G, 1, 2, 8>(m, stream);
      [[fallthrough]];
    case 3:
      *name = "mmt4d_mfma_128x64";
      if constexpr (!RHS_I4) return launch_direct<KIND, RHS_I4, NARROW, G, 2, 1, 8>(m, stream);
      [[fallthrough]];
    default:
      *name = "mmt4d_mfma_64x64";
      if constexpr (!RHS_I4) {
        if (direct) return launch_direct<KIND, RHS_I4, NARROW, G, 1, 1, 8>(m, stream);
      }
      return launch_staged<KIND, RHS_I4, NARROW, G, 1, 1, 2>(m, stream);
  }
}

}  // namespace
#endif  // UK_MFMA_KERNEL_BODIES

}  // namespace uk

#endif  // IREE_AMD_CSRC_MMT4D_MFMA_KERNELS_H_
