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
// Data flow per chunk: global -> registers (issued two chunks ahead) -> LDS,
// stored fragment-major so that a wavefront fetches one 32-row x 32-byte MFMA
// operand with a single conflict-free 128-bit LDS read per lane -> registers
// (read one chunk ahead) -> MFMA.
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
typedef int v16i32 __attribute__((ext_vector_type(16)));
typedef float v16f32 __attribute__((ext_vector_type(16)));
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
struct AccType { typedef v16i32 type; typedef int scalar; };
template <> struct AccType<kF16> { typedef v16f32 type; typedef float scalar; };
template <> struct AccType<kBF16> { typedef v16f32 type; typedef float scalar; };

template <int KIND>
__device__ __forceinline__ typename AccType<KIND>::type mfma(uint4 row_operand, uint4 col_operand,
                                                             typename AccType<KIND>::type acc) {
  if constexpr (KIND == kI8) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(v4i32, row_operand),
                                                 __builtin_bit_cast(v4i32, col_operand), acc, 0, 0, 0);
  } else if constexpr (KIND == kF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8f16, row_operand),
                                                  __builtin_bit_cast(v8f16, col_operand), acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf16, row_operand),
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

template <int KIND, bool RHS_I4, int G, int AM, int BN, int MIN_BLOCKS, bool TAIL>
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
      for (int j = 0; j < BN; ++j) acc[i][j] = mfma<KIND>(fb[j][kk], fa[i][kk], acc[i][j]);
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

  // Epilogue. Lane l holds, for fragment (i, j): lhs row 32*i + (l & 31) and, in
  // accumulator registers 4*q .. 4*q+3, rhs rows 32*j + 8*q + 4*(l >> 5) + {0..3}
  // of the wavefront's sub-block: four consecutive j0 of one output row.
  typedef typename AccType<KIND>::scalar scalar_t;
  typedef scalar_t quad_t __attribute__((ext_vector_type(4)));
  const int64_t row0 = first_row + wave_m * (32 * AM) + (lane & 31);
  const int64_t col0 = first_col + wave_n * (32 * BN) + 4 * (lane >> 5);
  const int64_t tile_elems = (int64_t)M0 * N0;
#pragma unroll
  for (int i = 0; i < AM; ++i) {
    const int64_t row = row0 + 32 * i;
    if (row >= total_rows) continue;
    const int64_t row_off = (row >> a.log2_M0) * a.out_stride0 + ((row & (M0 - 1)) << a.log2_N0);
#pragma unroll
    for (int j = 0; j < BN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = col0 + 32 * j + 8 * q;
        if (col >= total_cols) continue;
        quad_t* dst =
            (quad_t*)(a.out + 4 * (row_off + (col >> a.log2_N0) * tile_elems + (col & (N0 - 1))));
        quad_t v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                    acc[i][j][4 * q + 3]};
        if constexpr (RHS_I4) v = v >> 4;
        if (a.accumulate) v += *dst;
        *dst = v;
      }
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
    if (lhs_rb < 16 || lhs_rb > 64) return false;
    gather = 16;
  } else if (lhs_rb >= 16 && lhs_rb <= 64) {
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
  // Per-piece offsets from a workgroup's first tile are kept in 32 bits.
  const int64_t lhs_reach = ((256 >> lm0) + 1) * lhs_stride_bytes + 80 * ((int64_t)lhs_rb << lm0);
  const int64_t rhs_reach = ((256 >> ln0) + 1) * rhs_stride_bytes + 80 * ((int64_t)rhs_rb << ln0);
  if (lhs_reach >= (1ll << 32) || rhs_reach >= (1ll << 32)) return false;
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

template <int KIND, bool RHS_I4, int G, int AM, int BN, int MIN_BLOCKS>
hipError_t launch_tile(MfmaArgs m, hipStream_t stream) {
  const int64_t rows = (int64_t)m.M << m.log2_M0, cols = (int64_t)m.N << m.log2_N0;
  m.tile_rows = (int32_t)((rows + 64 * AM - 1) / (64 * AM));
  m.tile_cols = (int32_t)((cols + 64 * BN - 1) / (64 * BN));
  const int64_t tiles = (int64_t)m.tile_rows * m.tile_cols;
  const unsigned grid = (unsigned)(((tiles + 7) / 8) * 8);
  // K ending inside a chunk needs the kernel variant with the zero-filling tail step.
  const bool tail = ((int64_t)m.K * m.lhs_rb) % 64 != 0;
  if (tail) {
    hipLaunchKernelGGL((mmt4d_mfma_kernel<KIND, RHS_I4, G, AM, BN, MIN_BLOCKS, true>), dim3(grid),
                       dim3(256), 0, stream, m);
  } else {
    hipLaunchKernelGGL((mmt4d_mfma_kernel<KIND, RHS_I4, G, AM, BN, MIN_BLOCKS, false>), dim3(grid),
                       dim3(256), 0, stream, m);
  }
  return hipGetLastError();
}

// Picks the largest block tile that still gives every compute unit work.
template <int KIND, bool RHS_I4, int G>
hipError_t launch_variant(const MfmaArgs& m, hipStream_t stream, const char** name) {
  const int64_t rows = (int64_t)m.M << m.log2_M0, cols = (int64_t)m.N << m.log2_N0;
  auto tiles = [&](int br, int bc) { return ((rows + br - 1) / br) * ((cols + bc - 1) / bc); };
  if (tiles(256, 256) >= 200) {
    *name = "mmt4d_mfma_256x256";
    return launch_tile<KIND, RHS_I4, G, 4, 4, 1>(m, stream);
  }
  if (tiles(128, 128) >= 200 || (rows > 64 && cols > 64)) {
    *name = "mmt4d_mfma_128x128";
    return launch_tile<KIND, RHS_I4, G, 2, 2, 2>(m, stream);
  }
  *name = "mmt4d_mfma_64x64";
  return launch_tile<KIND, RHS_I4, G, 1, 1, 2>(m, stream);
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
