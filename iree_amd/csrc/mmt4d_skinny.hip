// mmt4d for skinny left-hand sides in the narrow tile shapes that the
// reference's CPU targets pick for them: few lhs rows in total (e.g.
// M0 = 1, 2, 4 with M = 1) and row pieces (K0 elements) of 2, 4 or 8 bytes:
// the x86-64 1x16x2 int8 / bf16 and 1x16x1 f16 / f32 tiles, the Arm 1x8x4 and
// 1x8x8 int8 tiles and their 2- and 4-row siblings (mmt4d_x86_64_tiles.inl,
// mmt4d_arm_64_tiles.inl). An HBM-bandwidth kernel.
//
// With pieces that short, 16 contiguous bytes of the rhs are several rows of
// one k step, not one row: the wrong way round for an MFMA operand, and the
// matrix kernels cannot load an lhs whose tiles are narrower than 16 bytes per
// k step at all. Here nothing is transposed. The rhs of one tile row
// (N0 rows x K k steps, one contiguous stream) is read 16 bytes per lane, and
// each lane multiplies the 16 / G rows it holds with the lhs pieces of its
// k step on the VALU (v_dot4_i32_i8, v_dot2_i32_i16, FMAs on 16-bit floats
// widened to f32), keeping one accumulator per (lhs row, rhs row). The lhs is small and comes through the
// caches. At the end the lanes that hold the same rhs rows (they differ in
// k step) are summed with a butterfly of lane exchanges, the wavefronts of the
// workgroup (which split the stream between them) through LDS, both in a
// fixed order, so results do not depend on scheduling.
//
// f16f16f16 and bf16bf16bf16 are taken with the flag that skips the roundings
// between k steps (mmt4d_tile_generic.c:229-286, 319-376): f32 accumulators,
// one rounding to the 16-bit output at the end.
//
// Also here, because nothing else takes them but the generic kernel:
// s16s16s32 (v_dot2_i32_i16) and s16u4s32, the x86-64 VNNI tile 1x32x8 for
// 4-bit weights against 16-bit activations (mmt4d_x86_64_tiles.inl; unsigned
// nibbles, element 2j in the low nibble of byte j, mmt4d_tile_generic.c:108-142):
// a lane's 16 bytes are 4 rows x 8 nibbles of one k step, each byte is spread
// to a pair of 16-bit values and multiplied with the matching pair of the lhs.
// And s8s4s32 with the Arm tiles Mx8x8 and Mx8x16 (mmt4d_arm_64_tiles.inl;
// signed nibbles, mmt4d_tile_generic.c:11-51): the even and the odd nibbles of
// a dword are isolated in the high nibbles of two dwords (int8 values 16 times
// the weights) and multiplied with the even resp. odd lhs bytes of the k step,
// which are gathered once per lhs piece; the sums are shifted right by 4 at
// the end (exact; K * K0 < 131072 keeps 16x the sums inside int32). The Arm
// baseline tiles Mx16x2 have one byte per rhs row and k step: a lane's 16 bytes
// are 16 rows, and each row's two weights (x16, as above) are put beside each
// other in a dword for one v_dot4_i32_i8 with the lhs pair.
// And s16s8s32, for which the reference has the generic tile only
// (mmt4d_tile_generic.c:145-176): the rhs bytes are sign-extended to 16-bit
// pairs (v_perm_b32 with its sign-byte selectors) for v_dot2_i32_i16.
//
// And s8s8s32 Mx8x1 with M0 = 1, 2, 4 (the Arm baseline tiles without dot
// products, mmt4d_arm_64_tiles.inl:38-40): a k step of the rhs is 8 bytes, so a
// lane's 16 bytes are the tile's 8 rows at two consecutive k steps; each row's
// two bytes are put beside each other for one v_dot4_i32_i8 with the two lhs
// bytes of those k steps.
//
// More than 8 lhs rows are worked off in slabs of 8, each streaming the rhs
// again: what the block kernels can load they do faster (the caller prefers
// them), what they cannot is still far better off here than with one thread
// per output element.
#include "uk_device.h"
#include "uk_internal.h"

namespace uk {
namespace {

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef _Float16 v2f16 __attribute__((ext_vector_type(2)));
typedef short v2i16 __attribute__((ext_vector_type(2)));

enum Kind { kI8 = 0, kF16 = 1, kBF16 = 2, kF32 = 3, kI16 = 4, kI16U4 = 5, kI8I4 = 6, kI16I8 = 7 };

struct SkinnyArgs {
  const uint8_t* lhs;
  const uint8_t* rhs;
  uint8_t* out;
  int64_t lhs_stride_bytes, rhs_stride_bytes;
  int64_t out_stride0;  // elements
  int64_t tile_bytes;   // K * N0 * (bytes of an rhs row piece): one rhs tile row
  int32_t rows;         // M * M0
  int32_t row0;         // first lhs row of this launch (the kernel covers rows row0 .. row0 + ROWS - 1)
  int32_t N, K;
  int32_t log2_M0, log2_N0;
  int32_t accumulate;
};

template <int KIND> struct Acc { typedef float type; };
template <> struct Acc<kI8> { typedef int32_t type; };
template <> struct Acc<kI16> { typedef int32_t type; };
template <> struct Acc<kI16U4> { typedef int32_t type; };
template <> struct Acc<kI8I4> { typedef int32_t type; };
template <> struct Acc<kI16I8> { typedef int32_t type; };
// The lhs piece of one k step in registers. Same bytes as an rhs piece (G, zero-extended to two dwords), except:
// s16u4s32: 8 values of 16 bits against 8 nibbles; s8s4s32: 8 or 16 bytes against as many nibbles, kept as one
// dword of the even and one of the odd bytes per 8 (2 bytes as they are); s16s8s32: twice the bytes of the rhs piece.
template <int KIND> struct LhsPiece { typedef uint2 type; };
template <> struct LhsPiece<kI16U4> { typedef uint4 type; };
template <> struct LhsPiece<kI8I4> { typedef uint4 type; };
template <> struct LhsPiece<kI16I8> { typedef uint4 type; };

__device__ __forceinline__ int32_t dot2_i16(uint32_t a, uint32_t b, int32_t c) {
  return __builtin_amdgcn_sdot2(__builtin_bit_cast(v2i16, a), __builtin_bit_cast(v2i16, b), c, false);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
__device__ __forceinline__ float f16_lo(uint32_t w) { return (float)__builtin_bit_cast(v2f16, w)[0]; }
__device__ __forceinline__ float f16_hi(uint32_t w) { return (float)__builtin_bit_cast(v2f16, w)[1]; }

template <int KIND, int G>
__device__ __forceinline__ typename LhsPiece<KIND>::type load_lhs_piece(const uint8_t* p) {
  if constexpr (KIND == kI16U4) return *(const uint4*)p;
  else if constexpr (KIND == kI16I8) {
    if constexpr (G == 2) return make_uint4(*(const uint32_t*)p, 0, 0, 0);
    else if constexpr (G == 4) {
      const uint2 half = *(const uint2*)p;
      return make_uint4(half.x, half.y, 0, 0);
    } else return *(const uint4*)p;
  } else if constexpr (KIND == kI8I4 && G == 1) return make_uint4(*(const uint16_t*)p, 0, 0, 0);
  else if constexpr (KIND == kI8I4) {
    uint4 raw = make_uint4(0, 0, 0, 0);
    if constexpr (G == 4) {
      const uint2 half = *(const uint2*)p;
      raw.x = half.x; raw.y = half.y;
    } else {
      raw = *(const uint4*)p;
    }
    return make_uint4(__builtin_amdgcn_perm(raw.y, raw.x, 0x06040200u), __builtin_amdgcn_perm(raw.y, raw.x, 0x07050301u),
                      __builtin_amdgcn_perm(raw.w, raw.z, 0x06040200u), __builtin_amdgcn_perm(raw.w, raw.z, 0x07050301u));
  } else if constexpr (G == 2) return make_uint2(*(const uint16_t*)p, 0);
  else if constexpr (G == 4) return make_uint2(*(const uint32_t*)p, 0);
  else return *(const uint2*)p;
}

// acc[r] += (row r of the 16 / G rows in `v`) . (lhs piece l), all of one k step.
template <int KIND, int G>
__device__ __forceinline__ void multiply_piece(const uint4 v, const typename LhsPiece<KIND>::type l,
                                               typename Acc<KIND>::type* acc) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  if constexpr (KIND == kI8I4 && G == 1) {
    // 16 rows of two nibbles each against the lhs pair in the low half of l.x.
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t evens = (w[d] << 4) & 0xF0F0F0F0u, odds = w[d] & 0xF0F0F0F0u;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        // byte 0: row r of `evens`, byte 1: row r of `odds`, zeros above
        const uint32_t pair = __builtin_amdgcn_perm(odds, evens, 0x0C0C0400u + 0x0101u * r);
        acc[4 * d + r] = __builtin_amdgcn_sdot4((int)pair, (int)l.x, acc[4 * d + r], false);
      }
    }
  } else if constexpr (KIND == kI16I8) {
    const uint32_t lhs[4] = {l.x, l.y, l.z, l.w};
    // The four bytes of a dword as two pairs of 16-bit values. The selectors 8..11 of
    // v_perm_b32 give the sign of bytes 1, 3 (second operand) and 5, 7 (first operand)
    // as 0x00 or 0xFF; the dword shifted up by a byte has bytes 0 and 2 at 5 and 7.
    uint32_t pairs[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pairs[2 * i] = __builtin_amdgcn_perm(w[i] << 8, w[i], 0x08010A00u);
      pairs[2 * i + 1] = __builtin_amdgcn_perm(w[i] << 8, w[i], 0x09030B02u);
    }
    constexpr int PPR = G / 2;  // pairs per row piece
#pragma unroll
    for (int r = 0; r < 16 / G; ++r)
#pragma unroll
      for (int q = 0; q < PPR; ++q) acc[r] = dot2_i16(pairs[r * PPR + q], lhs[q], acc[r]);
  } else if constexpr (KIND == kI8I4) {
    static_assert(G == 4 || G == 8, "8 or 16 nibbles per row piece");
    const uint32_t lhs[4] = {l.x, l.y, l.z, l.w};
#pragma unroll
    for (int i = 0; i < 16 / G; ++i) {
#pragma unroll
      for (int d = 0; d < G / 4; ++d) {
        const uint32_t nibbles = w[i * (G / 4) + d];
        acc[i] = __builtin_amdgcn_sdot4((int)((nibbles << 4) & 0xF0F0F0F0u), (int)lhs[2 * d], acc[i], false);
        acc[i] = __builtin_amdgcn_sdot4((int)(nibbles & 0xF0F0F0F0u), (int)lhs[2 * d + 1], acc[i], false);
      }
    }
  } else if constexpr (KIND == kI16U4) {
    static_assert(G == 4, "8 nibbles per row piece");
    const uint32_t lhs[4] = {l.x, l.y, l.z, l.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        // byte b of the row: its low nibble to bits 0..3, its high nibble to bits 16..19
        const uint32_t twice = __builtin_amdgcn_perm(0, w[i], 0x0C000C00u + 0x00010001u * b);
        const uint32_t pair = (twice & 0xFu) | ((twice >> 4) & 0x000F0000u);
        acc[i] = dot2_i16(pair, lhs[b], acc[i]);
      }
    }
  } else if constexpr (KIND == kI16) {
    if constexpr (G == 2) {
      // Two rows per dword: the lhs value in the low resp. high half, zero in the other.
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] = dot2_i16(w[i], l.x, acc[2 * i]);
        acc[2 * i + 1] = dot2_i16(w[i], l.x << 16, acc[2 * i + 1]);
      }
    } else if constexpr (G == 4) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = dot2_i16(w[i], l.x, acc[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[i] = dot2_i16(w[2 * i + 1], l.y, dot2_i16(w[2 * i], l.x, acc[i]));
    }
  } else if constexpr (KIND == kI8 && G == 1) {
    // 8 rows at k step 2j (bytes 0..7) and at 2j + 1 (bytes 8..15); l.x holds the two lhs bytes.
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const uint32_t pair = __builtin_amdgcn_perm(w[2 + (r >> 2)], w[r >> 2], 0x0C0C0400u + 0x0101u * (r & 3));
      acc[r] = __builtin_amdgcn_sdot4((int)pair, (int)l.x, acc[r], false);
    }
  } else if constexpr (KIND == kI8) {
    if constexpr (G == 2) {
      // Two rows per dword: the lhs pair in the low resp. high half, zeros in the other.
      const int lo = (int)l.x, hi = (int)(l.x << 16);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] = __builtin_amdgcn_sdot4((int)w[i], lo, acc[2 * i], false);
        acc[2 * i + 1] = __builtin_amdgcn_sdot4((int)w[i], hi, acc[2 * i + 1], false);
      }
    } else if constexpr (G == 4) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_sdot4((int)w[i], (int)l.x, acc[i], false);
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        acc[i] = __builtin_amdgcn_sdot4((int)w[2 * i], (int)l.x, acc[i], false);
        acc[i] = __builtin_amdgcn_sdot4((int)w[2 * i + 1], (int)l.y, acc[i], false);
      }
    }
  } else if constexpr (KIND == kF32) {
    if constexpr (G == 4) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(__uint_as_float(w[i]), __uint_as_float(l.x), acc[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        acc[i] = fmaf(__uint_as_float(w[2 * i]), __uint_as_float(l.x), acc[i]);
        acc[i] = fmaf(__uint_as_float(w[2 * i + 1]), __uint_as_float(l.y), acc[i]);
      }
    }
  } else {
    // 16-bit floats, widened to f32 (exact) and accumulated in f32 in k0 order.
    auto lo = [](uint32_t x) { return KIND == kF16 ? f16_lo(x) : bf16_lo(x); };
    auto hi = [](uint32_t x) { return KIND == kF16 ? f16_hi(x) : bf16_hi(x); };
    if constexpr (G == 2) {
      const float l0 = lo(l.x);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] = fmaf(lo(w[i]), l0, acc[2 * i]);
        acc[2 * i + 1] = fmaf(hi(w[i]), l0, acc[2 * i + 1]);
      }
    } else if constexpr (G == 4) {
      const float l0 = lo(l.x), l1 = hi(l.x);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(hi(w[i]), l1, fmaf(lo(w[i]), l0, acc[i]));
    } else {
      const float l0 = lo(l.x), l1 = hi(l.x), l2 = lo(l.y), l3 = hi(l.y);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        acc[i] = fmaf(hi(w[2 * i]), l1, fmaf(lo(w[2 * i]), l0, acc[i]));
        acc[i] = fmaf(hi(w[2 * i + 1]), l3, fmaf(lo(w[2 * i + 1]), l2, acc[i]));
      }
    }
  }
}

__device__ __forceinline__ int32_t exchange(int32_t v, int lane_xor) { return __shfl_xor(v, lane_xor, 64); }
__device__ __forceinline__ float exchange(float v, int lane_xor) { return __shfl_xor(v, lane_xor, 64); }

// G: bytes of a row piece; ROWS: lhs rows the kernel keeps accumulators for
// (a.rows <= ROWS); UNROLL: 1 KiB blocks of the rhs stream a wavefront has in
// flight; NARROW: the output has the 16-bit type of the operands. One
// workgroup of four wavefronts per rhs tile row.
template <int KIND, int G, int ROWS, int UNROLL, bool NARROW>
__global__ __launch_bounds__(256) void mmt4d_skinny_kernel(const SkinnyArgs a) {
  static_assert(!NARROW || KIND == kF16 || KIND == kBF16, "16-bit outputs are floats");
  typedef typename Acc<KIND>::type acc_t;
  // (One-byte pieces of int8: 8-row tiles, two k steps per lane.)
  constexpr bool TWO_KSTEPS = KIND == kI8 && G == 1;
  constexpr int R = TWO_KSTEPS ? 8 : 16 / G;  // rhs rows in a lane's 16 bytes
  __shared__ acc_t partial[4][ROWS][32];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int32_t M0 = 1 << a.log2_M0, N0 = 1 << a.log2_N0;
  // One k step of the rhs is N0 * G bytes = `lanes_per_kstep` lanes; a block of
  // 1 KiB holds whole k steps, so a lane keeps its rows from block to block.
  const int log2_kstep_bytes = a.log2_N0 + (G == 1 ? 0 : (G == 2 ? 1 : (G == 4 ? 2 : 3)));
  const int log2_lanes_per_kstep = TWO_KSTEPS ? 0 : log2_kstep_bytes - 4;
  const int32_t kstep_in_block = TWO_KSTEPS ? 2 * lane : lane >> log2_lanes_per_kstep;
  constexpr int LHS_G = KIND == kI16U4 ? 16 : (KIND == kI8I4 || KIND == kI16I8 ? 2 * G : G);  // bytes of an lhs row piece
  const int32_t lhs_kstep_bytes = LHS_G << a.log2_M0;

  const uint8_t* rhs_tile = a.rhs + (int64_t)blockIdx.x * a.rhs_stride_bytes;
  const uint8_t* lhs_row[ROWS];
#pragma unroll
  for (int m = 0; m < ROWS; ++m) {
    const int row = a.row0 + m < a.rows ? a.row0 + m : a.rows - 1;  // clamp: computed, not stored
    lhs_row[m] = a.lhs + (int64_t)(row >> a.log2_M0) * a.lhs_stride_bytes + (row & (M0 - 1)) * LHS_G;
  }

  acc_t acc[ROWS][R];
#pragma unroll
  for (int m = 0; m < ROWS; ++m)
#pragma unroll
    for (int r = 0; r < R; ++r) acc[m][r] = 0;

  const int64_t blocks = (a.tile_bytes + 1023) >> 10;
  for (int64_t j0 = wave; j0 < blocks; j0 += 4 * UNROLL) {
    uint4 v[UNROLL];
    typename LhsPiece<KIND>::type l[UNROLL][ROWS];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t off = ((j0 + 4 * u) << 10) + 16 * lane;
      const bool inside = off < a.tile_bytes;
      v[u] = make_uint4(0, 0, 0, 0);
      if (TWO_KSTEPS && inside && off + 16 > a.tile_bytes) {
        // An odd K: the stream ends after this lane's first k step.
        const uint2 half = *(const uint2*)(rhs_tile + off);
        v[u].x = half.x;
        v[u].y = half.y;
      } else if (inside) {
        v[u] = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4i32*)(rhs_tile + off)));
      }
      // The lhs piece of this lane's k step.
      const int64_t kstep = inside ? ((j0 + 4 * u) << (10 - log2_kstep_bytes)) + kstep_in_block : 0;
#pragma unroll
      for (int m = 0; m < ROWS; ++m) {
        if constexpr (TWO_KSTEPS) {
          const uint8_t* p = lhs_row[m] + kstep * lhs_kstep_bytes;
          const uint32_t second = kstep + 1 < a.K ? p[lhs_kstep_bytes] : 0u;
          l[u][m] = make_uint2((uint32_t)p[0] | (second << 8), 0);
        } else {
          l[u][m] = load_lhs_piece<KIND, G>(lhs_row[m] + kstep * lhs_kstep_bytes);
        }
        if (!inside) l[u][m] = typename LhsPiece<KIND>::type{};  // 0 * 0, whatever the lhs holds there
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int m = 0; m < ROWS; ++m) multiply_piece<KIND, G>(v[u], l[u][m], acc[m]);
  }

  // Lanes that are a multiple of lanes_per_kstep apart hold the same rhs rows.
  for (int s = 1 << log2_lanes_per_kstep; s < 64; s <<= 1) {
#pragma unroll
    for (int m = 0; m < ROWS; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r) acc[m][r] += exchange(acc[m][r], s);
  }
  if (lane < (1 << log2_lanes_per_kstep)) {
#pragma unroll
    for (int m = 0; m < ROWS; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r) partial[wave][m][R * lane + r] = acc[m][r];
  }
  __syncthreads();
  const int t = threadIdx.x;
  const int slab_row = t >> a.log2_N0, j0 = t & (N0 - 1);
  const int m = a.row0 + slab_row;
  if (slab_row < ROWS && m < a.rows) {
    acc_t sum = partial[0][slab_row][j0];
    sum += partial[1][slab_row][j0];
    sum += partial[2][slab_row][j0];
    sum += partial[3][slab_row][j0];
    if constexpr (KIND == kI8I4) sum >>= 4;
    const int64_t index = (int64_t)(m >> a.log2_M0) * a.out_stride0 +
                          ((int64_t)blockIdx.x << (a.log2_M0 + a.log2_N0)) + ((m & (M0 - 1)) << a.log2_N0) + j0;
    if constexpr (NARROW) {
      constexpr int EBITS = KIND == kF16 ? 5 : 8;
      uint16_t* dst = (uint16_t*)a.out + index;
      if (a.accumulate) sum += widen16<EBITS>(*dst);
      *dst = narrow16<EBITS>(sum);
    } else {
      acc_t* dst = (acc_t*)a.out + index;
      if (a.accumulate) sum += *dst;
      *dst = sum;
    }
  }
}

int log2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int l = 0;
  while ((1ll << l) < v) ++l;
  return l;
}

bool make_args(const Mmt4dArgs& a, bool probe_only, int* kind, int* piece_bytes, bool* narrow, SkinnyArgs* s) {
  int elem_bytes;
  *narrow = false;
  const bool skip_roundings = a.flags & IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS;
  switch (a.flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: *kind = kI8; elem_bytes = 1; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: *kind = kF16; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *kind = kBF16; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: *kind = kF32; elem_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S16S32: *kind = kI16; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16U4S32: *kind = kI16U4; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: *kind = kI8I4; elem_bytes = 1; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S8S32: *kind = kI16I8; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16:
      if (!skip_roundings) return false;
      *kind = kF16; elem_bytes = 2; *narrow = true;
      break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16:
      if (!skip_roundings) return false;
      *kind = kBF16; elem_bytes = 2; *narrow = true;
      break;
    default: return false;
  }
  const bool u4 = *kind == kI16U4, i4 = *kind == kI8I4, i16i8 = *kind == kI16I8;
  if (u4 && a.K0 != 8) return false;
  if (i4 && a.K0 != 2 && a.K0 != 8 && a.K0 != 16) return false;
  const int g = u4 ? 4 : (i4 ? a.K0 / 2 : (i16i8 ? a.K0 : a.K0 * elem_bytes));  // bytes of an rhs row piece
  const int lhs_g = u4 ? 16 : (i4 ? a.K0 : (i16i8 ? 2 * a.K0 : g));
  // int8 Mx8x1 (8x8x1 goes to the matrix kernels first, see mmt4d_skinny_preferred, and comes here when they cannot
  // load it: K shorter than a chunk, misaligned lhs).
  const bool two_ksteps = *kind == kI8 && g == 1 && a.N0 == 8 && a.M0 <= 8;
  if (g != 2 && g != 4 && g != 8 && !(i4 && g == 1) && !two_ksteps) return false;
  const int lm0 = log2_exact(a.M0), ln0 = log2_exact(a.N0);
  // A k step of the rhs must be whole 16-byte vectors (or half of one, above).
  if (lm0 < 0 || ln0 < 0 || a.M0 > 16 || a.N0 > 32 || (a.N0 * g < 16 && !two_ksteps)) return false;
  *piece_bytes = g;
  // What no matrix kernel takes.
  if (probe_only) return a.M0 * lhs_g < 16 || *kind == kI16 || u4 || i16i8 || (i4 && a.K0 < 16);
  // 16x-scaled int4 accumulation must not overflow int32.
  if (i4 && (int64_t)a.K * a.K0 >= 131072) return false;
  if (a.M * a.M0 > 0x7FFFFFFF || a.M <= 0 || a.K <= 0 || a.N <= 0 || a.N > 0x7FFFFFFF) return false;
  if ((u4 || i4) && (a.rhs_stride0 & 1)) return false;
  const int64_t lhs_stride_bytes = a.lhs_stride0 * elem_bytes;
  const int64_t rhs_stride_bytes = (u4 || i4) ? a.rhs_stride0 / 2 : (i16i8 ? a.rhs_stride0 : a.rhs_stride0 * elem_bytes);
  if ((uintptr_t)a.rhs % 16 || (a.N > 1 && rhs_stride_bytes % 16)) return false;
  if ((uintptr_t)a.lhs % lhs_g || (a.M > 1 && lhs_stride_bytes % lhs_g)) return false;
  if ((uintptr_t)a.out % (*narrow ? 2 : 4)) return false;
  s->lhs = a.lhs; s->rhs = a.rhs; s->out = a.out;
  s->lhs_stride_bytes = lhs_stride_bytes;
  s->rhs_stride_bytes = rhs_stride_bytes;
  s->out_stride0 = a.out_stride0;
  s->tile_bytes = a.K * a.N0 * g;
  s->rows = (int32_t)(a.M * a.M0);
  s->row0 = 0;
  s->N = (int32_t)a.N;
  s->K = (int32_t)a.K;
  s->log2_M0 = lm0;
  s->log2_N0 = ln0;
  s->accumulate = (a.flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) ? 1 : 0;
  return true;
}

template <int KIND, int G, bool NARROW>
hipError_t launch_piece(const SkinnyArgs& all_rows, hipStream_t stream) {
  // Fewer lhs rows leave registers for more of the rhs stream in flight. More
  // than 8 rows: one launch per slab of 8.
  const dim3 grid((unsigned)all_rows.N), block(256);
  SkinnyArgs s = all_rows;
  for (s.row0 = 0; s.row0 < s.rows; s.row0 += 8) {
    const int left = s.rows - s.row0;
    if (left <= 1) hipLaunchKernelGGL((mmt4d_skinny_kernel<KIND, G, 1, 16, NARROW>), grid, block, 0, stream, s);
    else if (left <= 2) hipLaunchKernelGGL((mmt4d_skinny_kernel<KIND, G, 2, 16, NARROW>), grid, block, 0, stream, s);
    else if (left <= 4) hipLaunchKernelGGL((mmt4d_skinny_kernel<KIND, G, 4, 8, NARROW>), grid, block, 0, stream, s);
    else hipLaunchKernelGGL((mmt4d_skinny_kernel<KIND, G, 8, 4, NARROW>), grid, block, 0, stream, s);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <int KIND, bool NARROW>
hipError_t launch_kind(const SkinnyArgs& s, int piece_bytes, hipStream_t stream) {
  if (piece_bytes == 4) return launch_piece<KIND, 4, NARROW>(s, stream);
  if (piece_bytes == 8) return launch_piece<KIND, 8, NARROW>(s, stream);
  if constexpr (KIND == kI8) {
    if (piece_bytes == 1) return launch_piece<KIND, 1, NARROW>(s, stream);
  }
  if constexpr (KIND != kF32) return launch_piece<KIND, 2, NARROW>(s, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_skinny(const Mmt4dArgs& a, hipStream_t stream, const char** name) {
  int kind, piece_bytes;
  bool narrow;
  SkinnyArgs s;
  if (!make_args(a, false, &kind, &piece_bytes, &narrow, &s)) return hipErrorInvalidValue;
  *name = "mmt4d_skinny";
  switch (kind) {
    case kI8: return launch_kind<kI8, false>(s, piece_bytes, stream);
    case kF16:
      return narrow ? launch_kind<kF16, true>(s, piece_bytes, stream) : launch_kind<kF16, false>(s, piece_bytes, stream);
    case kBF16:
      return narrow ? launch_kind<kBF16, true>(s, piece_bytes, stream) : launch_kind<kBF16, false>(s, piece_bytes, stream);
    case kI16: return launch_kind<kI16, false>(s, piece_bytes, stream);
    case kI16U4: return launch_piece<kI16U4, 4, false>(s, stream);
    case kI8I4:
      if (piece_bytes == 1) return launch_piece<kI8I4, 1, false>(s, stream);
      return piece_bytes == 4 ? launch_piece<kI8I4, 4, false>(s, stream) : launch_piece<kI8I4, 8, false>(s, stream);
    case kI16I8: return launch_kind<kI16I8, false>(s, piece_bytes, stream);
    default: return launch_kind<kF32, false>(s, piece_bytes, stream);
  }
}

}  // namespace

// Measured on 1 x 14336 x 4096 problems: with up to 4 lhs rows this kernel is
// at the HBM rate (bf16 1x16x2 18 us, int8 1x16x2 10 us) and level with the
// 64x64 matrix kernel where that applies; with 8 rows it is VALU bound (int8
// 8x16x2 41 us against 23 us, bf16 8x16x2 32 against 23 us).
bool mmt4d_skinny_preferred(const Mmt4dArgs& a) {
  int lhs_bits, rhs_bits, out_bits;
  if (!mmt4d_type_bits(a.flags, &lhs_bits, &rhs_bits, &out_bits)) return false;
  // (8-row tiles of one-byte pieces are 8 bytes per k step, but the matrix kernels load them k-major.)
  const bool k_major_for_mfma = a.K0 * lhs_bits == 8 && a.M0 >= 8;
  return a.M * a.M0 <= 4 || (a.M0 * a.K0 * lhs_bits / 8 < 16 && !k_major_for_mfma);
}

Mmt4dLauncher select_mmt4d_skinny(const Mmt4dArgs& a, bool probe_only) {
  int kind, piece_bytes;
  bool narrow;
  SkinnyArgs s;
  return make_args(a, probe_only, &kind, &piece_bytes, &narrow, &s) ? launch_skinny : nullptr;
}

}  // namespace uk
