// mmt4d for skinny left-hand sides (at most 16 lhs rows in total, e.g. the
// LLM decode shapes M0 in {1, 4, 16} with M = 1): an HBM-bandwidth kernel.
//
// Every rhs element is used exactly once, so the rhs streams from global memory
// straight into MFMA operand registers, no LDS: for N0 = 16 a wavefront's
// 16-row x 64-byte operand (lane l: row l & 15, 16-byte column l >> 4) covers
// whole consecutive k steps of one tile, i.e. each load instruction reads 1 KiB
// of contiguous memory. The (small, L2-resident) lhs is loaded the same way and
// shared by the TN rhs tiles a wavefront works on. The wavefronts of a
// workgroup split K between them and reduce through LDS in a fixed order, so
// results do not depend on scheduling. The matrix pipe is mostly idle here by
// design; it is used because its operand layout matches the tiled rhs exactly
// and it keeps the VALU out of the inner loop.
//
// Covers s8s8s32, f16f16f32 and bf16bf16f32 with N0 = 16 and 16, 32 or 64
// bytes per (k, row) piece, and s8s4s32 (int4 weights) with N0 = 16 and
// K0 = 32 or 64 (mmt4d_gemv_i4_kernel below).
#include "uk_internal.h"

namespace uk {
namespace {

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf16 __attribute__((ext_vector_type(8)));

enum Kind { kI8 = 0, kF16 = 1, kBF16 = 2, kI8I4 = 3 };

struct GemvArgs {
  const uint8_t* lhs;
  const uint8_t* rhs;
  uint8_t* out;
  int64_t lhs_stride_bytes, rhs_stride_bytes;
  int64_t out_stride0;  // elements
  int32_t M, N, K;
  int32_t log2_M0;
  int32_t rb, log2_rb;  // bytes of one (k, row) piece
  int32_t steps;        // MFMA K-steps: ceil(K * rb / 64)
  int32_t accumulate;
};

template <int KIND> struct Acc { typedef v4i32 type; };
template <> struct Acc<kF16> { typedef v4f32 type; };
template <> struct Acc<kBF16> { typedef v4f32 type; };

template <int KIND>
__device__ __forceinline__ typename Acc<KIND>::type mfma16(uint4 row_operand, uint4 col_operand,
                                                           typename Acc<KIND>::type acc) {
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

// TN: rhs tiles per workgroup. UNROLL: K-steps whose loads are in flight together.
template <int KIND, int TN, int UNROLL, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void mmt4d_gemv_kernel(const GemvArgs a) {
  typedef typename Acc<KIND>::type acc_t;
  __shared__ acc_t partial[kWaves][TN][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = lane & 15, g = lane >> 4;
  const int32_t M0 = 1 << a.log2_M0;
  const int32_t lhs_rows = a.M << a.log2_M0;  // <= 16

  // Per-lane byte offset of its 16-byte operand column inside one K-step, as a
  // function of the step: k1 = (64*step + 16*g) >> log2_rb.
  const int32_t ksteps_per_step = 64 >> a.log2_rb;
  const int32_t k1_lane = (16 * g) >> a.log2_rb;
  const int32_t within = (16 * g) & (a.rb - 1);
  const int64_t rhs_kstep = (int64_t)a.rb * 16;
  const int64_t lhs_kstep = (int64_t)a.rb << a.log2_M0;

  const bool lhs_valid = row < lhs_rows;
  const uint8_t* lhs_lane = a.lhs + (int64_t)(row >> a.log2_M0) * a.lhs_stride_bytes +
                            (int64_t)(row & (M0 - 1)) * a.rb + k1_lane * lhs_kstep + within;
  const int64_t tile0 = (int64_t)blockIdx.x * TN;
  const uint8_t* rhs_lane[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int64_t tile = tile0 + t < a.N ? tile0 + t : a.N - 1;  // clamp: computed, not stored
    rhs_lane[t] = a.rhs + tile * a.rhs_stride_bytes + (int64_t)row * a.rb + k1_lane * rhs_kstep + within;
  }

  acc_t acc[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t) acc[t] = acc_t{0, 0, 0, 0};

  // This wavefront's share of the K-steps.
  const int32_t per_wave = (a.steps + kWaves - 1) / kWaves;
  const int32_t s_begin = wave * per_wave;
  const int32_t s_end = min(s_begin + per_wave, a.steps);
  // Steps whose k steps all lie below K need no checks.
  const int32_t full_steps = a.K / ksteps_per_step;

  int32_t s = s_begin;
  for (; s + UNROLL <= min(s_end, full_steps); s += UNROLL) {
    uint4 l[UNROLL], r[UNROLL][TN];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t k1 = (int64_t)(s + u) * ksteps_per_step;
      l[u] = make_uint4(0, 0, 0, 0);
      if (lhs_valid) l[u] = *(const uint4*)(lhs_lane + k1 * lhs_kstep);
#pragma unroll
      for (int t = 0; t < TN; ++t) r[u][t] = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4i32*)(rhs_lane[t] + k1 * rhs_kstep)));
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < TN; ++t) acc[t] = mfma16<KIND>(r[u][t], l[u], acc[t]);
  }
  for (; s < s_end; ++s) {
    const int64_t k1 = (int64_t)s * ksteps_per_step;
    const bool in_k = k1 + k1_lane < a.K;
    uint4 l = make_uint4(0, 0, 0, 0);
    if (lhs_valid && in_k) l = *(const uint4*)(lhs_lane + k1 * lhs_kstep);
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      uint4 r = make_uint4(0, 0, 0, 0);
      if (in_k) r = *(const uint4*)(rhs_lane[t] + k1 * rhs_kstep);
      acc[t] = mfma16<KIND>(r, l, acc[t]);
    }
  }

#pragma unroll
  for (int t = 0; t < TN; ++t) partial[wave][t][lane] = acc[t];
  __syncthreads();
  if (wave != 0) return;
  // Lane l holds lhs row l & 15 and rhs rows 4*(l >> 4) + {0..3} of each tile:
  // four consecutive j0 of output row i0.
  if (!lhs_valid) return;
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    if (tile0 + t >= a.N) continue;
    acc_t v = partial[0][t][lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) v += partial[w][t][lane];
    acc_t* dst = (acc_t*)(a.out + 4 * ((int64_t)(row >> a.log2_M0) * a.out_stride0 +
                                       (tile0 + t) * ((int64_t)M0 * 16) +
                                       (int64_t)(row & (M0 - 1)) * 16 + 4 * g));
    if (a.accumulate) v += *dst;
    *dst = v;
  }
}

// The same product for more than 4 lhs rows, where the lhs operand of a K-step
// is as large as a rhs tile's (1 KiB) and the kernel above pulls all of it
// through L2 again for every rhs tile. Here one workgroup per compute unit
// stays for the whole launch: its wavefronts split K, wavefront w copies the lhs
// operands of its K share into a private slice of LDS once, and then streams
// the rhs tiles of the unit's range past them, the loads of the next tile in
// flight while the current one is multiplied. No barrier before the final sum.
// The rhs is dealt out in HALF tiles (rhs rows 0-7 or 8-15 of a tile: 128
// contiguous bytes of every k step for 16-byte row pieces) so that every unit
// gets the same number of bytes also when tiles / units is not whole (896 tiles
// on 256 units: 3.5); a half tile is a tile with half the lanes' loads masked,
// its missing rows multiply as zeros and are not stored. Partial sums meet in
// LDS in wavefront order: results do not depend on scheduling.
// Needs steps == kWaves * UNROLL (one batch of loads per wavefront and tile).
template <int KIND, int kWaves, int UNROLL, int MAX_TILES>
// (The register budget is said explicitly: two buffers of UNROLL loads and MAX_TILES accumulators; left to its
// own devices with 8 wavefronts the compiler takes all 256 registers for the shorter instantiation and still spills.)
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(UNROLL >= 16 ? 2 : 3, UNROLL >= 16 ? 2 : 3)))
void mmt4d_gemv_resident_lhs_kernel(const GemvArgs a) {
  typedef typename Acc<KIND>::type acc_t;
  extern __shared__ uint4 gemv_lds[];  // [kWaves][UNROLL][64] lhs operands; then [MAX_TILES][kWaves][64] partial sums
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row = lane & 15, g = lane >> 4;
  const int32_t M0 = 1 << a.log2_M0;
  const int32_t lhs_rows = a.M << a.log2_M0;  // <= 16

  // This unit's range of half tiles.
  const int64_t halves = 2 * (int64_t)a.N;
  const int64_t h0 = (int64_t)blockIdx.x * halves / gridDim.x, h1 = ((int64_t)blockIdx.x + 1) * halves / gridDim.x;
  if (h1 <= h0) return;
  const int64_t t0 = h0 >> 1, t1 = (h1 - 1) >> 1;
  const int tiles = (int)(t1 - t0 + 1);  // <= MAX_TILES (checked on the host)
  const bool skip_low_half_of_first = h0 & 1, skip_high_half_of_last = h1 & 1;
  // When every unit gets whole tiles and equally many, it takes one of every round of gridDim.x tiles instead of
  // its range: ranges of 4 tiles of 128 KiB put the units' streams 512 KiB apart, a power of two that the memory
  // channels do not like (16 x 16384 x 4096 bf16: 5.59 -> 5.80 TB/s; with half tiles in play the ranges are the
  // faster deal, 5.83 against 5.67 at 14336).
  const bool rounds = a.N % gridDim.x == 0;
  auto tile_of = [&](int u) -> int64_t { return rounds ? blockIdx.x + (int64_t)gridDim.x * u : t0 + u; };

  const int32_t ksteps_per_step = 64 >> a.log2_rb;
  const int32_t k1_lane = (16 * g) >> a.log2_rb;
  const int32_t within = (16 * g) & (a.rb - 1);
  const int64_t rhs_kstep = (int64_t)a.rb * 16;
  const int64_t lhs_kstep = (int64_t)a.rb << a.log2_M0;
  const bool lhs_valid = row < lhs_rows;
  const int64_t k1_first = (int64_t)(wave * UNROLL) * ksteps_per_step;  // this wavefront's share of K
  const uint8_t* lhs_lane = a.lhs + (int64_t)(row >> a.log2_M0) * a.lhs_stride_bytes +
                            (int64_t)(row & (M0 - 1)) * a.rb + (k1_lane + k1_first) * lhs_kstep + within;
  const uint8_t* rhs_lane = a.rhs + (int64_t)row * a.rb + (k1_lane + k1_first) * rhs_kstep + within;
  const int64_t rhs_step_bytes = ksteps_per_step * rhs_kstep, lhs_step_bytes = ksteps_per_step * lhs_kstep;

  auto tile_rows_loaded = [&](int u) -> bool {
    if (u == 0 && skip_low_half_of_first && row < 8) return false;
    if (u == tiles - 1 && skip_high_half_of_last && row >= 8) return false;
    return true;
  };
  // (Lanes whose rows of a half tile belong to another unit load nothing and keep what they held: rhs row n only
  // ever reaches column n of the result, and those columns are not stored.)
  uint4 r[2][UNROLL];
#pragma unroll
  for (int s = 0; s < UNROLL; ++s) r[0][s] = r[1][s] = make_uint4(0, 0, 0, 0);
  auto fetch = [&](int u, uint4* dst) {
    const uint8_t* p = rhs_lane + tile_of(u) * a.rhs_stride_bytes;
    const bool loaded = tile_rows_loaded(u);
#pragma unroll
    for (int s = 0; s < UNROLL; ++s)
      if (loaded) dst[s] = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4i32*)(p + s * rhs_step_bytes)));
  };
  fetch(0, r[0]);
  uint4* own_lhs = gemv_lds + (wave * UNROLL) * 64 + lane;
  {
    uint4 l[UNROLL];
#pragma unroll
    for (int s = 0; s < UNROLL; ++s) {
      l[s] = make_uint4(0, 0, 0, 0);
      if (lhs_valid) l[s] = *(const uint4*)(lhs_lane + s * lhs_step_bytes);
    }
#pragma unroll
    for (int s = 0; s < UNROLL; ++s) own_lhs[s * 64] = l[s];
  }

  acc_t acc[MAX_TILES];
#pragma unroll
  for (int u = 0; u < MAX_TILES; ++u) acc[u] = acc_t{0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < MAX_TILES; ++u) {
    if (u < tiles) {
      if (u + 1 < tiles) fetch(u + 1, r[(u + 1) & 1]);
#pragma unroll
      for (int s = 0; s < UNROLL; ++s) acc[u] = mfma16<KIND>(r[u & 1][s], own_lhs[s * 64], acc[u]);
    }
  }

  __syncthreads();  // the lhs slices are no longer read: their memory takes the partial sums
  acc_t* partial = (acc_t*)gemv_lds;
#pragma unroll
  for (int u = 0; u < MAX_TILES; ++u)
    if (u < tiles) partial[(u * kWaves + wave) * 64 + lane] = acc[u];
  __syncthreads();
  // Lane l holds lhs row l & 15 and rhs rows 4*(l >> 4) + {0..3} of each tile: four consecutive j0 of output row i0.
  for (int u = wave; u < tiles; u += kWaves) {
    if (!lhs_valid) continue;
    if (u == 0 && skip_low_half_of_first && g < 2) continue;
    if (u == tiles - 1 && skip_high_half_of_last && g >= 2) continue;
    acc_t v = partial[(u * kWaves) * 64 + lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) v += partial[(u * kWaves + w) * 64 + lane];
    acc_t* dst = (acc_t*)(a.out + 4 * ((int64_t)(row >> a.log2_M0) * a.out_stride0 + tile_of(u) * ((int64_t)M0 * 16) +
                                       (int64_t)(row & (M0 - 1)) * 16 + 4 * g));
    if (a.accumulate) v += *dst;
    *dst = v;
  }
}

// int8 values equal to 16x the signed nibbles of 8 bytes, in element order
// (element 2b in the low nibble of byte b, mmt4d_tile_generic.c:35-45): even
// and odd elements are isolated in the high nibbles of two dwords whose bytes
// are then interleaved. Products with these are 16x too large and exact.
__device__ __forceinline__ uint4 widen_i4_times16(uint32_t lo, uint32_t hi) {
  const uint32_t even0 = (lo << 4) & 0xF0F0F0F0u, odd0 = lo & 0xF0F0F0F0u;
  const uint32_t even1 = (hi << 4) & 0xF0F0F0F0u, odd1 = hi & 0xF0F0F0F0u;
  uint4 r;
  r.x = __builtin_amdgcn_perm(odd0, even0, 0x05010400u);
  r.y = __builtin_amdgcn_perm(odd0, even0, 0x07030602u);
  r.z = __builtin_amdgcn_perm(odd1, even1, 0x05010400u);
  r.w = __builtin_amdgcn_perm(odd1, even1, 0x07030602u);
  return r;
}

// The same without the interleaving: the even elements of each dword, then the
// odd ones (6 instructions instead of 10). For products with an lhs operand whose
// bytes are in the same order (lhs_bytes_even_then_odd).
__device__ __forceinline__ uint4 widen_i4_times16_even_then_odd(uint32_t lo, uint32_t hi) {
  return make_uint4((lo << 4) & 0xF0F0F0F0u, lo & 0xF0F0F0F0u, (hi << 4) & 0xF0F0F0F0u, hi & 0xF0F0F0F0u);
}
__device__ __forceinline__ uint4 lhs_bytes_even_then_odd(uint4 v) {
  return make_uint4(__builtin_amdgcn_perm(v.y, v.x, 0x06040200u), __builtin_amdgcn_perm(v.y, v.x, 0x07050301u),
                    __builtin_amdgcn_perm(v.w, v.z, 0x06040200u), __builtin_amdgcn_perm(v.w, v.z, 0x07050301u));
}

// s8s4s32 for a skinny lhs: the int4 rhs streams at half a byte per weight.
// One step covers 128 values of K. Lane l (row l & 15, g = l >> 4) loads the 16
// bytes = 32 nibbles of its rhs row at K values 32*g .. 32*g + 31 of the step
// (for K0 = 32 that is row l & 15 of k step g: the wavefront reads 1 KiB of
// contiguous rhs per load instruction), widens them to two int8 operands, and
// multiplies each with the matching 16 bytes of the lhs (the MFMA sums over K in
// whatever order the two operands agree on). Accumulators carry 16x the result
// until the end; K * K0 < 131072 keeps that inside int32.
// TN rhs tiles per workgroup share each lhs operand: with 16 lhs rows the lhs
// is twice the bytes of one rhs tile per step (int8 against int4), all of it
// through L2 for every workgroup.
template <int TN, int UNROLL, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void mmt4d_gemv_i4_kernel(const GemvArgs a) {
  __shared__ v4i32 partial[kWaves][TN][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = lane & 15, g = lane >> 4;
  const int32_t M0 = 1 << a.log2_M0;
  const int32_t lhs_rows = a.M << a.log2_M0;  // <= 16
  // a.rb / a.log2_rb describe the lhs row piece (K0 bytes); the rhs piece is half of it.
  const int32_t rhs_rb = a.rb >> 1, log2_rhs_rb = a.log2_rb - 1;
  const int64_t lhs_kstep = (int64_t)a.rb << a.log2_M0;
  const bool lhs_valid = row < lhs_rows;
  const uint8_t* lhs_lane = a.lhs + (int64_t)(row >> a.log2_M0) * a.lhs_stride_bytes +
                            (int64_t)(row & (M0 - 1)) * a.rb + ((32 * g) >> a.log2_rb) * lhs_kstep +
                            ((32 * g) & (a.rb - 1));
  const int64_t lhs_step_bytes = (int64_t)128 << a.log2_M0;
  const int64_t tile0 = (int64_t)blockIdx.x * TN;
  const uint8_t* rhs_lane[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int64_t tile = tile0 + t < a.N ? tile0 + t : a.N - 1;  // clamp: computed, not stored
    rhs_lane[t] = a.rhs + tile * a.rhs_stride_bytes + (int64_t)row * rhs_rb +
                  ((16 * g) >> log2_rhs_rb) * ((int64_t)rhs_rb * 16) + ((16 * g) & (rhs_rb - 1));
  }

  const int32_t per_wave = (a.steps + kWaves - 1) / kWaves;
  const int32_t s_begin = wave * per_wave;
  const int32_t s_end = min(s_begin + per_wave, a.steps);

  v4i32 acc[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t) acc[t] = v4i32{0, 0, 0, 0};
  auto multiply = [&](int t, uint4 r, uint4 l0, uint4 l1) {
    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i32, widen_i4_times16(r.x, r.y)),
                                                   __builtin_bit_cast(v4i32, l0), acc[t], 0, 0, 0);
    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i32, widen_i4_times16(r.z, r.w)),
                                                   __builtin_bit_cast(v4i32, l1), acc[t], 0, 0, 0);
  };
  int32_t s = s_begin;
  // (Lanes of lhs rows that do not exist never load: their operands stay zero, set once.)
  uint4 l0[UNROLL], l1[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) l0[u] = l1[u] = make_uint4(0, 0, 0, 0);
  for (; s + UNROLL <= s_end; s += UNROLL) {
    uint4 r[UNROLL][TN];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
      for (int t = 0; t < TN; ++t)
        r[u][t] = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4i32*)(rhs_lane[t] + (int64_t)(s + u) * 1024)));
      if (lhs_valid) {
        l0[u] = *(const uint4*)(lhs_lane + (s + u) * lhs_step_bytes);
        l1[u] = *(const uint4*)(lhs_lane + (s + u) * lhs_step_bytes + 16);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < TN; ++t) multiply(t, r[u][t], l0[u], l1[u]);
  }
  for (; s < s_end; ++s) {
    uint4 l0 = make_uint4(0, 0, 0, 0), l1 = l0;
    if (lhs_valid) {
      l0 = *(const uint4*)(lhs_lane + s * lhs_step_bytes);
      l1 = *(const uint4*)(lhs_lane + s * lhs_step_bytes + 16);
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) multiply(t, *(const uint4*)(rhs_lane[t] + (int64_t)s * 1024), l0, l1);
  }

#pragma unroll
  for (int t = 0; t < TN; ++t) partial[wave][t][lane] = acc[t];
  __syncthreads();
  if (wave != 0 || !lhs_valid) return;
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    if (tile0 + t >= a.N) continue;
    v4i32 v = partial[0][t][lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) v += partial[w][t][lane];
    v = v4i32{v.x >> 4, v.y >> 4, v.z >> 4, v.w >> 4};
    v4i32* dst = (v4i32*)(a.out + 4 * ((int64_t)(row >> a.log2_M0) * a.out_stride0 + (tile0 + t) * ((int64_t)M0 * 16) +
                                       (int64_t)(row & (M0 - 1)) * 16 + 4 * g));
    if (a.accumulate) v += *dst;
    *dst = v;
  }
}

// The resident-lhs form of the int4 kernel (see mmt4d_gemv_resident_lhs_kernel): with 16 lhs rows the int8 lhs
// operands of a step are twice the bytes of a rhs tile's nibbles, all of it through L2 again for every tile. One
// workgroup per compute unit, wavefront w keeps the lhs operands of its K share (two 16-byte pieces per lane
// and step) in LDS and streams the unit's half tiles past them. Needs steps == kWaves * UNROLL.
template <int kWaves, int UNROLL, int MAX_TILES>
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(4, 4)))  // (128 registers, as with 16 wavefronts)
void mmt4d_gemv_i4_resident_lhs_kernel(const GemvArgs a) {
  extern __shared__ uint4 gemv_lds[];  // [kWaves][UNROLL][2][64] lhs operands; then [MAX_TILES][kWaves][64] partial sums
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row = lane & 15, g = lane >> 4;
  const int32_t M0 = 1 << a.log2_M0;
  const int32_t lhs_rows = a.M << a.log2_M0;  // <= 16
  const int32_t rhs_rb = a.rb >> 1, log2_rhs_rb = a.log2_rb - 1;
  const int64_t lhs_kstep = (int64_t)a.rb << a.log2_M0;
  const int64_t lhs_step_bytes = (int64_t)128 << a.log2_M0;

  const int64_t halves = 2 * (int64_t)a.N;
  const int64_t h0 = (int64_t)blockIdx.x * halves / gridDim.x, h1 = ((int64_t)blockIdx.x + 1) * halves / gridDim.x;
  if (h1 <= h0) return;
  const int64_t t0 = h0 >> 1, t1 = (h1 - 1) >> 1;
  const int tiles = (int)(t1 - t0 + 1);  // <= MAX_TILES (checked on the host)
  const bool skip_low_half_of_first = h0 & 1, skip_high_half_of_last = h1 & 1;

  const bool lhs_valid = row < lhs_rows;
  const int32_t first_step = wave * UNROLL;  // this wavefront's share of K
  const uint8_t* lhs_lane = a.lhs + (int64_t)(row >> a.log2_M0) * a.lhs_stride_bytes +
                            (int64_t)(row & (M0 - 1)) * a.rb + ((32 * g) >> a.log2_rb) * lhs_kstep +
                            ((32 * g) & (a.rb - 1)) + first_step * lhs_step_bytes;
  const uint8_t* rhs_lane = a.rhs + t0 * a.rhs_stride_bytes + (int64_t)row * rhs_rb +
                            ((16 * g) >> log2_rhs_rb) * ((int64_t)rhs_rb * 16) + ((16 * g) & (rhs_rb - 1)) +
                            (int64_t)first_step * 1024;

  auto tile_rows_loaded = [&](int u) -> bool {
    if (u == 0 && skip_low_half_of_first && row < 8) return false;
    if (u == tiles - 1 && skip_high_half_of_last && row >= 8) return false;
    return true;
  };
  // Loads of up to DEPTH - 1 tiles in flight ahead of the one being multiplied (8 KiB per wavefront and tile).
  constexpr int DEPTH = 4;
  // (Lanes whose rows of a half tile belong to another unit load nothing and keep what they held, see above.)
  uint4 r[DEPTH][UNROLL];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
#pragma unroll
    for (int s = 0; s < UNROLL; ++s) r[d][s] = make_uint4(0, 0, 0, 0);
  auto fetch = [&](int u, uint4* dst) {
    const uint8_t* p = rhs_lane + (int64_t)u * a.rhs_stride_bytes;
    const bool loaded = tile_rows_loaded(u);
#pragma unroll
    for (int s = 0; s < UNROLL; ++s)
      if (loaded) dst[s] = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4i32*)(p + (int64_t)s * 1024)));
  };
#pragma unroll
  for (int u = 0; u < DEPTH - 1; ++u)
    if (u < tiles) fetch(u, r[u]);
  uint4* own_lhs = gemv_lds + (wave * UNROLL) * 128 + lane;
  {
    uint4 l0[UNROLL], l1[UNROLL];
#pragma unroll
    for (int s = 0; s < UNROLL; ++s) {
      l0[s] = l1[s] = make_uint4(0, 0, 0, 0);
      if (lhs_valid) {
        l0[s] = *(const uint4*)(lhs_lane + s * lhs_step_bytes);
        l1[s] = *(const uint4*)(lhs_lane + s * lhs_step_bytes + 16);
      }
    }
#pragma unroll
    for (int s = 0; s < UNROLL; ++s) {
      // (bytes reordered once, here, so that the nibbles need no interleaving in the loop)
      own_lhs[s * 128] = lhs_bytes_even_then_odd(l0[s]);
      own_lhs[s * 128 + 64] = lhs_bytes_even_then_odd(l1[s]);
    }
  }

  v4i32 acc[MAX_TILES];
#pragma unroll
  for (int u = 0; u < MAX_TILES; ++u) acc[u] = v4i32{0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < MAX_TILES; ++u) {
    if (u < tiles) {
      if (u + DEPTH - 1 < tiles) fetch(u + DEPTH - 1, r[(u + DEPTH - 1) % DEPTH]);
#pragma unroll
      for (int s = 0; s < UNROLL; ++s) {
        const uint4 w = r[u % DEPTH][s];
        acc[u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i32, widen_i4_times16_even_then_odd(w.x, w.y)),
                                                       __builtin_bit_cast(v4i32, own_lhs[s * 128]), acc[u], 0, 0, 0);
        acc[u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i32, widen_i4_times16_even_then_odd(w.z, w.w)),
                                                       __builtin_bit_cast(v4i32, own_lhs[s * 128 + 64]), acc[u], 0, 0, 0);
      }
    }
  }

  __syncthreads();  // the lhs slices are no longer read: their memory takes the partial sums
  v4i32* partial = (v4i32*)gemv_lds;
#pragma unroll
  for (int u = 0; u < MAX_TILES; ++u)
    if (u < tiles) partial[(u * kWaves + wave) * 64 + lane] = acc[u];
  __syncthreads();
  for (int u = wave; u < tiles; u += kWaves) {
    if (!lhs_valid) continue;
    if (u == 0 && skip_low_half_of_first && g < 2) continue;
    if (u == tiles - 1 && skip_high_half_of_last && g >= 2) continue;
    v4i32 v = partial[(u * kWaves) * 64 + lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) v += partial[(u * kWaves + w) * 64 + lane];
    v = v4i32{v.x >> 4, v.y >> 4, v.z >> 4, v.w >> 4};
    v4i32* dst = (v4i32*)(a.out + 4 * ((int64_t)(row >> a.log2_M0) * a.out_stride0 + (t0 + u) * ((int64_t)M0 * 16) +
                                       (int64_t)(row & (M0 - 1)) * 16 + 4 * g));
    if (a.accumulate) v += *dst;
    *dst = v;
  }
}

int log2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int l = 0;
  while ((1ll << l) < v) ++l;
  return l;
}

bool make_args(const Mmt4dArgs& a, bool probe_only, int* kind, GemvArgs* g) {
  int elem_bytes;
  bool i4 = false;
  switch (a.flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: *kind = kI8; elem_bytes = 1; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: *kind = kI8I4; elem_bytes = 1; i4 = true; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: *kind = kF16; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *kind = kBF16; elem_bytes = 2; break;
    default: return false;
  }
  const int lm0 = log2_exact(a.M0);
  const int rb = a.K0 * elem_bytes;
  if (lm0 < 0 || a.M0 > 16 || a.N0 != 16) return false;
  if (rb != 16 && rb != 32 && rb != 64) return false;
  if (i4 && rb == 16) return false;  // 8-byte rhs row pieces: two rows per 16-byte load
  if (probe_only) return a.M0 < 16;  // 16-row tiles only when the whole lhs is that skinny
  if (a.M * a.M0 > 16 || a.K == 0) return false;
  // Worth it only when the rhs is long enough to stream.
  if (a.N < 16) return false;
  const int64_t lhs_stride_bytes = a.lhs_stride0 * elem_bytes;
  const int64_t rhs_stride_bytes = i4 ? a.rhs_stride0 / 2 : a.rhs_stride0 * elem_bytes;
  // int4: whole steps of 128 K values only, and the 16x-scaled sums must fit int32.
  if (i4 && (((int64_t)a.K * a.K0) % 128 != 0 || (int64_t)a.K * a.K0 >= 131072)) return false;
  if ((uintptr_t)a.lhs % 16 || (a.M > 1 && lhs_stride_bytes % 16)) return false;
  if ((uintptr_t)a.rhs % 16 || rhs_stride_bytes % 16) return false;
  if ((uintptr_t)a.out % 16 || (a.M > 1 && a.out_stride0 % 4)) return false;
  g->lhs = a.lhs; g->rhs = a.rhs; g->out = a.out;
  g->lhs_stride_bytes = lhs_stride_bytes;
  g->rhs_stride_bytes = rhs_stride_bytes;
  g->out_stride0 = a.out_stride0;
  g->M = (int32_t)a.M; g->N = (int32_t)a.N; g->K = (int32_t)a.K;
  g->log2_M0 = lm0;
  g->rb = rb;
  g->log2_rb = log2_exact(rb);
  g->steps = i4 ? (int32_t)((int64_t)a.K * a.K0 / 128) : (int32_t)(((int64_t)a.K * rb + 63) / 64);
  g->accumulate = (a.flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) ? 1 : 0;
  return true;
}

// Compute units of the current device (one persistent workgroup each).
int compute_units() {
  static int cached[64] = {0};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
  if (cached[device] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    cached[device] = n;
  }
  return cached[device];
}

// The resident-lhs kernel, if it fits: more than 4 lhs rows, K in whole 64-byte
// steps whose number is what one of the instantiations splits over its
// wavefronts, at least a tile per compute unit and at most MAX_TILES of them.
template <int KIND>
bool launch_resident_lhs(const GemvArgs& g, hipStream_t stream, hipError_t* status) {
  constexpr int MAX_TILES = 8;
  // (With 1 or 4 lhs rows the kernel above is the faster one: 6.14 against 6.0 TB/s at 896 tiles.)
  if ((g.M << g.log2_M0) <= 4) return false;
  if (((int64_t)g.K * g.rb) % 64 != 0) return false;
  const int units = compute_units();
  if (units <= 0 || g.N < units) return false;
  // (most tiles any unit gets: ceil(2N / units) half tiles can touch that many / 2 + 1 tiles)
  if ((2 * (int64_t)g.N + units - 1) / units / 2 + 1 > MAX_TILES) return false;
  auto launch = [&](auto kernel, int waves, int unroll) {
    const int lds_bytes = waves * (unroll > MAX_TILES ? unroll : MAX_TILES) * 1024;
    *status = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (*status != hipSuccess) return;
    // Nearly all units with whole tiles each beat all units with half tiles at the ends of their ranges (1000
    // tiles: 250 units x 4 tiles 6.06 TB/s, 256 units 5.85); seven eighths of the units do not (896 tiles on 224: 5.80
    // against 5.88).
    int used = units;
    for (int u = units; u >= units - units / 16; --u)
      if (g.N % u == 0) { used = u; break; }
    hipLaunchKernelGGL(kernel, dim3(used), dim3(64 * waves), lds_bytes, stream, g);
    *status = hipGetLastError();
  };
  // (8 wavefronts with 16 loads each in flight twice over; 16 wavefronts x 8 measured no better than the kernel above.)
  switch (g.steps) {
    case 128: launch(mmt4d_gemv_resident_lhs_kernel<KIND, 8, 16, MAX_TILES>, 8, 16); return true;
    case 64: launch(mmt4d_gemv_resident_lhs_kernel<KIND, 8, 8, MAX_TILES>, 8, 8); return true;
    default: return false;
  }
}

template <int KIND>
hipError_t launch_kind(const GemvArgs& g, hipStream_t stream, const char** name) {
  hipError_t status;
  if (launch_resident_lhs<KIND>(g, stream, &status)) {
    *name = "mmt4d_gemv_resident_lhs";
    return status;
  }
  // One rhs tile per workgroup (most workgroups, best balance over the CUs),
  // 4 wavefronts splitting K, 16 KiB of rhs in flight per wavefront.
  constexpr int TN = 1, UNROLL = 16, WAVES = 4;
  hipLaunchKernelGGL((mmt4d_gemv_kernel<KIND, TN, UNROLL, WAVES>), dim3((g.N + TN - 1) / TN),
                     dim3(64 * WAVES), 0, stream, g);
  return hipGetLastError();
}

hipError_t launch_gemv(const Mmt4dArgs& a, hipStream_t stream, const char** name) {
  int kind;
  GemvArgs g;
  if (!make_args(a, false, &kind, &g)) return hipErrorInvalidValue;
  *name = "mmt4d_gemv";
  if (kind == kI8I4) {
    // More than 4 lhs rows and a tile or more per compute unit, or six tiles or more per unit with any number of
    // rows (28672 x 8192, one row: 0.69 -> 0.71 of the HBM peak; at 3.5 tiles per unit the kernel below is ahead,
    // 0.51 against 0.48): the resident-lhs kernel, where its instantiations fit the number of steps (each of 128
    // values of K; the lhs of 64 steps fills 128 KiB of LDS).
    const int units = compute_units();
    constexpr int MAX_TILES = 8;
    if (((g.M << g.log2_M0) > 4 || g.N >= 6 * (int64_t)units) && units > 0 && g.N >= units && (2 * (int64_t)g.N + units - 1) / units / 2 + 1 <= MAX_TILES &&
        (g.steps == 64 || g.steps == 32)) {
      const int lds_bytes = 128 * 1024;  // the lhs operands of 64 steps; the partial sums need less
      // (16 wavefronts x 4 steps with three tiles' loads in flight: 0.65 of the HBM peak at 16 x 28672 x 8192 against
      // 0.62 for the kernel below; 8 wavefronts x 8 steps 0.63, deeper prefetch slower.)
      void (*kernel)(const GemvArgs) = g.steps == 64 ? mmt4d_gemv_i4_resident_lhs_kernel<16, 4, MAX_TILES>
                                                     : mmt4d_gemv_i4_resident_lhs_kernel<8, 4, MAX_TILES>;
      const hipError_t attr = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (attr != hipSuccess) return attr;
      *name = "mmt4d_gemv_resident_lhs";
      hipLaunchKernelGGL(kernel, dim3(units), dim3(g.steps == 64 ? 1024 : 512), lds_bytes, stream, g);
      return hipGetLastError();
    }
    // More than 4 lhs rows: two rhs tiles per workgroup (measured on 16 rows x
    // 65536 x 8192: 4.5 TB/s with one, 5.9 with two, 4.9 with four).
    if ((g.M << g.log2_M0) > 4) {
      hipLaunchKernelGGL((mmt4d_gemv_i4_kernel<2, 8, 4>), dim3((g.N + 1) / 2), dim3(256), 0, stream, g);
    } else {
      hipLaunchKernelGGL((mmt4d_gemv_i4_kernel<1, 8, 4>), dim3(g.N), dim3(256), 0, stream, g);
    }
    return hipGetLastError();
  }
  if (kind == kI8) return launch_kind<kI8>(g, stream, name);
  if (kind == kF16) return launch_kind<kF16>(g, stream, name);
  return launch_kind<kBF16>(g, stream, name);
}

}  // namespace

Mmt4dLauncher select_mmt4d_gemv(const Mmt4dArgs& a, bool probe_only) {
  int kind;
  GemvArgs g;
  return make_args(a, probe_only, &kind, &g) ? launch_gemv : nullptr;
}

}  // namespace uk
