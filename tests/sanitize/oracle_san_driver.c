/* Drives oracle/uk_oracle.c under AddressSanitizer + UndefinedBehaviorSanitizer
 * on the CPU. Every operand is an exact-size heap allocation, placed so that
 * `buffer + offset` is its first byte: a read or write one element outside
 * what the reference's addressing (mmt4d.c:70-83, pack_test.c:13-71,
 * unpack_test.c:13-58) touches is reported by the sanitizer and fails the
 * test. Shapes: ragged sizes, strides with gaps, every type flag, both
 * transposes. Prints "oracle sanitizer run ok" at the end. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/iree_uk_mi355x.h"

void oracle_mmt4d(const iree_uk_mmt4d_params_t* p);
void oracle_mmt4d_mt(const iree_uk_mmt4d_params_t* p, int threads);
void oracle_pack(const iree_uk_pack_params_t* p);
void oracle_unpack(const iree_uk_unpack_params_t* p);

static uint64_t rng_state = 0x1234567ull;
static uint32_t rng(void) {
  rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
  return (uint32_t)(rng_state >> 33);
}

static void* filled(size_t bytes) {
  uint8_t* p = (uint8_t*)malloc(bytes ? bytes : 1);
  if (!p) abort();
  for (size_t i = 0; i < bytes; ++i) p[i] = (uint8_t)rng();
  return p;
}

static const struct { uint32_t type; int lhs_bits, rhs_bits, out_bits; } kTypes[] = {
    {IREE_UK_FLAG_MMT4D_TYPE_F32F32F32, 32, 32, 32}, {IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 8, 8, 32},
    {IREE_UK_FLAG_MMT4D_TYPE_F16F16F32, 16, 16, 32}, {IREE_UK_FLAG_MMT4D_TYPE_F16F16F16, 16, 16, 16},
    {IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32, 16, 16, 32}, {IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16, 16, 16, 16},
    {IREE_UK_FLAG_MMT4D_TYPE_S16S16S32, 16, 16, 32}, {IREE_UK_FLAG_MMT4D_TYPE_S16U4S32, 16, 4, 32},
    {IREE_UK_FLAG_MMT4D_TYPE_S16S8S32, 16, 8, 32}, {IREE_UK_FLAG_MMT4D_TYPE_S8S4S32, 8, 4, 32},
};

static void run_mmt4d(void) {
  static const int shapes[][6] = {  /* M, N, K, M0, N0, K0 */
      {1, 1, 1, 1, 1, 2}, {3, 2, 5, 8, 8, 4}, {2, 3, 4, 16, 16, 2}, {1, 4, 3, 1, 16, 8},
      {2, 2, 0, 4, 8, 2}, {5, 1, 2, 3, 5, 6}, {0, 3, 2, 8, 8, 4}, {2, 0, 2, 8, 8, 4}};
  for (size_t t = 0; t < sizeof kTypes / sizeof kTypes[0]; ++t) {
    for (size_t s = 0; s < sizeof shapes / sizeof shapes[0]; ++s) {
      for (int accumulate = 0; accumulate < 2; ++accumulate) {
        for (int gap = 0; gap < 2; ++gap) {
          const int64_t M = shapes[s][0], N = shapes[s][1], K = shapes[s][2];
          const int M0 = shapes[s][3], N0 = shapes[s][4], K0 = shapes[s][5];
          iree_uk_mmt4d_params_t p;
          memset(&p, 0, sizeof p);
          p.M = M; p.N = N; p.K = K; p.M0 = M0; p.N0 = N0; p.K0 = K0;
          p.flags = kTypes[t].type | (accumulate ? IREE_UK_FLAG_MMT4D_ACCUMULATE : 0) |
                    IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION | ((s & 1) ? IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS : 0);
          /* Strides in elements; a gap of 8 elements keeps sub-byte rows on byte boundaries. */
          p.lhs_stride0 = K * M0 * K0 + 8 * gap;
          p.rhs_stride0 = K * N0 * K0 + 8 * gap;
          p.out_stride0 = N * M0 * N0 + 8 * gap;
          const size_t lhs_bytes = M ? (size_t)(((M - 1) * p.lhs_stride0 + K * M0 * K0) * kTypes[t].lhs_bits / 8) : 0;
          const size_t rhs_bytes = N ? (size_t)(((N - 1) * p.rhs_stride0 + K * N0 * K0) * kTypes[t].rhs_bits / 8) : 0;
          const size_t out_bytes = M ? (size_t)(((M - 1) * p.out_stride0 + N * M0 * N0) * kTypes[t].out_bits / 8) : 0;
          /* A non-zero offset with the base moved back by as much: the
           * reference's tests do the same (mmt4d_test.c:395-402). */
          const int64_t off = 16 * (int64_t)(s + 1);
          uint8_t* lhs = (uint8_t*)filled(lhs_bytes);
          uint8_t* rhs = (uint8_t*)filled(rhs_bytes);
          uint8_t* out = (uint8_t*)filled(out_bytes);
          p.lhs_offset = off; p.lhs_buffer = lhs - off * kTypes[t].lhs_bits / 8;
          p.rhs_offset = off; p.rhs_buffer = rhs - off * kTypes[t].rhs_bits / 8;
          p.out_offset = off; p.out_buffer = out - off * kTypes[t].out_bits / 8;
          if (gap) oracle_mmt4d_mt(&p, 3); else oracle_mmt4d(&p);
          free(lhs); free(rhs); free(out);
        }
      }
    }
  }
}

static const struct { uint32_t pack, unpack; int bytes; } kCopyTypes[] = {
    {IREE_UK_FLAG_PACK_TYPE_F32F32, IREE_UK_FLAG_UNPACK_TYPE_F32F32, 4},
    {IREE_UK_FLAG_PACK_TYPE_I8I8, 0, 1},
    {IREE_UK_FLAG_PACK_TYPE_I32I32, IREE_UK_FLAG_UNPACK_TYPE_I32I32, 4},
    {IREE_UK_FLAG_PACK_TYPE_F16F16, IREE_UK_FLAG_UNPACK_TYPE_F16F16, 2},
    {IREE_UK_FLAG_PACK_TYPE_BF16BF16, IREE_UK_FLAG_UNPACK_TYPE_BF16BF16, 2},
};

static void run_pack_unpack(void) {
  static const int shapes[][4] = {  /* rows, cols, tile0, tile1 */
      {1, 1, 1, 1}, {7, 5, 4, 2}, {16, 33, 16, 1}, {9, 9, 8, 8}, {3, 40, 2, 16}, {0, 4, 2, 2}, {5, 0, 2, 2}};
  for (size_t t = 0; t < sizeof kCopyTypes / sizeof kCopyTypes[0]; ++t) {
    for (size_t s = 0; s < sizeof shapes / sizeof shapes[0]; ++s) {
      for (uint32_t transpose = 0; transpose < 4; ++transpose) {
        for (int gap = 0; gap < 2; ++gap) {
          const int64_t rows = shapes[s][0], cols = shapes[s][1];
          const int64_t T0 = shapes[s][2], T1 = shapes[s][3];
          const int e = kCopyTypes[t].bytes;
          const int inner = transpose & 1, outer = (transpose >> 1) & 1;
          const int64_t O0 = (rows + T0 - 1) / T0 + (s == 1), O1 = (cols + T1 - 1) / T1;
          /* Sizes as stored: transposes swap the roles (pack_test.c:13-71). */
          const int64_t size0 = outer ? O1 : O0, size1 = outer ? O0 : O1;
          const int64_t size2 = inner ? T1 : T0, size3 = inner ? T0 : T1;
          const int64_t stride1 = 1 + gap;                    /* 2-D side, elements */
          const int64_t stride0 = cols * stride1 + 3 * gap;
          const int64_t tiled_stride0 = size1 * size2 * size3 + 5 * gap;
          const size_t flat_bytes = rows && cols ? (size_t)(((rows - 1) * stride0 + (cols - 1) * stride1 + 1) * e) : 0;
          const size_t tiled_bytes = size0 && size1 ? (size_t)(((size0 - 1) * tiled_stride0 + size1 * size2 * size3) * e) : 0;
          uint8_t* flat = (uint8_t*)filled(flat_bytes);
          uint8_t* tiled = (uint8_t*)filled(tiled_bytes);
          const int64_t off = 8 * (int64_t)(s + 1);

          iree_uk_pack_params_t p;
          memset(&p, 0, sizeof p);
          p.in_buffer = flat - off * e; p.in_offset = off;
          p.in_stride0 = stride0; p.in_stride1 = stride1;
          p.out_buffer = tiled - off * e; p.out_offset = off;
          p.out_stride0 = tiled_stride0; p.out_stride1 = size2 * size3;
          p.in_size0 = rows; p.in_size1 = cols;
          p.out_size0 = size0; p.out_size1 = size1; p.out_size2 = size2; p.out_size3 = size3;
          p.padding_value = 0xA5A5A5A5A5A5A5A5ull;
          p.flags = kCopyTypes[t].pack | (inner ? IREE_UK_FLAG_PACK_TRANSPOSE_INNER : 0) |
                    (outer ? IREE_UK_FLAG_PACK_TRANSPOSE_OUTER : 0);
          oracle_pack(&p);

          if (kCopyTypes[t].unpack) {
            iree_uk_unpack_params_t u;
            memset(&u, 0, sizeof u);
            u.in_buffer = tiled - off * e; u.in_offset = off;
            u.in_stride0 = tiled_stride0; u.in_stride1 = size2 * size3;
            u.out_buffer = flat - off * e; u.out_offset = off;
            u.out_stride0 = stride0; u.out_stride1 = stride1;
            u.in_size0 = size0; u.in_size1 = size1; u.in_size2 = size2; u.in_size3 = size3;
            u.out_size0 = rows; u.out_size1 = cols;
            u.flags = kCopyTypes[t].unpack | (inner ? IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER : 0) |
                      (outer ? IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER : 0);
            oracle_unpack(&u);
          }
          free(flat); free(tiled);
        }
      }
    }
  }
}

int main(void) {
  run_mmt4d();
  run_pack_unpack();
  puts("oracle sanitizer run ok");
  return 0;
}
