/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the reference microkernels' results, used only as
 * the checker in tests, in the smoke check and as the "port" CPU baseline of
 * the benchmark. Nothing in the library under iree_amd/ may call into it.
 *
 * What each function follows in the reference
 * (paths relative to runtime/src/iree/builtins/ukernel/):
 *   oracle_mmt4d      mmt4d.c:55-141 (operand addressing, early exits) and
 *                     mmt4d_tile_generic.c:11-376 (per-type arithmetic)
 *   oracle_pack       tools/pack_test.c:13-71 (index map), pack.c:106-109
 *   oracle_unpack     tools/unpack_test.c:13-58 (index map), unpack.c:84-86
 *   oracle_f16_to_f32 / oracle_bf16_to_f32 / oracle_f32_to_f16 /
 *   oracle_f32_to_bf16   common.h:665-792
 *
 * Pinning status: every function here is checked (tests/test_oracle_*.py)
 * against the compiled reference over the reference's own test grid, against
 * the literal tensors of tests/e2e/tensor_ops/{pack,unpack}.mlir, against numpy
 * integer matmul / reshape+transpose identities, and against hand-computed
 * known-answer values for the int4 nibble order and the f16 subnormal flush.
 * No function is "parity unpinned".
 *
 * Build: gcc -O2 -ffp-contract=off -shared -fPIC (see oracle/Makefile). The
 * contraction switch matters only for f32f32f32, where a*b is not exact.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/iree_uk_mi355x.h"

#define ORACLE_EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* 16-bit float formats                                                       */
/* ------------------------------------------------------------------------ */

/* Widening conversion shared by f16 (5 exponent bits) and bf16 (8). Inputs with
 * a zero exponent field (zero and subnormals) give a signed zero; NaNs give the
 * all-ones-mantissa quiet NaN. */
static float widen16(uint16_t h, int ebits) {
  const int mbits = 15 - ebits;
  const uint32_t sign = (uint32_t)(h >> 15) << 31;
  const uint32_t efield = (h >> mbits) & ((1u << ebits) - 1u);
  const uint32_t mfield = h & ((1u << mbits) - 1u);
  uint32_t bits;
  if (efield == (1u << ebits) - 1u) {
    bits = sign | 0x7F800000u | (mfield ? 0x007FFFFFu : 0u);
  } else if (efield == 0) {
    bits = sign;
  } else {
    const uint32_t e32 = efield + 127u - ((1u << (ebits - 1)) - 1u);
    bits = sign | (e32 << 23) | (mfield << (23 - mbits));
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* Narrowing conversion, round to nearest even on the mantissa. Quirks kept on
 * purpose because the reference has them: f32 subnormal inputs and results
 * below the 16-bit format's exponent range become zero, but an unbiased
 * exponent of exactly -(2^(ebits-1)) is still encoded through the normal path,
 * which yields exponent field 0 with the rounded mantissa bits. */
static uint16_t narrow16(float f, int ebits) {
  const int mbits = 15 - ebits;
  const int half = 1 << (ebits - 1);
  uint32_t bits;
  memcpy(&bits, &f, 4);
  const uint32_t sign = (bits >> 31) << 15;
  const uint32_t e32 = (bits >> 23) & 0xFFu;
  const uint32_t m32 = bits & 0x007FFFFFu;
  const uint32_t emask16 = ((1u << ebits) - 1u) << mbits;
  const uint32_t mmask16 = (1u << mbits) - 1u;
  if (e32 == 0xFFu) return (uint16_t)(sign | emask16 | (m32 ? mmask16 : 0u));
  if (e32 == 0) return (uint16_t)sign;
  int e = (int)e32 - 128; /* the reference's "arithmetic exponent" */
  if (e >= half) return (uint16_t)(sign | emask16);
  if (e < -half) return (uint16_t)sign;
  const uint32_t even_bit = 1u << (23 - mbits);
  const uint32_t odd_bit = even_bit >> 1;
  uint32_t m = m32 + ((m32 & even_bit) ? odd_bit : odd_bit - 1u);
  if (m > 0x007FFFFFu) {
    m = 0;
    ++e;
  }
  const uint32_t efield = (uint32_t)(e + half) << mbits;
  return (uint16_t)(sign | efield | (m >> (23 - mbits)));
}

ORACLE_EXPORT float oracle_f16_to_f32(uint16_t h) { return widen16(h, 5); }
ORACLE_EXPORT float oracle_bf16_to_f32(uint16_t h) { return widen16(h, 8); }
ORACLE_EXPORT uint16_t oracle_f32_to_f16(float f) { return narrow16(f, 5); }
ORACLE_EXPORT uint16_t oracle_f32_to_bf16(float f) { return narrow16(f, 8); }

/* ------------------------------------------------------------------------ */
/* mmt4d                                                                      */
/* ------------------------------------------------------------------------ */

/* Bit widths of (lhs, rhs, out) elements for a type flag, 0 if unknown. */
static int mmt4d_bits(uint32_t type, int* lhs, int* rhs, int* out) {
  switch (type) {
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: *lhs = 32; *rhs = 32; *out = 32; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: *lhs = 8; *rhs = 8; *out = 32; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: *lhs = 16; *rhs = 16; *out = 32; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16: *lhs = 16; *rhs = 16; *out = 16; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *lhs = 16; *rhs = 16; *out = 32; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: *lhs = 16; *rhs = 16; *out = 16; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S16S32: *lhs = 16; *rhs = 16; *out = 32; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S16U4S32: *lhs = 16; *rhs = 4; *out = 32; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S8S32: *lhs = 16; *rhs = 8; *out = 32; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: *lhs = 8; *rhs = 4; *out = 32; return 1;
    default: return 0;
  }
}

/* One output element: the sum over k (outer) and k0 (inner), in that order, of
 * lhs[k][i0][k0] * rhs[k][j0][k0], added to `*out` when accumulating.
 * `lrow` / `rrow` point at element (k=0, i0, k0=0) resp. (k=0, j0, k0=0);
 * consecutive k are `lstep` / `rstep` BYTES apart. */
static void dot_element(uint32_t type, int accumulate, int skip_round,
                        const uint8_t* lrow, int64_t lstep, const uint8_t* rrow,
                        int64_t rstep, int64_t K, int K0, void* out) {
  switch (type) {
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: {
      int32_t acc = accumulate ? *(int32_t*)out : 0;
      for (int64_t k = 0; k < K; ++k) {
        const int8_t* l = (const int8_t*)(lrow + k * lstep);
        const int8_t* r = (const int8_t*)(rrow + k * rstep);
        for (int k0 = 0; k0 < K0; ++k0) acc += (int32_t)l[k0] * (int32_t)r[k0];
      }
      *(int32_t*)out = acc;
      return;
    }
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: {
      /* Byte b of a row holds element 2b in its low nibble and 2b+1 in its
       * high nibble, both two's-complement 4-bit. */
      int32_t acc = accumulate ? *(int32_t*)out : 0;
      for (int64_t k = 0; k < K; ++k) {
        const int8_t* l = (const int8_t*)(lrow + k * lstep);
        const uint8_t* r = rrow + k * rstep;
        for (int k0 = 0; k0 < K0; ++k0) {
          const int nib = (k0 & 1) ? (r[k0 >> 1] >> 4) : (r[k0 >> 1] & 0xF);
          const int32_t rv = (nib ^ 8) - 8;
          acc += (int32_t)l[k0] * rv;
        }
      }
      *(int32_t*)out = acc;
      return;
    }
    case IREE_UK_FLAG_MMT4D_TYPE_S16S16S32: {
      int32_t acc = accumulate ? *(int32_t*)out : 0;
      for (int64_t k = 0; k < K; ++k) {
        const int16_t* l = (const int16_t*)(lrow + k * lstep);
        const int16_t* r = (const int16_t*)(rrow + k * rstep);
        for (int k0 = 0; k0 < K0; ++k0)
          acc = (int32_t)((uint32_t)acc + (uint32_t)((int32_t)l[k0] * (int32_t)r[k0]));
      }
      *(int32_t*)out = acc;
      return;
    }
    case IREE_UK_FLAG_MMT4D_TYPE_S16S8S32: {
      int32_t acc = accumulate ? *(int32_t*)out : 0;
      for (int64_t k = 0; k < K; ++k) {
        const int16_t* l = (const int16_t*)(lrow + k * lstep);
        const int8_t* r = (const int8_t*)(rrow + k * rstep);
        for (int k0 = 0; k0 < K0; ++k0)
          acc = (int32_t)((uint32_t)acc + (uint32_t)((int32_t)l[k0] * (int32_t)r[k0]));
      }
      *(int32_t*)out = acc;
      return;
    }
    case IREE_UK_FLAG_MMT4D_TYPE_S16U4S32: {
      /* Same nibble order as s8s4s32 but the nibbles are unsigned. */
      int32_t acc = accumulate ? *(int32_t*)out : 0;
      for (int64_t k = 0; k < K; ++k) {
        const int16_t* l = (const int16_t*)(lrow + k * lstep);
        const uint8_t* r = rrow + k * rstep;
        for (int k0 = 0; k0 < K0; ++k0) {
          const int32_t rv = (k0 & 1) ? (r[k0 >> 1] >> 4) : (r[k0 >> 1] & 0xF);
          acc = (int32_t)((uint32_t)acc + (uint32_t)((int32_t)l[k0] * rv));
        }
      }
      *(int32_t*)out = acc;
      return;
    }
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: {
      float acc = accumulate ? *(float*)out : 0.f;
      for (int64_t k = 0; k < K; ++k) {
        const float* l = (const float*)(lrow + k * lstep);
        const float* r = (const float*)(rrow + k * rstep);
        for (int k0 = 0; k0 < K0; ++k0) acc += l[k0] * r[k0];
      }
      *(float*)out = acc;
      return;
    }
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32:
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: {
      const int eb = type == IREE_UK_FLAG_MMT4D_TYPE_F16F16F32 ? 5 : 8;
      float acc = accumulate ? *(float*)out : 0.f;
      for (int64_t k = 0; k < K; ++k) {
        const uint16_t* l = (const uint16_t*)(lrow + k * lstep);
        const uint16_t* r = (const uint16_t*)(rrow + k * rstep);
        for (int k0 = 0; k0 < K0; ++k0) acc += widen16(l[k0], eb) * widen16(r[k0], eb);
      }
      *(float*)out = acc;
      return;
    }
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16:
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: {
      const int eb = type == IREE_UK_FLAG_MMT4D_TYPE_F16F16F16 ? 5 : 8;
      uint16_t* o = (uint16_t*)out;
      if (skip_round) {
        /* f32 accumulator, one rounding at the end. */
        float acc = accumulate ? widen16(*o, eb) : 0.f;
        for (int64_t k = 0; k < K; ++k) {
          const uint16_t* l = (const uint16_t*)(lrow + k * lstep);
          const uint16_t* r = (const uint16_t*)(rrow + k * rstep);
          for (int k0 = 0; k0 < K0; ++k0) acc += widen16(l[k0], eb) * widen16(r[k0], eb);
        }
        *o = narrow16(acc, eb);
      } else {
        /* 16-bit accumulator, rounded after every multiply-add. */
        uint16_t acc = accumulate ? *o : 0;
        for (int64_t k = 0; k < K; ++k) {
          const uint16_t* l = (const uint16_t*)(lrow + k * lstep);
          const uint16_t* r = (const uint16_t*)(rrow + k * rstep);
          for (int k0 = 0; k0 < K0; ++k0)
            acc = narrow16(widen16(acc, eb) + widen16(l[k0], eb) * widen16(r[k0], eb), eb);
        }
        *o = acc;
      }
      return;
    }
    default:
      return;
  }
}

/* Rows [m_begin, m_end) of tiles. */
static void mmt4d_rows(const iree_uk_mmt4d_params_t* p, int64_t m_begin, int64_t m_end) {
  const uint32_t type = p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK;
  int lb, rb, ob;
  if (!mmt4d_bits(type, &lb, &rb, &ob)) return;
  const int accumulate = (p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  const int skip_round = (p->flags & IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) != 0;
  if (p->M == 0 || p->N == 0 || (p->K == 0 && accumulate)) return;
  const int64_t M0 = p->M0, N0 = p->N0, K0 = p->K0;
  const uint8_t* lhs = (const uint8_t*)p->lhs_buffer + p->lhs_offset * lb / 8;
  const uint8_t* rhs = (const uint8_t*)p->rhs_buffer + p->rhs_offset * rb / 8;
  uint8_t* out = (uint8_t*)p->out_buffer + p->out_offset * ob / 8;
  const int64_t lstep = M0 * K0 * lb / 8, rstep = N0 * K0 * rb / 8;
  for (int64_t i = m_begin; i < m_end; ++i) {
    const uint8_t* lpanel = lhs + i * p->lhs_stride0 * lb / 8;
    for (int64_t j = 0; j < p->N; ++j) {
      const uint8_t* rpanel = rhs + j * p->rhs_stride0 * rb / 8;
      uint8_t* otile = out + (i * p->out_stride0 + j * M0 * N0) * ob / 8;
      for (int64_t i0 = 0; i0 < M0; ++i0) {
        for (int64_t j0 = 0; j0 < N0; ++j0) {
          dot_element(type, accumulate, skip_round, lpanel + i0 * K0 * lb / 8, lstep,
                      rpanel + j0 * K0 * rb / 8, rstep, p->K, (int)K0,
                      otile + (i0 * N0 + j0) * ob / 8);
        }
      }
    }
  }
}

ORACLE_EXPORT void oracle_mmt4d(const iree_uk_mmt4d_params_t* p) { mmt4d_rows(p, 0, p->M); }

typedef struct {
  const iree_uk_mmt4d_params_t* p;
  int64_t begin, end;
} mmt4d_job_t;

static void* mmt4d_worker(void* arg) {
  mmt4d_job_t* job = (mmt4d_job_t*)arg;
  mmt4d_rows(job->p, job->begin, job->end);
  return NULL;
}

/* Same result as oracle_mmt4d; rows of tiles are split over `threads`. */
ORACLE_EXPORT void oracle_mmt4d_mt(const iree_uk_mmt4d_params_t* p, int threads) {
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  pthread_t tid[256];
  mmt4d_job_t job[256];
  for (int t = 0; t < threads; ++t) {
    job[t].p = p;
    job[t].begin = p->M * t / threads;
    job[t].end = p->M * (t + 1) / threads;
    pthread_create(&tid[t], NULL, mmt4d_worker, &job[t]);
  }
  for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
}

/* ------------------------------------------------------------------------ */
/* pack / unpack                                                              */
/* ------------------------------------------------------------------------ */

static int pack_elem_bytes(uint32_t type) {
  switch (type) {
    case IREE_UK_FLAG_PACK_TYPE_F32F32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_I8I8: return 1;
    case IREE_UK_FLAG_PACK_TYPE_I32I32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_F16F16: return 2;
    case IREE_UK_FLAG_PACK_TYPE_BF16BF16: return 2;
    default: return 0;
  }
}

/* The tiled side of pack/unpack as seen from the 2-D side: tile counts and tile
 * sizes along 2-D dimensions 0 and 1, and the element strides of the four
 * loops (tile index 0, tile index 1, within-tile 0, within-tile 1). */
typedef struct {
  int64_t outer0, outer1, tile0, tile1;
  int64_t s_outer0, s_outer1, s_tile0, s_tile1;
} tiled_view_t;

static tiled_view_t tiled_view(int64_t size0, int64_t size1, int64_t size2, int64_t size3,
                               int64_t stride0, int transpose_inner, int transpose_outer) {
  tiled_view_t v;
  v.outer0 = size0; v.outer1 = size1; v.tile0 = size2; v.tile1 = size3;
  v.s_outer0 = stride0; v.s_outer1 = size2 * size3; v.s_tile0 = size3; v.s_tile1 = 1;
  int64_t t;
  if (transpose_outer) {
    t = v.outer0; v.outer0 = v.outer1; v.outer1 = t;
    t = v.s_outer0; v.s_outer0 = v.s_outer1; v.s_outer1 = t;
  }
  if (transpose_inner) {
    t = v.tile0; v.tile0 = v.tile1; v.tile1 = t;
    t = v.s_tile0; v.s_tile0 = v.s_tile1; v.s_tile1 = t;
  }
  return v;
}

ORACLE_EXPORT void oracle_pack(const iree_uk_pack_params_t* p) {
  const int e = pack_elem_bytes(p->flags & IREE_UK_FLAG_PACK_TYPE_MASK);
  if (!e) return;
  if (p->out_size0 == 0 || p->out_size1 == 0 || p->out_size2 == 0 || p->out_size3 == 0) return;
  const tiled_view_t v = tiled_view(p->out_size0, p->out_size1, p->out_size2, p->out_size3,
                                    p->out_stride0,
                                    (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER) != 0,
                                    (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER) != 0);
  const uint8_t* in = (const uint8_t*)p->in_buffer + p->in_offset * e;
  uint8_t* out = (uint8_t*)p->out_buffer + p->out_offset * e;
  uint8_t pad[8];
  memcpy(pad, &p->padding_value, 8); /* little endian: low bytes first */
  for (int64_t o0 = 0; o0 < v.outer0; ++o0)
    for (int64_t o1 = 0; o1 < v.outer1; ++o1)
      for (int64_t t0 = 0; t0 < v.tile0; ++t0)
        for (int64_t t1 = 0; t1 < v.tile1; ++t1) {
          const int64_t i0 = o0 * v.tile0 + t0, i1 = o1 * v.tile1 + t1;
          uint8_t* dst =
              out + (o0 * v.s_outer0 + o1 * v.s_outer1 + t0 * v.s_tile0 + t1 * v.s_tile1) * e;
          if (i0 < p->in_size0 && i1 < p->in_size1)
            memcpy(dst, in + (i0 * p->in_stride0 + i1 * p->in_stride1) * e, e);
          else
            memcpy(dst, pad, e);
        }
}

static int unpack_elem_bytes(uint32_t type) {
  switch (type) {
    case IREE_UK_FLAG_UNPACK_TYPE_F32F32: return 4;
    case IREE_UK_FLAG_UNPACK_TYPE_I32I32: return 4;
    case IREE_UK_FLAG_UNPACK_TYPE_F16F16: return 2;
    case IREE_UK_FLAG_UNPACK_TYPE_BF16BF16: return 2;
    default: return 0;
  }
}

ORACLE_EXPORT void oracle_unpack(const iree_uk_unpack_params_t* p) {
  const int e = unpack_elem_bytes(p->flags & IREE_UK_FLAG_UNPACK_TYPE_MASK);
  if (!e) return;
  if (p->out_size0 == 0 || p->out_size1 == 0) return;
  const tiled_view_t v = tiled_view(p->in_size0, p->in_size1, p->in_size2, p->in_size3,
                                    p->in_stride0,
                                    (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER) != 0,
                                    (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER) != 0);
  const uint8_t* in = (const uint8_t*)p->in_buffer + p->in_offset * e;
  uint8_t* out = (uint8_t*)p->out_buffer + p->out_offset * e;
  for (int64_t i0 = 0; i0 < p->out_size0; ++i0) {
    const int64_t o0 = i0 / v.tile0, t0 = i0 % v.tile0;
    for (int64_t i1 = 0; i1 < p->out_size1; ++i1) {
      const int64_t o1 = i1 / v.tile1, t1 = i1 % v.tile1;
      memcpy(out + (i0 * p->out_stride0 + i1 * p->out_stride1) * e,
             in + (o0 * v.s_outer0 + o1 * v.s_outer1 + t0 * v.s_tile0 + t1 * v.s_tile1) * e, e);
    }
  }
}
