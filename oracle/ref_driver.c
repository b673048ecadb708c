/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Glue linked into oracle/_ref/libiree_uk_ref.so next to objects compiled from
 * the reference's own ukernel sources (see oracle/Makefile). It supplies what
 * the reference leaves to its embedder and adds threaded drivers so the
 * reference ukernels can be timed on all host cores:
 *   - iree_uk_assert_fail (declared extern at common.h:307-309),
 *   - ref_host_cpu_data: the x86-64 feature words the reference's tile
 *     selection reads (bit positions from schemas/cpu_feature_bits.inl:85-117),
 *   - ref_*_mt: static split of the outer M (rows of tiles) dimension (of N
 *     for matrix-vector shapes) over pthreads, each thread calling the
 *     reference entry point on its slice,
 *     which is the decomposition the reference's CPU backend applies when it
 *     distributes a dispatch over workgroups.
 * Parameter structs are declared from this repository's header; the layouts are
 * identical to the reference's by construction of the drop-in ABI.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../include/iree_uk_mi355x.h"

#define REF_EXPORT __attribute__((visibility("default")))

static int g_fail_count = 0;
static int g_abort_on_fail = 1;

void iree_uk_assert_fail(const char* file, int line, const char* function, const char* condition) {
  fprintf(stderr, "%s:%d: %s: reference ukernel assertion failed: %s\n", file, line, function,
          condition);
  fflush(stderr);
  __atomic_add_fetch(&g_fail_count, 1, __ATOMIC_RELAXED);
  if (g_abort_on_fail) abort();
}

REF_EXPORT void ref_mmt4d(const iree_uk_mmt4d_params_t* p) { iree_uk_mmt4d_p(p); }
REF_EXPORT uint32_t ref_mmt4d_info(const iree_uk_mmt4d_params_t* p) {
  return iree_uk_mmt4d_info_p(p);
}
REF_EXPORT void ref_pack(const iree_uk_pack_params_t* p) { iree_uk_pack_p(p); }
REF_EXPORT void ref_unpack(const iree_uk_unpack_params_t* p) { iree_uk_unpack_p(p); }
REF_EXPORT void ref_query_tile_sizes_2d(const iree_uk_query_tile_sizes_2d_params_t* p,
                                        iree_uk_query_tile_sizes_2d_out_params_t* o) {
  iree_uk_query_tile_sizes_2d(p, o);
}

/* Fills the 8 feature words for the CPU this runs on. */
REF_EXPORT void ref_host_cpu_data(uint64_t out[8]) {
  memset(out, 0, 8 * sizeof(uint64_t));
#if defined(__x86_64__)
  __builtin_cpu_init();
  uint64_t w = 0;
#define FEATURE(name, bit) \
  if (__builtin_cpu_supports(name)) w |= 1ull << (bit)
  FEATURE("sse3", 0);
  FEATURE("ssse3", 1);
  FEATURE("sse4.1", 2);
  FEATURE("sse4.2", 3);
  FEATURE("avx", 10);
  FEATURE("fma", 11);
  FEATURE("f16c", 14);
  FEATURE("avx2", 15);
  FEATURE("avx512f", 20);
  FEATURE("avx512cd", 21);
  FEATURE("avx512vl", 22);
  FEATURE("avx512dq", 23);
  FEATURE("avx512bw", 24);
  FEATURE("avx512vnni", 28);
  FEATURE("avx512bf16", 31);
#undef FEATURE
  out[0] = w;
#endif
}

typedef struct {
  int kind; /* 0 mmt4d, 1 pack, 2 unpack */
  iree_uk_mmt4d_params_t mm;
  iree_uk_pack_params_t pk;
  iree_uk_unpack_params_t up;
} job_t;

static void* worker(void* arg) {
  job_t* j = (job_t*)arg;
  if (j->kind == 0) iree_uk_mmt4d_p(&j->mm);
  if (j->kind == 1) iree_uk_pack_p(&j->pk);
  if (j->kind == 2) iree_uk_unpack_p(&j->up);
  return NULL;
}

static void run_jobs(job_t* jobs, int n) {
  pthread_t tid[256];
  for (int t = 0; t < n; ++t) pthread_create(&tid[t], NULL, worker, &jobs[t]);
  for (int t = 0; t < n; ++t) pthread_join(tid[t], NULL);
}

static int clamp_threads(int threads) { return threads < 1 ? 1 : (threads > 256 ? 256 : threads); }

/* mmt4d with rows of tiles [M*t/T, M*(t+1)/T) on thread t; with fewer rows of
 * tiles than threads (matrix-vector shapes) the rhs panels are split instead. */
REF_EXPORT void ref_mmt4d_mt(const iree_uk_mmt4d_params_t* p, int threads) {
  threads = clamp_threads(threads);
  job_t* jobs = (job_t*)calloc(threads, sizeof(job_t));
  const int split_n = p->M < threads && p->N > p->M;
  for (int t = 0; t < threads; ++t) {
    jobs[t].kind = 0;
    jobs[t].mm = *p;
    if (split_n) {
      const int64_t b = p->N * t / threads, e = p->N * (t + 1) / threads;
      jobs[t].mm.N = e - b;
      jobs[t].mm.rhs_offset = p->rhs_offset + b * p->rhs_stride0;
      jobs[t].mm.out_offset = p->out_offset + b * p->M0 * p->N0;
    } else {
      const int64_t b = p->M * t / threads, e = p->M * (t + 1) / threads;
      jobs[t].mm.M = e - b;
      jobs[t].mm.lhs_offset = p->lhs_offset + b * p->lhs_stride0;
      jobs[t].mm.out_offset = p->out_offset + b * p->out_stride0;
    }
  }
  run_jobs(jobs, threads);
  free(jobs);
}

/* pack without TRANSPOSE_OUTER, split over rows of output tiles. */
REF_EXPORT int ref_pack_mt(const iree_uk_pack_params_t* p, int threads) {
  if (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER) return -1;
  threads = clamp_threads(threads);
  const int64_t tile0 =
      (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER) ? p->out_size3 : p->out_size2;
  job_t* jobs = (job_t*)calloc(threads, sizeof(job_t));
  for (int t = 0; t < threads; ++t) {
    const int64_t b = p->out_size0 * t / threads, e = p->out_size0 * (t + 1) / threads;
    int64_t rows = p->in_size0 - b * tile0;
    if (rows < 0) rows = 0;
    if (rows > (e - b) * tile0) rows = (e - b) * tile0;
    jobs[t].kind = 1;
    jobs[t].pk = *p;
    jobs[t].pk.out_size0 = e - b;
    jobs[t].pk.in_size0 = rows;
    jobs[t].pk.in_offset = p->in_offset + b * tile0 * p->in_stride0;
    jobs[t].pk.out_offset = p->out_offset + b * p->out_stride0;
  }
  run_jobs(jobs, threads);
  free(jobs);
  return 0;
}

/* unpack without TRANSPOSE_OUTER, split over rows of input tiles. */
REF_EXPORT int ref_unpack_mt(const iree_uk_unpack_params_t* p, int threads) {
  if (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER) return -1;
  threads = clamp_threads(threads);
  const int64_t tile0 =
      (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER) ? p->in_size3 : p->in_size2;
  job_t* jobs = (job_t*)calloc(threads, sizeof(job_t));
  for (int t = 0; t < threads; ++t) {
    const int64_t b = p->in_size0 * t / threads, e = p->in_size0 * (t + 1) / threads;
    int64_t rows = p->out_size0 - b * tile0;
    if (rows < 0) rows = 0;
    if (rows > (e - b) * tile0) rows = (e - b) * tile0;
    jobs[t].kind = 2;
    jobs[t].up = *p;
    jobs[t].up.in_size0 = e - b;
    jobs[t].up.out_size0 = rows;
    jobs[t].up.in_offset = p->in_offset + b * p->in_stride0;
    jobs[t].up.out_offset = p->out_offset + b * tile0 * p->out_stride0;
  }
  run_jobs(jobs, threads);
  free(jobs);
  return 0;
}

REF_EXPORT int ref_fail_count(void) { return g_fail_count; }
REF_EXPORT void ref_set_abort_on_fail(int v) { g_abort_on_fail = v; }
