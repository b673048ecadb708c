// Drives the host side of the C ABI (iree_amd/csrc/uk_api.hip: parameter
// checks, early exits, operand region arithmetic, staging decisions) built
// with AddressSanitizer + UndefinedBehaviorSanitizer on the host pass. No
// kernel needs to run: without a GPU every call that gets past the checks
// ends in the failure handler with a HIP error, with one it computes. What the
// sanitizers watch is the arithmetic on the way (sizes near the limits the
// reference's checks admit, mmt4d.c:26-33, pack.c:51-103, unpack.c:31-81).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/iree_uk_mi355x.h"

static int g_failures = 0;
static void on_failure(const char*, int, const char*, const char*) { ++g_failures; }

#define EXPECT(cond)                                                    \
  do {                                                                  \
    if (!(cond)) {                                                      \
      fprintf(stderr, "%s:%d: expectation failed: %s\n", __FILE__, __LINE__, #cond); \
      exit(1);                                                          \
    }                                                                   \
  } while (0)

static iree_uk_mmt4d_params_t mmt4d_base(std::vector<uint8_t>& buf) {
  iree_uk_mmt4d_params_t p;
  memset(&p, 0, sizeof p);
  p.lhs_buffer = p.rhs_buffer = p.out_buffer = buf.data();
  p.M = p.N = p.K = 1;
  p.M0 = p.N0 = 8;
  p.K0 = 4;
  p.lhs_stride0 = p.rhs_stride0 = 32;
  p.out_stride0 = 64;
  p.flags = IREE_UK_FLAG_MMT4D_TYPE_S8S8S32;
  return p;
}

static int failures_of_mmt4d(const iree_uk_mmt4d_params_t& p) {
  const int before = g_failures;
  iree_uk_mmt4d_p(&p);
  iree_uk_mi355x_mmt4d_noalloc_p(&p);
  return g_failures - before;
}

int main() {
  iree_uk_mi355x_set_fail_handler(on_failure);
  std::vector<uint8_t> buf(1 << 16, 1);

  // Rejected by the checks: exactly one report per call, whatever else is in the struct.
  {
    iree_uk_mmt4d_params_t p = mmt4d_base(buf);
    p.flags |= 0x800;
    EXPECT(failures_of_mmt4d(p) == 2);
    p = mmt4d_base(buf); p.M = -1; EXPECT(failures_of_mmt4d(p) == 2);
    p = mmt4d_base(buf); p.K = (int64_t)1 << 31; EXPECT(failures_of_mmt4d(p) == 2);
    p = mmt4d_base(buf); p.K0 = 1 << 15; EXPECT(failures_of_mmt4d(p) == 2);
    p = mmt4d_base(buf); p.M = 2; p.out_stride0 = 1; EXPECT(failures_of_mmt4d(p) == 2);
    EXPECT(g_failures == 10);
    const int before = g_failures;
    iree_uk_mmt4d_p(nullptr);
    iree_uk_pack_p(nullptr);
    iree_uk_unpack_p(nullptr);
    iree_uk_query_tile_sizes_2d(nullptr, nullptr);
    EXPECT(g_failures == before + 4);
  }
  // Early exits never look at the buffers.
  {
    const int before = g_failures;
    iree_uk_mmt4d_params_t p = mmt4d_base(buf);
    p.lhs_buffer = p.rhs_buffer = p.out_buffer = nullptr;
    p.M = 0; iree_uk_mmt4d_p(&p);
    p.M = 1; p.N = 0; iree_uk_mmt4d_p(&p);
    p.N = 1; p.K = 0; p.flags |= IREE_UK_FLAG_MMT4D_ACCUMULATE; iree_uk_mmt4d_p(&p);
    EXPECT(g_failures == before);
  }
  // The largest values the checks admit, every type: the region arithmetic
  // must not overflow (signed overflow is what UBSan reports). Such a call
  // cannot be served; it has to end in one failure report.
  {
    static const uint32_t types[] = {IREE_UK_FLAG_MMT4D_TYPE_F32F32F32, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32,
                                     IREE_UK_FLAG_MMT4D_TYPE_F16F16F16, IREE_UK_FLAG_MMT4D_TYPE_S16U4S32,
                                     IREE_UK_FLAG_MMT4D_TYPE_S8S4S32};
    for (uint32_t type : types) {
      iree_uk_mmt4d_params_t p = mmt4d_base(buf);
      p.flags = type;
      p.M = p.N = p.K = ((int64_t)1 << 31) - 1;
      p.M0 = p.N0 = (1 << 15) - 1;
      p.K0 = (1 << 15) - 2;
      p.lhs_stride0 = p.rhs_stride0 = p.out_stride0 = INT64_MAX - 7;
      p.lhs_offset = p.rhs_offset = p.out_offset = INT64_MAX - 7;
      EXPECT(failures_of_mmt4d(p) == 2);
      EXPECT(iree_uk_mmt4d_info_p(&p) == 0);
    }
    iree_uk_pack_params_t k;
    memset(&k, 0, sizeof k);
    k.in_buffer = k.out_buffer = buf.data();
    k.flags = IREE_UK_FLAG_PACK_TYPE_F32F32 | IREE_UK_FLAG_PACK_TRANSPOSE_INNER | IREE_UK_FLAG_PACK_TRANSPOSE_OUTER;
    k.in_size0 = k.in_size1 = INT64_MAX;
    k.in_stride0 = k.in_stride1 = INT64_MAX;
    k.out_size0 = k.out_size1 = k.out_size2 = k.out_size3 = INT64_MAX;
    k.out_stride0 = INT64_MAX;
    k.out_stride1 = 1;  // == out_size2 * out_size3 only if that product wrapped
    k.in_offset = k.out_offset = INT64_MAX;
    int before = g_failures;
    iree_uk_pack_p(&k);
    EXPECT(g_failures == before + 1);
    k.out_size2 = k.out_size3 = (int64_t)1 << 31;
    k.out_stride1 = (int64_t)1 << 62;
    before = g_failures;
    iree_uk_pack_p(&k);
    EXPECT(g_failures == before + 1);

    iree_uk_unpack_params_t u;
    memset(&u, 0, sizeof u);
    u.in_buffer = u.out_buffer = buf.data();
    u.flags = IREE_UK_FLAG_UNPACK_TYPE_I32I32 | IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER;
    u.in_size0 = u.in_size1 = INT64_MAX;
    u.in_size2 = u.in_size3 = (int64_t)1 << 31;
    u.in_stride0 = INT64_MAX;
    u.in_stride1 = (int64_t)1 << 62;
    u.out_size0 = u.out_size1 = INT64_MAX;
    u.out_stride0 = u.out_stride1 = INT64_MAX;
    u.in_offset = u.out_offset = INT64_MAX;
    before = g_failures;
    iree_uk_unpack_p(&u);
    EXPECT(g_failures == before + 1);
  }
  // Ordinary calls on host memory, exact-size allocations: on a machine with a
  // GPU they compute (and ASan watches the row copies); without one each ends
  // in one failure report from the HIP runtime.
  {
    const int M = 3, N = 2, K = 5, M0 = 8, N0 = 8, K0 = 4, gap = 16;
    std::vector<int8_t> lhs((M - 1) * (K * M0 * K0 + gap) + K * M0 * K0, 1);
    std::vector<int8_t> rhs((N - 1) * (K * N0 * K0 + gap) + K * N0 * K0, 2);
    std::vector<int32_t> out((M - 1) * (N * M0 * N0 + gap) + N * M0 * N0, 3);
    iree_uk_mmt4d_params_t p;
    memset(&p, 0, sizeof p);
    p.lhs_buffer = lhs.data(); p.rhs_buffer = rhs.data(); p.out_buffer = out.data();
    p.lhs_stride0 = K * M0 * K0 + gap; p.rhs_stride0 = K * N0 * K0 + gap; p.out_stride0 = N * M0 * N0 + gap;
    p.M = M; p.N = N; p.K = K; p.M0 = M0; p.N0 = N0; p.K0 = K0;
    p.flags = IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 | IREE_UK_FLAG_MMT4D_ACCUMULATE;
    int before = g_failures;
    iree_uk_mmt4d_p(&p);
    const bool have_gpu = g_failures == before;
    if (have_gpu) {
      EXPECT(out[0] == 3 + 2 * K * K0);
      EXPECT(out[N * M0 * N0] == 3);  // the gap between output rows is not written
      iree_uk_mi355x_mmt4d_noalloc_p(&p);
      EXPECT(out[0] == 3 + 4 * K * K0);
    } else {
      EXPECT(g_failures == before + 1);
    }
    // Broadcast lhs (stride 0) and overlapping rhs rows are accepted.
    p.lhs_stride0 = 0;
    p.rhs_stride0 = N0 * K0;
    before = g_failures;
    iree_uk_mmt4d_p(&p);
    EXPECT(g_failures == before + (have_gpu ? 0 : 1));

    const int rows = 7, cols = 5;
    std::vector<float> flat(rows * cols, 1.f), tiled(2 * 3 * 4 * 2, 0.f);
    iree_uk_pack_params_t k;
    memset(&k, 0, sizeof k);
    k.in_buffer = flat.data(); k.out_buffer = tiled.data();
    k.in_stride0 = cols; k.in_stride1 = 1;
    k.in_size0 = rows; k.in_size1 = cols;
    k.out_size0 = 2; k.out_size1 = 3; k.out_size2 = 4; k.out_size3 = 2;
    k.out_stride0 = 24; k.out_stride1 = 8;
    k.flags = IREE_UK_FLAG_PACK_TYPE_F32F32;
    before = g_failures;
    iree_uk_pack_p(&k);
    EXPECT(g_failures == before + (have_gpu ? 0 : 1));
    iree_uk_unpack_params_t u;
    memset(&u, 0, sizeof u);
    u.in_buffer = tiled.data(); u.out_buffer = flat.data();
    u.in_stride0 = 24; u.in_stride1 = 8;
    u.in_size0 = 2; u.in_size1 = 3; u.in_size2 = 4; u.in_size3 = 2;
    u.out_size0 = rows; u.out_size1 = cols;
    u.out_stride0 = cols; u.out_stride1 = 1;
    u.flags = IREE_UK_FLAG_UNPACK_TYPE_F32F32;
    before = g_failures;
    iree_uk_unpack_p(&u);
    EXPECT(g_failures == before + (have_gpu ? 0 : 1));
    if (have_gpu) EXPECT(flat[rows * cols - 1] == 1.f && tiled[7 * 2] == 1.f);
  }
  puts("shim sanitizer run ok");
  return 0;
}
