// Host side of the MFMA mmt4d kernels: which problems they cover, and the
// dispatch to the per-type translation units (mmt4d_mfma_kernels.h describes
// the kernels).
#include "mmt4d_mfma_kernels.h"

namespace uk {
namespace {

int log2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int l = 0;
  while ((1ll << l) < v) ++l;
  return l;
}

struct Plan {
  int kind;
  bool rhs_i4;
  bool narrow;  // 16-bit output, rounded once at the end
  int gather;   // 16 or 4
  MfmaArgs args;
};

// Fills `plan` if the problem is covered. With `probe_only` only type and tile
// shape are looked at.
bool make_plan(const Mmt4dArgs& a, bool probe_only, Plan* plan) {
  int kind, elem_bytes;
  bool i4 = false, narrow = false;
  // With a 16-bit output the reference rounds the accumulator after every
  // multiply-add unless told to skip that (mmt4d_tile_generic.c:229-286,
  // 319-376): only the skipping variant (f32 accumulator, one rounding at the
  // end) is something a matrix pipe can compute.
  const bool skip_roundings = a.flags & IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS;
  switch (a.flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: kind = kI8; elem_bytes = 1; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: kind = kI8; elem_bytes = 1; i4 = true; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: kind = kF16; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: kind = kBF16; elem_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: kind = kF32; elem_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16:
      if (!skip_roundings) return false;
      kind = kF16; elem_bytes = 2; narrow = true;
      break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16:
      if (!skip_roundings) return false;
      kind = kBF16; elem_bytes = 2; narrow = true;
      break;
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
  } else if (lhs_rb == 1 && kind == kI8) {
    // int8 K0 = 1 (the Arm baseline tiles Mx8x1): k-major operands, transposed
    // on the way out of LDS; tiles of 8 or 16 rows, direct-to-LDS kernel only.
    if (lm0 < 3 || ln0 < 3) return false;
    gather = 1;
  } else if (lhs_rb == 4 || lhs_rb == 2 || lhs_rb == 8) {
    // 2 and 8 (e.g. the x86-64 int8 16x16x2 and f16 16x16x1 tiles, the Arm int8
    // 8x8x8 tiles) run on the direct-to-LDS kernel only: see below.
    gather = lhs_rb;
  } else {
    return false;
  }
  plan->kind = kind;
  plan->rhs_i4 = i4;
  plan->narrow = narrow;
  plan->gather = gather;
  if (probe_only) return true;

  // Alignment of every vector access the kernel makes.
  const int lhs_align = gather == 4 ? 4 : 16;  // (also for 1-, 2- and 8-byte pieces: 16 bytes per lane)
  const int rhs_align = i4 ? 8 : lhs_align;
  const int64_t lhs_stride_bytes = a.lhs_stride0 * elem_bytes;
  const int64_t rhs_stride_bytes = i4 ? a.rhs_stride0 / 2 : a.rhs_stride0 * elem_bytes;
  if (((uintptr_t)a.lhs % lhs_align) || (a.M > 1 && lhs_stride_bytes % lhs_align)) return false;
  if (((uintptr_t)a.rhs % rhs_align) || (a.N > 1 && rhs_stride_bytes % rhs_align)) return false;
  // (four consecutive outputs per store: 16 bytes, 8 with a 16-bit output)
  if (((uintptr_t)a.out % (narrow ? 8 : 16)) || (a.M > 1 && a.out_stride0 % 4)) return false;
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
  if ((gather == 1 || gather == 2 || gather == 8) && !mfma_direct_covers(m, gather, i4)) return false;
  return true;
}

hipError_t launch_mfma(const Mmt4dArgs& a, hipStream_t stream, const char** name) {
  Plan plan;
  if (!make_plan(a, false, &plan)) return hipErrorInvalidValue;
  const MfmaArgs& m = plan.args;
  switch (plan.kind) {
    case kI8: return launch_mfma_i8(m, plan.gather, plan.rhs_i4, stream, name);
    case kF16: return launch_mfma_f16(m, plan.gather, plan.narrow, stream, name);
    case kBF16: return launch_mfma_bf16(m, plan.gather, plan.narrow, stream, name);
    default: return launch_mfma_f32(m, plan.gather, stream, name);
  }
}

}  // namespace

Mmt4dLauncher select_mmt4d_mfma(const Mmt4dArgs& a, bool probe_only) {
  Plan plan;
  return make_plan(a, probe_only, &plan) ? launch_mfma : nullptr;
}

}  // namespace uk
