// Host side of the C ABI: parameter checks, operand address resolution, host /
// device pointer classification with staging, kernel selection and launch.
//
// The checks restate the reference's debug-build assertions
// (mmt4d.c:12-48, pack.c:51-103, unpack.c:31-81) and are always on here: a
// rejected call costs microseconds next to a kernel launch, and an out-of-range
// parameter reaching a GPU kernel can fault the device rather than one process.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "uk_internal.h"

#define UK_API extern "C" __attribute__((visibility("default")))

// Default failure handler; an embedder's strong definition replaces it.
extern "C" __attribute__((visibility("default"), weak)) void iree_uk_assert_fail(
    const char* file, int line, const char* function, const char* condition) {
  fflush(stdout);
  fprintf(stderr, "%s:%d: %s: iree_uk_mi355x check failed: %s\n", file, line, function, condition);
  fflush(stderr);
  abort();
}

namespace uk {
hipError_t launch_pack_generic(const PackArgs& a, hipStream_t stream, const char** name);
hipError_t launch_unpack_generic(const UnpackArgs& a, hipStream_t stream, const char** name);
}  // namespace uk

namespace {

thread_local hipStream_t tl_stream = nullptr;
thread_local bool tl_async = false;
thread_local const char* tl_last_kernel = "";
std::atomic<iree_uk_mi355x_fail_handler_t> g_fail_handler{nullptr};

void report_failure(const char* file, int line, const char* function, const char* condition) {
  iree_uk_mi355x_fail_handler_t h = g_fail_handler.load(std::memory_order_acquire);
  if (h) {
    h(file, line, function, condition);
  } else {
    iree_uk_assert_fail(file, line, function, condition);
  }
}

// Checks a parameter condition; on failure reports it and leaves the entry
// point (which returns void) without launching anything.
#define UK_REQUIRE(cond)                                      \
  do {                                                        \
    if (!(cond)) {                                            \
      report_failure(__FILE__, __LINE__, __func__, #cond);    \
      return;                                                 \
    }                                                         \
  } while (0)

// Checks a HIP call inside a function returning bool (true = ok).
#define UK_HIP_OK(expr)                                                       \
  do {                                                                        \
    hipError_t uk_err_ = (expr);                                              \
    if (uk_err_ != hipSuccess) {                                              \
      char uk_msg_[256];                                                      \
      snprintf(uk_msg_, sizeof uk_msg_, "%s -> %s", #expr, hipGetErrorString(uk_err_)); \
      report_failure(__FILE__, __LINE__, __func__, uk_msg_);                  \
      return false;                                                           \
    }                                                                         \
  } while (0)

// outer * tile >= size for non-negative values, without forming a product
// that may not fit.
bool tiles_cover(int64_t outer, int64_t tile, int64_t size) {
  if (size == 0) return true;
  if (outer == 0 || tile == 0) return false;
  return outer >= size / tile + (size % tile != 0);
}

bool in_unsigned_range(int64_t v, int bits) { return v >= 0 && v < ((int64_t)1 << bits); }

// True if a kernel on the current device may dereference `p`.
bool device_accessible(const void* p) {
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, p);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // plain host memory is reported as an error
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged ||
         attr.type == hipMemoryTypeHost;
}

// Per-thread device staging buffers for host operands (grow-only, released
// when the thread exits).
struct StageBuffer {
  void* ptr = nullptr;
  size_t capacity = 0;
  ~StageBuffer() {
    // At process teardown the HIP runtime may already be gone: errors are moot.
    if (ptr) (void)hipFree(ptr);
  }
};
thread_local StageBuffer tl_stage[3];

// Static staging memory of the allocation-free entry point: one array per
// device, owned by the code object, resolved to a device address once per
// device (the array's name is only a host-side handle for that lookup).
constexpr size_t kScratchBytes = (size_t)IREE_UK_MI355X_NOALLOC_MAX_STAGED_BYTES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
std::atomic<unsigned char*> g_scratch_ptr[kMaxDevices];
// One call at a time may stage host operands in a device's array: taken with a
// try-lock (a second caller is told so instead of waiting or corrupting the
// first one's operands), held until the call's results are back on the host.
std::atomic<bool> g_scratch_busy[kMaxDevices];

struct ScratchLease {
  std::atomic<bool>* flag = nullptr;
  ScratchLease() = default;
  ScratchLease(const ScratchLease&) = delete;
  ScratchLease& operator=(const ScratchLease&) = delete;
  ~ScratchLease() {
    if (flag) flag->store(false, std::memory_order_release);
  }
};

// Device address of the current device's `scratch` (nullptr after reporting
// a failure).
unsigned char* scratch_for_current_device(int* device_out = nullptr) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (device_out) *device_out = device;
  unsigned char* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (ptr) return ptr;
  void* resolved = nullptr;
  if (hipGetSymbolAddress(&resolved, HIP_SYMBOL(scratch)) != hipSuccess || !resolved) {
    (void)hipGetLastError();
    return nullptr;
  }
  // Two threads racing here resolve the same address.
  g_scratch_ptr[device].store((unsigned char*)resolved, std::memory_order_release);
  return (unsigned char*)resolved;
}

// Where the calling entry point mirrors host operands: the thread's grow-only
// buffers (may call hipMalloc), or a bump allocator over the device's static
// scratch (never allocates; fails when the operands do not fit).
struct Stager {
  unsigned char* fixed_base = nullptr;  // non-null: static scratch
  size_t fixed_used = 0;
  bool no_alloc = false;
  bool copies_issued = false;           // something was enqueued on the stream for this call
  ScratchLease lease;                   // held while the static scratch is in use
};

size_t rounded_for_scratch(size_t bytes) { return (bytes + 255) & ~(size_t)255; }

bool stage_reserve(Stager& stager, int slot, size_t bytes, void** out) {
  if (stager.no_alloc) {
    if (!stager.fixed_base) {
      int device = -1;
      unsigned char* base = scratch_for_current_device(&device);
      if (!base) {
        report_failure(__FILE__, __LINE__, __func__, "hipGetSymbolAddress(scratch) failed on the current device");
        return false;
      }
      bool expected = false;
      if (!g_scratch_busy[device].compare_exchange_strong(expected, true, std::memory_order_acq_rel)) {
        report_failure(__FILE__, __LINE__, __func__,
                       "static staging memory busy: another iree_uk_mi355x_mmt4d_noalloc_p call with host "
                       "operands is running on this device");
        return false;
      }
      stager.lease.flag = &g_scratch_busy[device];
      stager.fixed_base = base;
    }
    const size_t rounded = rounded_for_scratch(bytes);
    if (rounded > kScratchBytes - stager.fixed_used) {
      report_failure(__FILE__, __LINE__, __func__,
                     "host operands exceed IREE_UK_MI355X_NOALLOC_MAX_STAGED_BYTES of static staging memory");
      return false;
    }
    *out = stager.fixed_base + stager.fixed_used;
    stager.fixed_used += rounded;
    return true;
  }
  StageBuffer& s = tl_stage[slot];
  if (s.capacity < bytes) {
    if (s.ptr) UK_HIP_OK(hipFree(s.ptr));
    s.ptr = nullptr;
    s.capacity = 0;
    size_t cap = bytes + bytes / 4 + 256;
    UK_HIP_OK(hipMalloc(&s.ptr, cap));
    s.capacity = cap;
  }
  *out = s.ptr;
  return true;
}

// int64 arithmetic on caller-provided sizes that records overflow instead of
// wrapping (the checks of the reference admit sizes whose products do not fit).
struct Checked {
  bool ok = true;
  int64_t mul(int64_t a, int64_t b) {
    int64_t r = 0;
    if (__builtin_mul_overflow(a, b, &r)) ok = false;
    return ok ? r : 0;
  }
  int64_t add(int64_t a, int64_t b) {
    int64_t r = 0;
    if (__builtin_add_overflow(a, b, &r)) ok = false;
    return ok ? r : 0;
  }
  // Bytes of `elems` elements of `bits` bits each (sub-byte types: the callers
  // have checked that the count is a whole number of bytes).
  int64_t bytes(int64_t elems, int bits) { return bits >= 8 ? mul(elems, bits / 8) : elems / (8 / bits); }
};

// `base + bytes` without the undefined behaviour of pointer arithmetic outside
// an object: callers may pass `allocation - offset` as the base.
const uint8_t* offset_pointer(const void* base, int64_t bytes) {
  return (const uint8_t*)((uintptr_t)base + (uintptr_t)bytes);
}

// A strided set of rows inside one operand: `rows` rows of `width` bytes,
// `pitch` bytes apart; `span` is the byte count from the first to the last
// touched byte.
struct RowRegion {
  int64_t rows = 0, width = 0, pitch = 0, span = 0;
};

RowRegion make_region(Checked& c, int64_t rows, int64_t width, int64_t pitch) {
  RowRegion r;
  r.rows = rows; r.width = width; r.pitch = pitch;
  r.span = rows <= 0 || width <= 0 ? 0 : c.add(c.mul(rows - 1, pitch), width);
  return r;
}

// The same bytes as one row (for operands whose rows overlap or interleave).
RowRegion as_one_span(const RowRegion& r) {
  RowRegion o;
  o.rows = 1; o.width = r.span; o.pitch = 0; o.span = r.span;
  return o;
}

bool copy_rows(void* dst, const void* src, const RowRegion& r, hipMemcpyKind kind, hipStream_t s) {
  if (r.span == 0) return true;
  if (r.rows == 1 || r.pitch == r.width) {
    UK_HIP_OK(hipMemcpyAsync(dst, src, (size_t)r.span, kind, s));
  } else {
    UK_HIP_OK(hipMemcpy2DAsync(dst, (size_t)r.pitch, src, (size_t)r.pitch, (size_t)r.width,
                               (size_t)r.rows, kind, s));
  }
  return true;
}

// Makes one operand reachable from the device. For a host operand the region is
// mirrored at the same layout in a staging buffer; `upload` says whether its
// current contents are needed on the device.
struct Staged {
  const void* host = nullptr;  // non-null iff staged
  void* dev = nullptr;
};

bool stage_operand(Stager& stager, int slot, const void* ptr, const RowRegion& region, bool upload,
                   hipStream_t stream, Staged* st, const void** dev_ptr, int known_on_device = -1) {
  *dev_ptr = ptr;
  if (region.span == 0) return true;
  const bool on_device = known_on_device < 0 ? device_accessible(ptr) : known_on_device != 0;
  if (tl_async) {
    // Nothing is staged in asynchronous mode, and a host address must not
    // reach a kernel: the device would fault.
    if (!on_device) {
      report_failure(__FILE__, __LINE__, __func__, "asynchronous mode needs device-accessible operands");
      return false;
    }
    return true;
  }
  if (on_device) return true;
  void* d = nullptr;
  if (!stage_reserve(stager, slot, (size_t)region.span, &d)) return false;
  if (upload) {
    stager.copies_issued = true;
    if (!copy_rows(d, ptr, region, hipMemcpyHostToDevice, stream)) return false;
  }
  st->host = ptr;
  st->dev = d;
  *dev_ptr = d;
  return true;
}

bool finish(hipStream_t stream, const Staged& out, const RowRegion& out_region, bool any_staged) {
  if (out.host && !copy_rows(const_cast<void*>(out.host), out.dev, out_region,
                             hipMemcpyDeviceToHost, stream)) {
    if (!tl_async) (void)hipStreamSynchronize(stream);
    return false;
  }
  if (!tl_async) UK_HIP_OK(hipStreamSynchronize(stream));
  (void)any_staged;
  return true;
}

bool launch_ok(hipError_t e, const char* what) {
  if (e == hipSuccess) return true;
  char msg[256];
  snprintf(msg, sizeof msg, "%s launch -> %s", what, hipGetErrorString(e));
  report_failure(__FILE__, __LINE__, __func__, msg);
  return false;
}

// Leaves an entry point early after a failure: in synchronous mode nothing
// of the call may still be in flight when it returns (uploads read the
// caller's memory, and the staging memory is about to be handed on).
void abandon(const Stager& stager, hipStream_t stream) {
  if (!tl_async && stager.copies_issued) (void)hipStreamSynchronize(stream);
}

uk::Mmt4dLauncher select_mmt4d(const uk::Mmt4dArgs& a, bool probe_only) {
  uk::Mmt4dLauncher l = nullptr;
  if ((l = uk::select_mmt4d_gemv(a, probe_only))) return l;
  const uk::Mmt4dLauncher skinny = uk::select_mmt4d_skinny(a, probe_only);
  if (skinny && (probe_only || uk::mmt4d_skinny_preferred(a))) return skinny;
  if ((l = uk::select_mmt4d_mfma(a, probe_only))) return l;
  return skinny;
}

int pack_elem_bytes(uint32_t flags) {
  switch (flags & IREE_UK_FLAG_PACK_TYPE_MASK) {
    case IREE_UK_FLAG_PACK_TYPE_F32F32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_I8I8: return 1;
    case IREE_UK_FLAG_PACK_TYPE_I32I32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_F16F16: return 2;
    case IREE_UK_FLAG_PACK_TYPE_BF16BF16: return 2;
    default: return 0;
  }
}

int unpack_elem_bytes(uint32_t flags) {
  switch (flags & IREE_UK_FLAG_UNPACK_TYPE_MASK) {
    case IREE_UK_FLAG_UNPACK_TYPE_F32F32: return 4;
    case IREE_UK_FLAG_UNPACK_TYPE_I32I32: return 4;
    case IREE_UK_FLAG_UNPACK_TYPE_F16F16: return 2;
    case IREE_UK_FLAG_UNPACK_TYPE_BF16BF16: return 2;
    default: return 0;
  }
}

}  // namespace

//===----------------------------------------------------------------------===//
// mmt4d
//===----------------------------------------------------------------------===//

namespace {

void mmt4d_impl(const iree_uk_mmt4d_params_t* p, Stager& stager) {
  tl_last_kernel = "";
  UK_REQUIRE(p != nullptr);
  // Checks of mmt4d.c:12-48.
  const uint32_t known = IREE_UK_FLAG_MMT4D_TYPE_MASK | IREE_UK_FLAG_MMT4D_ACCUMULATE |
                         IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS |
                         IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION;
  UK_REQUIRE(!(p->flags & ~known));
  int lb = 0, rb = 0, ob = 0;
  UK_REQUIRE(uk::mmt4d_type_bits(p->flags, &lb, &rb, &ob));
  UK_REQUIRE(in_unsigned_range(p->M, 31));
  UK_REQUIRE(in_unsigned_range(p->N, 31));
  UK_REQUIRE(in_unsigned_range(p->K, 31));
  UK_REQUIRE(in_unsigned_range(p->M0, 15));
  UK_REQUIRE(in_unsigned_range(p->N0, 15));
  UK_REQUIRE(in_unsigned_range(p->K0, 15));
  UK_REQUIRE(ob >= 8);
  UK_REQUIRE((p->K0 * lb) % 8 == 0);
  UK_REQUIRE((p->K0 * rb) % 8 == 0);
  // (stride * bits) % 8 without forming the product.
  UK_REQUIRE(((p->lhs_stride0 % 8) * lb) % 8 == 0);
  UK_REQUIRE(((p->rhs_stride0 % 8) * rb) % 8 == 0);
  UK_REQUIRE(((p->lhs_offset % 8) * lb) % 8 == 0);
  UK_REQUIRE(((p->rhs_offset % 8) * rb) % 8 == 0);

  // Early exits of mmt4d.c:105-113. (K == 0 without ACCUMULATE still has to
  // zero the output tiles, so it goes on to a kernel.)
  const bool accumulate = p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE;
  if (p->M == 0 || p->N == 0 || (p->K == 0 && accumulate)) return;
  if (p->M0 == 0 || p->N0 == 0) return;  // empty tiles: nothing to write

  Checked c;
  const RowRegion lhs_region = make_region(c, p->M, c.bytes(c.mul(p->K, (int64_t)p->M0 * p->K0), lb),
                                           c.bytes(p->lhs_stride0, lb));
  const RowRegion rhs_region = make_region(c, p->N, c.bytes(c.mul(p->K, (int64_t)p->N0 * p->K0), rb),
                                           c.bytes(p->rhs_stride0, rb));
  const RowRegion out_region = make_region(c, p->M, c.bytes(c.mul(p->N, (int64_t)p->M0 * p->N0), ob),
                                           c.bytes(p->out_stride0, ob));
  const int64_t lhs_offset_bytes = c.bytes(p->lhs_offset, lb), rhs_offset_bytes = c.bytes(p->rhs_offset, rb),
                out_offset_bytes = c.bytes(p->out_offset, ob);
  UK_REQUIRE(c.ok && "operand extents fit int64");
  // The reference puts no condition on the strides (mmt4d.c:12-48). Operand
  // rows may overlap or coincide (stride 0 broadcasts one panel); they are
  // only read. Rows of the output may not overlap here, because they are
  // written concurrently, and strides that walk backwards are not supported.
  UK_REQUIRE(p->M == 1 || p->lhs_stride0 >= 0);
  UK_REQUIRE(p->N == 1 || p->rhs_stride0 >= 0);
  UK_REQUIRE(p->M == 1 || out_region.pitch >= out_region.width);

  const void* lhs = offset_pointer(p->lhs_buffer, lhs_offset_bytes);
  const void* rhs = offset_pointer(p->rhs_buffer, rhs_offset_bytes);
  const void* out = offset_pointer(p->out_buffer, out_offset_bytes);

  hipStream_t stream = tl_stream;
  Staged s_lhs, s_rhs, s_out;
  const void *d_lhs, *d_rhs, *d_out;
  // A host operand whose rows overlap is staged as one span.
  auto as_copied = [](const RowRegion& r) { return r.rows > 1 && r.pitch < r.width ? as_one_span(r) : r; };
  const RowRegion lhs_copy = as_copied(lhs_region), rhs_copy = as_copied(rhs_region);
  int lhs_dev = -1, rhs_dev = -1, out_dev = -1;
  if (stager.no_alloc && !tl_async) {
    // Whether the host operands fit the static memory is settled before the
    // first byte is copied.
    lhs_dev = lhs_copy.span == 0 || device_accessible(lhs);
    rhs_dev = rhs_copy.span == 0 || device_accessible(rhs);
    out_dev = out_region.span == 0 || device_accessible(out);
    Checked need;
    int64_t total = 0;
    if (!lhs_dev) total = need.add(total, need.add(lhs_copy.span, 255) & ~(int64_t)255);
    if (!rhs_dev) total = need.add(total, need.add(rhs_copy.span, 255) & ~(int64_t)255);
    if (!out_dev) total = need.add(total, need.add(out_region.span, 255) & ~(int64_t)255);
    if (!need.ok || total > (int64_t)kScratchBytes) {
      report_failure(__FILE__, __LINE__, __func__,
                     "host operands exceed IREE_UK_MI355X_NOALLOC_MAX_STAGED_BYTES of static staging memory");
      return;
    }
  }
  if (!stage_operand(stager, 0, lhs, lhs_copy, true, stream, &s_lhs, &d_lhs, lhs_dev) ||
      !stage_operand(stager, 1, rhs, rhs_copy, true, stream, &s_rhs, &d_rhs, rhs_dev) ||
      !stage_operand(stager, 2, out, out_region, accumulate, stream, &s_out, &d_out, out_dev)) {
    abandon(stager, stream);
    return;
  }

  uk::Mmt4dArgs a;
  a.lhs = (const uint8_t*)d_lhs;
  a.rhs = (const uint8_t*)d_rhs;
  a.out = (uint8_t*)const_cast<void*>(d_out);
  a.lhs_stride0 = p->lhs_stride0;
  a.rhs_stride0 = p->rhs_stride0;
  a.out_stride0 = p->out_stride0;
  a.M = p->M; a.N = p->N; a.K = p->K;
  a.M0 = p->M0; a.N0 = p->N0; a.K0 = p->K0;
  a.flags = p->flags;

  // The int4 kernels carry 16x the sums in int32, which holds for a total depth
  // below 131072. A deeper product is computed as a chain of calls over slices
  // of K, every slice after the first accumulating onto the output (exact:
  // int32 addition wraps the same way in any grouping).
  const int64_t depth_limit = 131072;
  if ((p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) == IREE_UK_FLAG_MMT4D_TYPE_S8S4S32 && p->K0 > 0 &&
      p->K * p->K0 >= depth_limit && select_mmt4d(a, /*probe_only=*/true)) {
    // (A multiple of 8 k steps: whole 128-value steps of the matrix-vector kernel, whole chunks of the block kernels.)
    int64_t slice = (depth_limit - 1) / p->K0;
    if (slice > 8) slice &= ~(int64_t)7;
    for (int64_t k = 0; k < p->K; k += slice) {
      uk::Mmt4dArgs part = a;
      part.K = p->K - k < slice ? p->K - k : slice;
      part.lhs = a.lhs + k * p->M0 * p->K0;
      part.rhs = a.rhs + k * p->N0 * p->K0 / 2;
      if (k > 0) part.flags |= IREE_UK_FLAG_MMT4D_ACCUMULATE;
      uk::Mmt4dLauncher launcher = select_mmt4d(part, /*probe_only=*/false);
      if (!launcher) launcher = uk::launch_mmt4d_generic;
      if (!launch_ok(launcher(part, stream, &tl_last_kernel), "mmt4d")) {
        abandon(stager, stream);
        return;
      }
    }
    finish(stream, s_out, out_region, s_lhs.host || s_rhs.host || s_out.host);
    return;
  }

  uk::Mmt4dLauncher launcher = select_mmt4d(a, /*probe_only=*/false);
  if (!launcher) launcher = uk::launch_mmt4d_generic;
  if (!launch_ok(launcher(a, stream, &tl_last_kernel), "mmt4d")) {
    abandon(stager, stream);
    return;
  }
  finish(stream, s_out, out_region, s_lhs.host || s_rhs.host || s_out.host);
}

}  // namespace

UK_API void iree_uk_mmt4d_p(const iree_uk_mmt4d_params_t* p) {
  Stager stager;
  mmt4d_impl(p, stager);
}

UK_API void iree_uk_mi355x_mmt4d_noalloc_p(const iree_uk_mmt4d_params_t* p) {
  Stager stager;
  stager.no_alloc = true;
  mmt4d_impl(p, stager);
}

UK_API void iree_uk_mmt4d(const void* lhs_buffer, iree_uk_index_t lhs_offset,
                          iree_uk_index_t lhs_stride0, const void* rhs_buffer,
                          iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0,
                          void* out_buffer, iree_uk_index_t out_offset, iree_uk_index_t out_stride0,
                          iree_uk_index_t M, iree_uk_index_t N, iree_uk_index_t K, int32_t M0,
                          int32_t N0, int32_t K0, uint32_t flags, const uint64_t* cpu_data) {
  iree_uk_mmt4d_params_t p;
  p.lhs_buffer = lhs_buffer; p.lhs_offset = lhs_offset; p.lhs_stride0 = lhs_stride0;
  p.rhs_buffer = rhs_buffer; p.rhs_offset = rhs_offset; p.rhs_stride0 = rhs_stride0;
  p.out_buffer = out_buffer; p.out_offset = out_offset; p.out_stride0 = out_stride0;
  p.M = M; p.N = N; p.K = K; p.M0 = M0; p.N0 = N0; p.K0 = K0;
  p.flags = flags; p.cpu_data = cpu_data;
  iree_uk_mmt4d_p(&p);
}

UK_API uint32_t iree_uk_mmt4d_info_p(const iree_uk_mmt4d_params_t* p) {
  if (!p) return 0;
  int lb, rb, ob;
  if (!uk::mmt4d_type_bits(p->flags, &lb, &rb, &ob)) return 0;
  uk::Mmt4dArgs a;
  memset(&a, 0, sizeof a);
  a.M0 = p->M0; a.N0 = p->N0; a.K0 = p->K0;
  a.flags = p->flags;
  return select_mmt4d(a, /*probe_only=*/true)
             ? IREE_UK_FLAG_MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
             : 0u;
}

UK_API uint32_t iree_uk_mmt4d_info(int32_t M0, int32_t N0, int32_t K0, uint32_t flags,
                                   const uint64_t* cpu_data) {
  iree_uk_mmt4d_params_t p;
  memset(&p, 0, sizeof p);
  p.M0 = M0; p.N0 = N0; p.K0 = K0; p.flags = flags; p.cpu_data = cpu_data;
  return iree_uk_mmt4d_info_p(&p);
}

//===----------------------------------------------------------------------===//
// pack
//===----------------------------------------------------------------------===//

UK_API void iree_uk_pack_p(const iree_uk_pack_params_t* p) {
  tl_last_kernel = "";
  UK_REQUIRE(p != nullptr);
  // Checks of pack.c:51-103. The reference additionally limits one tile to its
  // 4 KiB stack buffer (pack.c:39-49); nothing here needs that limit.
  const uint32_t known = IREE_UK_FLAG_PACK_TRANSPOSE_INNER | IREE_UK_FLAG_PACK_TRANSPOSE_OUTER |
                         IREE_UK_FLAG_PACK_TYPE_MASK;
  UK_REQUIRE(!(p->flags & ~known));
  const int e = pack_elem_bytes(p->flags);
  UK_REQUIRE(e != 0);
  UK_REQUIRE(p->in_size0 >= 0);
  UK_REQUIRE(p->in_size1 >= 0);
  UK_REQUIRE(p->out_size0 >= 0);
  UK_REQUIRE(p->out_size1 >= 0);
  UK_REQUIRE(p->out_size2 >= 0);
  UK_REQUIRE(p->out_size3 >= 0);
  UK_REQUIRE(p->in_stride0 >= 0);
  UK_REQUIRE(p->in_stride1 >= 0);
  UK_REQUIRE(p->out_stride0 >= 0);
  Checked c;
  UK_REQUIRE(p->out_stride1 == c.mul(p->out_size2, p->out_size3) && c.ok);
  int64_t outer0 = p->out_size0, outer1 = p->out_size1;
  int64_t tile0 = p->out_size2, tile1 = p->out_size3;
  if (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER) { int64_t t = outer0; outer0 = outer1; outer1 = t; }
  if (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER) { int64_t t = tile0; tile0 = tile1; tile1 = t; }
  UK_REQUIRE(tiles_cover(outer0, tile0, p->in_size0));
  UK_REQUIRE(tiles_cover(outer1, tile1, p->in_size1));

  // Early exit of pack.c:106-109.
  if (p->out_size0 == 0 || p->out_size1 == 0 || p->out_size2 == 0 || p->out_size3 == 0) return;

  const bool have_input = p->in_size0 > 0 && p->in_size1 > 0;
  const RowRegion in_region =
      make_region(c, have_input ? p->in_size0 : 0, c.mul(c.add(c.mul(p->in_size1 - 1, p->in_stride1), 1), e),
                  c.mul(p->in_stride0, e));
  const RowRegion out_region = make_region(
      c, p->out_size0, c.mul(c.mul(p->out_size1, p->out_stride1), e), c.mul(p->out_stride0, e));
  const int64_t in_offset_bytes = c.mul(p->in_offset, e), out_offset_bytes = c.mul(p->out_offset, e);
  UK_REQUIRE(c.ok && "operand extents fit int64");
  UK_REQUIRE(p->out_size0 == 1 || out_region.pitch >= out_region.width);

  const void* in = offset_pointer(p->in_buffer, in_offset_bytes);
  const void* out = offset_pointer(p->out_buffer, out_offset_bytes);

  hipStream_t stream = tl_stream;
  Staged s_in, s_out;
  const void *d_in, *d_out;
  // A host input whose rows overlap or interleave (stride0 < row width) is
  // staged as one span.
  RowRegion in_copy = in_region;
  if (in_copy.rows > 1 && in_copy.pitch < in_copy.width) in_copy = as_one_span(in_region);
  Stager stager;
  if (!stage_operand(stager, 0, in, in_copy, true, stream, &s_in, &d_in) ||
      !stage_operand(stager, 2, out, out_region, false, stream, &s_out, &d_out)) {
    abandon(stager, stream);
    return;
  }

  uk::PackArgs a;
  a.in = (const uint8_t*)d_in;
  a.out = (uint8_t*)const_cast<void*>(d_out);
  a.in_stride0 = p->in_stride0; a.in_stride1 = p->in_stride1;
  a.out_stride0 = p->out_stride0;
  a.in_size0 = p->in_size0; a.in_size1 = p->in_size1;
  a.out_size0 = p->out_size0; a.out_size1 = p->out_size1;
  a.out_size2 = p->out_size2; a.out_size3 = p->out_size3;
  a.padding_value = p->padding_value;
  a.flags = p->flags;
  a.elem_bytes = e;
  if (!launch_ok(uk::launch_pack(a, stream, &tl_last_kernel), "pack")) {
    abandon(stager, stream);
    return;
  }
  finish(stream, s_out, out_region, s_in.host || s_out.host);
}

UK_API void iree_uk_pack(const void* in_buffer, iree_uk_index_t in_offset, iree_uk_index_t in_stride0,
                         iree_uk_index_t in_stride1, void* out_buffer, iree_uk_index_t out_offset,
                         iree_uk_index_t out_stride0, iree_uk_index_t out_stride1,
                         iree_uk_index_t in_size0, iree_uk_index_t in_size1,
                         iree_uk_index_t out_size0, iree_uk_index_t out_size1,
                         iree_uk_index_t out_size2, iree_uk_index_t out_size3,
                         uint64_t padding_value, uint32_t flags, const uint64_t* cpu_data) {
  iree_uk_pack_params_t p;
  p.in_buffer = in_buffer; p.in_offset = in_offset;
  p.in_stride0 = in_stride0; p.in_stride1 = in_stride1;
  p.out_buffer = out_buffer; p.out_offset = out_offset;
  p.out_stride0 = out_stride0; p.out_stride1 = out_stride1;
  p.in_size0 = in_size0; p.in_size1 = in_size1;
  p.out_size0 = out_size0; p.out_size1 = out_size1;
  p.out_size2 = out_size2; p.out_size3 = out_size3;
  p.padding_value = padding_value; p.flags = flags; p.cpu_data = cpu_data;
  iree_uk_pack_p(&p);
}

//===----------------------------------------------------------------------===//
// unpack
//===----------------------------------------------------------------------===//

UK_API void iree_uk_unpack_p(const iree_uk_unpack_params_t* p) {
  tl_last_kernel = "";
  UK_REQUIRE(p != nullptr);
  // Checks of unpack.c:31-81 (tile-size limit of its stack buffer left out).
  const uint32_t known = IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER |
                         IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER | IREE_UK_FLAG_UNPACK_TYPE_MASK;
  UK_REQUIRE(!(p->flags & ~known));
  const int e = unpack_elem_bytes(p->flags);
  UK_REQUIRE(e != 0);
  UK_REQUIRE(p->out_size0 >= 0);
  UK_REQUIRE(p->out_size1 >= 0);
  UK_REQUIRE(p->in_size0 >= 0);
  UK_REQUIRE(p->in_size1 >= 0);
  UK_REQUIRE(p->in_size2 >= 0);
  UK_REQUIRE(p->in_size3 >= 0);
  UK_REQUIRE(p->in_stride0 >= 0);
  Checked c;
  UK_REQUIRE(p->in_stride1 == c.mul(p->in_size2, p->in_size3) && c.ok);
  UK_REQUIRE(p->out_stride0 >= 0);
  UK_REQUIRE(p->out_stride1 >= 0);
  int64_t outer0 = p->in_size0, outer1 = p->in_size1;
  int64_t tile0 = p->in_size2, tile1 = p->in_size3;
  if (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER) { int64_t t = outer0; outer0 = outer1; outer1 = t; }
  if (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER) { int64_t t = tile0; tile0 = tile1; tile1 = t; }
  UK_REQUIRE(tiles_cover(outer0, tile0, p->out_size0));
  UK_REQUIRE(tiles_cover(outer1, tile1, p->out_size1));

  // Early exit of unpack.c:84-86.
  if (p->out_size0 == 0 || p->out_size1 == 0) return;

  const RowRegion in_region =
      make_region(c, p->in_size0, c.mul(c.mul(p->in_size1, p->in_stride1), e), c.mul(p->in_stride0, e));
  const RowRegion out_region =
      make_region(c, p->out_size0, c.mul(c.add(c.mul(p->out_size1 - 1, p->out_stride1), 1), e),
                  c.mul(p->out_stride0, e));
  const int64_t in_offset_bytes = c.mul(p->in_offset, e), out_offset_bytes = c.mul(p->out_offset, e);
  UK_REQUIRE(c.ok && "operand extents fit int64");
  UK_REQUIRE(p->in_size0 == 1 || in_region.pitch >= in_region.width);
  UK_REQUIRE(p->out_size0 == 1 || out_region.pitch >= out_region.width);

  const void* in = offset_pointer(p->in_buffer, in_offset_bytes);
  const void* out = offset_pointer(p->out_buffer, out_offset_bytes);

  hipStream_t stream = tl_stream;
  Staged s_in, s_out;
  const void *d_in, *d_out;
  Stager stager;
  // With an inner output stride the bytes between elements must survive the
  // round trip through the staging buffer, so the rows are uploaded first.
  if (!stage_operand(stager, 0, in, in_region, true, stream, &s_in, &d_in) ||
      !stage_operand(stager, 2, out, out_region, p->out_stride1 != 1, stream, &s_out, &d_out)) {
    abandon(stager, stream);
    return;
  }

  uk::UnpackArgs a;
  a.in = (const uint8_t*)d_in;
  a.out = (uint8_t*)const_cast<void*>(d_out);
  a.in_stride0 = p->in_stride0;
  a.out_stride0 = p->out_stride0; a.out_stride1 = p->out_stride1;
  a.in_size0 = p->in_size0; a.in_size1 = p->in_size1;
  a.in_size2 = p->in_size2; a.in_size3 = p->in_size3;
  a.out_size0 = p->out_size0; a.out_size1 = p->out_size1;
  a.flags = p->flags;
  a.elem_bytes = e;
  if (!launch_ok(uk::launch_unpack(a, stream, &tl_last_kernel), "unpack")) {
    abandon(stager, stream);
    return;
  }
  finish(stream, s_out, out_region, s_in.host || s_out.host);
}

UK_API void iree_uk_unpack(const void* in_buffer, iree_uk_index_t in_offset,
                           iree_uk_index_t in_stride0, iree_uk_index_t in_stride1, void* out_buffer,
                           iree_uk_index_t out_offset, iree_uk_index_t out_stride0,
                           iree_uk_index_t out_stride1, iree_uk_index_t in_size0,
                           iree_uk_index_t in_size1, iree_uk_index_t in_size2,
                           iree_uk_index_t in_size3, iree_uk_index_t out_size0,
                           iree_uk_index_t out_size1, uint32_t flags, const uint64_t* cpu_data) {
  iree_uk_unpack_params_t p;
  p.in_buffer = in_buffer; p.in_offset = in_offset;
  p.in_stride0 = in_stride0; p.in_stride1 = in_stride1;
  p.out_buffer = out_buffer; p.out_offset = out_offset;
  p.out_stride0 = out_stride0; p.out_stride1 = out_stride1;
  p.in_size0 = in_size0; p.in_size1 = in_size1; p.in_size2 = in_size2; p.in_size3 = in_size3;
  p.out_size0 = out_size0; p.out_size1 = out_size1;
  p.flags = flags; p.cpu_data = cpu_data;
  iree_uk_unpack_p(&p);
}

//===----------------------------------------------------------------------===//
// query_tile_sizes
//===----------------------------------------------------------------------===//

UK_API void iree_uk_query_tile_sizes_2d(const iree_uk_query_tile_sizes_2d_params_t* p,
                                        iree_uk_query_tile_sizes_2d_out_params_t* o) {
  UK_REQUIRE(p != nullptr && o != nullptr);
  // Tile shapes whose mmt4d runs on an MFMA kernel of this library: one
  // 16x16 MFMA output block per tile, K0 = the bytes one lane feeds per MFMA.
  int M0 = 16, N0 = 16, K0 = 0;
  switch (p->flags & IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK) {
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32: K0 = 64; break;
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32:
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F16:
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16F32:
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16BF16: K0 = 16; break;
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F32F32F32: K0 = 4; break;
    default: break;
  }
  UK_REQUIRE(K0 != 0);
  switch (p->flags & IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK) {
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_LHS: o->tile_size0 = M0; o->tile_size1 = K0; break;
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RHS: o->tile_size0 = N0; o->tile_size1 = K0; break;
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RESULT: o->tile_size0 = M0; o->tile_size1 = N0; break;
    default: UK_REQUIRE(!"unknown operand role");
  }
}

//===----------------------------------------------------------------------===//
// Entry points without a reference counterpart
//===----------------------------------------------------------------------===//

UK_API int iree_uk_mi355x_multi_mma_i32_16x16x64_i8(const void* a, const void* b, void* c, long long outer_m,
                                                    long long outer_n, int32_t k_size, int32_t intrinsics_m,
                                                    int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n,
                                                    int32_t intrinsics_k) {
  tl_last_kernel = "";
  // Device pointers only: the data-tiled operands of a GPU dispatch never live on the host.
  if (!device_accessible(a) || !device_accessible(b) || !device_accessible(c)) return (int)hipErrorInvalidValue;
  const hipError_t e = uk::launch_multi_mma_i8(a, b, c, outer_m, outer_n, k_size, intrinsics_m, subgroups_m,
                                               intrinsics_n, subgroups_n, intrinsics_k, tl_stream);
  if (e != hipSuccess) return (int)e;
  tl_last_kernel = "multi_mma_i32_16x16x64_i8";
  if (!tl_async) {
    const hipError_t s = hipStreamSynchronize(tl_stream);
    if (s != hipSuccess) return (int)s;
  }
  return 0;
}

UK_API int iree_uk_mi355x_version(void) { return 100; }

UK_API int iree_uk_mi355x_init(int device_ordinal) {
  hipError_t e = device_ordinal < 0 ? hipGetDevice(&device_ordinal) : hipSetDevice(device_ordinal);
  if (e != hipSuccess) return (int)e;
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, device_ordinal);
  if (e != hipSuccess) return (int)e;
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return (int)hipErrorInvalidDevice;
  // Resolve this device's static staging memory now, so that the
  // allocation-free entry point does nothing but copies and launches.
  if (device_ordinal < kMaxDevices && hipSetDevice(device_ordinal) == hipSuccess &&
      !scratch_for_current_device())
    return (int)hipErrorInvalidSymbol;
  return 0;
}

UK_API void iree_uk_mi355x_set_stream(void* stream, int asynchronous) {
  tl_stream = (hipStream_t)stream;
  tl_async = asynchronous != 0;
}

UK_API void iree_uk_mi355x_set_fail_handler(iree_uk_mi355x_fail_handler_t handler) {
  g_fail_handler.store(handler, std::memory_order_release);
}

UK_API const char* iree_uk_mi355x_last_kernel(void) { return tl_last_kernel; }
