/*
 * C ABI of the MI355X (gfx950) data-tiled matmul microkernel library.
 *
 * The first group of entry points keeps the names, argument order, argument
 * meaning, struct layouts and flag values of the reference CPU microkernels in
 * runtime/src/iree/builtins/ukernel so that a caller of those can link against
 * this library unchanged. The second group (prefix iree_uk_mi355x_) has no
 * counterpart in the reference: it exposes what a GPU implementation needs in
 * addition (device selection, stream-ordered launches).
 *
 * Pointer arguments may be host pointers or HIP device pointers. Classification
 * looks only at `buffer + offset` (never at `buffer` itself, which the
 * reference's own tests set to an address before the allocation), see
 * iree_uk_mi355x_set_stream() for the rules.
 *
 * Everything here is plain C: no HIP or torch types appear in a signature.
 */
#ifndef IREE_UK_MI355X_H_
#define IREE_UK_MI355X_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Signed 64-bit index type on 64-bit targets (reference: common.h:269-275). */
typedef long long iree_uk_index_t;

/*===--------------------------------------------------------------------===*/
/* Flag values. Fixed by the reference compiler and runtime sharing them      */
/* (reference: exported_bits.h:29-49, 56-66, 73-83).                          */
/*===--------------------------------------------------------------------===*/

#define IREE_UK_FLAG_MMT4D_TYPE_MASK 0xFF
#define IREE_UK_FLAG_MMT4D_TYPE_NONE 0x00
#define IREE_UK_FLAG_MMT4D_TYPE_F32F32F32 0x01
#define IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 0x02
#define IREE_UK_FLAG_MMT4D_TYPE_F16F16F32 0x03
#define IREE_UK_FLAG_MMT4D_TYPE_F16F16F16 0x04
#define IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32 0x05
#define IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16 0x06
#define IREE_UK_FLAG_MMT4D_TYPE_S16S16S32 0x07
#define IREE_UK_FLAG_MMT4D_TYPE_S16U4S32 0x08
#define IREE_UK_FLAG_MMT4D_TYPE_S16S8S32 0x09
#define IREE_UK_FLAG_MMT4D_TYPE_S8S4S32 0x0A
#define IREE_UK_FLAG_MMT4D_TYPE_END 0x0B
#define IREE_UK_FLAG_MMT4D_ACCUMULATE 0x100
#define IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION 0x200
#define IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS 0x400
#define IREE_UK_FLAG_MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION 0x1

#define IREE_UK_FLAG_PACK_TYPE_MASK 0xFF
#define IREE_UK_FLAG_PACK_TYPE_NONE 0x00
#define IREE_UK_FLAG_PACK_TYPE_F32F32 0x01
#define IREE_UK_FLAG_PACK_TYPE_I8I8 0x02
#define IREE_UK_FLAG_PACK_TYPE_I32I32 0x03
#define IREE_UK_FLAG_PACK_TYPE_F16F16 0x04
#define IREE_UK_FLAG_PACK_TYPE_BF16BF16 0x05
#define IREE_UK_FLAG_PACK_TRANSPOSE_INNER 0x100
#define IREE_UK_FLAG_PACK_TRANSPOSE_OUTER 0x200

#define IREE_UK_FLAG_UNPACK_TYPE_MASK 0xFF
#define IREE_UK_FLAG_UNPACK_TYPE_NONE 0x00
#define IREE_UK_FLAG_UNPACK_TYPE_F32F32 0x01
#define IREE_UK_FLAG_UNPACK_TYPE_I32I32 0x03
#define IREE_UK_FLAG_UNPACK_TYPE_F16F16 0x04
#define IREE_UK_FLAG_UNPACK_TYPE_BF16BF16 0x05
#define IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER 0x100
#define IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER 0x200

#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK 0xFF
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_NONE 0x00
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_LHS 0x01
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RHS 0x02
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RESULT 0x03
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK 0xFF00
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_NONE 0x0000
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F32F32F32 0x0100
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32 0x0200
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32 0x0300
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F16 0x0400
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16F32 0x0500
#define IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16BF16 0x0600

/*===--------------------------------------------------------------------===*/
/* Parameter structs (field order and types are ABI).                         */
/*===--------------------------------------------------------------------===*/

/* reference: mmt4d_internal.h:14-32. Offsets and strides count ELEMENTS of the
 * operand's type (4-bit elements included); M, N, K count tiles. Only the
 * outermost dimension of each operand is strided. */
typedef struct iree_uk_mmt4d_params_t {
  const void* lhs_buffer;
  iree_uk_index_t lhs_offset;
  iree_uk_index_t lhs_stride0;
  const void* rhs_buffer;
  iree_uk_index_t rhs_offset;
  iree_uk_index_t rhs_stride0;
  void* out_buffer;
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t M;
  iree_uk_index_t N;
  iree_uk_index_t K;
  int32_t M0;
  int32_t N0;
  int32_t K0;
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_mmt4d_params_t;

/* reference: pack_internal.h:12-30. */
typedef struct iree_uk_pack_params_t {
  const void* in_buffer;
  iree_uk_index_t in_offset;
  iree_uk_index_t in_stride0;
  iree_uk_index_t in_stride1;
  void* out_buffer;
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t out_stride1;
  iree_uk_index_t in_size0;
  iree_uk_index_t in_size1;
  iree_uk_index_t out_size0;
  iree_uk_index_t out_size1;
  iree_uk_index_t out_size2;
  iree_uk_index_t out_size3;
  uint64_t padding_value;
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_pack_params_t;

/* reference: unpack_internal.h:12-29. */
typedef struct iree_uk_unpack_params_t {
  const void* in_buffer;
  iree_uk_index_t in_offset;
  iree_uk_index_t in_stride0;
  iree_uk_index_t in_stride1;
  void* out_buffer;
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t out_stride1;
  iree_uk_index_t in_size0;
  iree_uk_index_t in_size1;
  iree_uk_index_t in_size2;
  iree_uk_index_t in_size3;
  iree_uk_index_t out_size0;
  iree_uk_index_t out_size1;
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_unpack_params_t;

/* reference: query_tile_sizes.h:17-27. */
typedef struct iree_uk_query_tile_sizes_2d_params_t {
  uint32_t flags;
  iree_uk_index_t size0;
  iree_uk_index_t size1;
  const uint64_t* cpu_data;
} iree_uk_query_tile_sizes_2d_params_t;

typedef struct iree_uk_query_tile_sizes_2d_out_params_t {
  iree_uk_index_t tile_size0;
  iree_uk_index_t tile_size1;
} iree_uk_query_tile_sizes_2d_out_params_t;

/*===--------------------------------------------------------------------===*/
/* Entry points shared with the reference.                                    */
/*===--------------------------------------------------------------------===*/

/* out[M,N,M0,N0] (+)= lhs[M,K,M0,K0] * rhs[N,K,N0,K0]^T.
 * Replaces: mmt4d.h:14-21 (flat form), mmt4d_internal.h:35 (struct form),
 * implemented by mmt4d.c:115-177. `cpu_data` is accepted and ignored (may be
 * NULL). IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION is accepted;
 * tile shapes without an MFMA kernel always run on the generic GPU kernel.
 * Strides (the reference checks none, mmt4d.c:12-48): lhs_stride0 and
 * rhs_stride0 may be anything non-negative, 0 and values shorter than a panel
 * included (panels that coincide or overlap are only read). Deviations, both
 * reported through the failure handler with the output left untouched: output
 * rows that overlap (M > 1 and out_stride0 < N * M0 * N0; they are written
 * concurrently here) and negative strides where there is more than one row.
 * Tiles one row tall (M0 = 1) make a row-major [M, K] matrix the lhs and a
 * row-major [M, N * N0] matrix the result as they stand: no pack of the lhs
 * and no unpack are needed then. */
void iree_uk_mmt4d(const void* lhs_buffer, iree_uk_index_t lhs_offset,
                   iree_uk_index_t lhs_stride0, const void* rhs_buffer,
                   iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0,
                   void* out_buffer, iree_uk_index_t out_offset,
                   iree_uk_index_t out_stride0, iree_uk_index_t M,
                   iree_uk_index_t N, iree_uk_index_t K, int32_t M0, int32_t N0,
                   int32_t K0, uint32_t flags, const uint64_t* cpu_data);
void iree_uk_mmt4d_p(const iree_uk_mmt4d_params_t* params);

/* Bit 0 is set iff a kernel specialised for (type, M0, N0, K0) exists, here an
 * MFMA or bandwidth-tuned kernel rather than the one-thread-per-element one.
 * Replaces: mmt4d.h:25-27, mmt4d_internal.h:40, mmt4d.c:143-149,179-185. */
uint32_t iree_uk_mmt4d_info(int32_t M0, int32_t N0, int32_t K0, uint32_t flags,
                            const uint64_t* cpu_data);
uint32_t iree_uk_mmt4d_info_p(const iree_uk_mmt4d_params_t* params);

/* 2-D -> 4-D tiled copy with padding and optional inner/outer transposes.
 * Replaces: pack.h:26-34, pack_internal.h:32, pack.c:315-352. */
void iree_uk_pack(const void* in_buffer, iree_uk_index_t in_offset,
                  iree_uk_index_t in_stride0, iree_uk_index_t in_stride1,
                  void* out_buffer, iree_uk_index_t out_offset,
                  iree_uk_index_t out_stride0, iree_uk_index_t out_stride1,
                  iree_uk_index_t in_size0, iree_uk_index_t in_size1,
                  iree_uk_index_t out_size0, iree_uk_index_t out_size1,
                  iree_uk_index_t out_size2, iree_uk_index_t out_size3,
                  uint64_t padding_value, uint32_t flags,
                  const uint64_t* cpu_data);
void iree_uk_pack_p(const iree_uk_pack_params_t* params);

/* Inverse of pack; writes only the out_size0 x out_size1 logical region.
 * Replaces: unpack.h:17-25, unpack_internal.h:31, unpack.c:249-285. */
void iree_uk_unpack(const void* in_buffer, iree_uk_index_t in_offset,
                    iree_uk_index_t in_stride0, iree_uk_index_t in_stride1,
                    void* out_buffer, iree_uk_index_t out_offset,
                    iree_uk_index_t out_stride0, iree_uk_index_t out_stride1,
                    iree_uk_index_t in_size0, iree_uk_index_t in_size1,
                    iree_uk_index_t in_size2, iree_uk_index_t in_size3,
                    iree_uk_index_t out_size0, iree_uk_index_t out_size1,
                    uint32_t flags, const uint64_t* cpu_data);
void iree_uk_unpack_p(const iree_uk_unpack_params_t* params);

/* Tile sizes the matmul kernels of this library prefer for an operand.
 * Replaces: query_tile_sizes.h:29-31, query_tile_sizes.c:34-75. */
void iree_uk_query_tile_sizes_2d(
    const iree_uk_query_tile_sizes_2d_params_t* params,
    iree_uk_query_tile_sizes_2d_out_params_t* out_params);

/* Called when a parameter check or a HIP call fails. The library provides a
 * weak default that prints to stderr and aborts; an embedder may define its
 * own (reference: common.h:307-321 leaves the definition to the embedder). If
 * the handler returns, the entry point returns without launching anything. */
void iree_uk_assert_fail(const char* file, int line, const char* function,
                         const char* condition);

/*===--------------------------------------------------------------------===*/
/* Entry points without a counterpart in the reference.                       */
/*===--------------------------------------------------------------------===*/

/* The in-dispatch int8 microkernel of the ROCm backend's calling convention
 * for gfx950 (iree_amd/csrc/device/iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8.h;
 * the reference has the gfx942 one, compiler/plugins/target/ROCM/builtins/
 * ukernel/iree_uk_amdgpu_multi_mma_mfma_i32_16x16x32_i8.c:82-181), run over a
 * grid of outer_m x outer_n data-tiled tiles, one workgroup each:
 *   a: [outer_m][k_size][subgroups_m][intrinsics_m][64][intrinsics_k] vectors of 16 int8,
 *   b: [outer_n][k_size][subgroups_n][intrinsics_n][64][intrinsics_k],
 *   c: [outer_m][outer_n][subgroups_m][subgroups_n][intrinsics_m][intrinsics_n][64] vectors of 4 int32,
 * c += a * b^T in the MFMA's operand layout (lane l of an A/B vector block: row
 * l % 16, K bytes 16*(l / 16)..+15 of 64; lane l of a C block: rows
 * 4*(l / 16)+{0..3}, column l % 16). Device pointers only. The parameter
 * combinations are compile-time instantiations; returns 0, or a HIP error
 * code (hipErrorInvalidValue for a combination that is not instantiated). It
 * exists to test and measure the device microkernel; there is no host entry
 * point like it in the reference. */
int iree_uk_mi355x_multi_mma_i32_16x16x64_i8(const void* a, const void* b, void* c, long long outer_m,
                                             long long outer_n, int32_t k_size, int32_t intrinsics_m,
                                             int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n,
                                             int32_t intrinsics_k);

/* iree_uk_mmt4d_p for callers that cannot allocate. It has no counterpart in
 * the reference (whose microkernels never allocate, being CPU code); it is for
 * callers that may not call hipMalloc where they call a microkernel: tight
 * serving loops, harnesses that forbid allocation, code around HIP graph
 * capture. Same parameters, checks, kernels and results as iree_uk_mmt4d_p.
 * The difference: operands at host addresses are mirrored in a fixed array of
 * IREE_UK_MI355X_NOALLOC_MAX_STAGED_BYTES of device memory that the library's
 * code object holds on every device it runs on until the process ends, instead
 * of in staging buffers grown with hipMalloc. Each host operand takes its span
 * (first to last touched byte) rounded up to 256 bytes; a call whose host
 * operands need more in total reports "host operands exceed ..." through the
 * failure handler and returns without launching. Device operands take none.
 * The call makes no hipMalloc/hipFree. All calls on one device share that
 * array, one at a time: a call with host operands holds it from its first
 * upload until its results are back on the host, and a second such call that
 * arrives on the same device meanwhile (from another thread) is not run: it
 * reports "static staging memory busy" through the failure handler and
 * returns, leaving its output untouched; the caller may repeat it. The array
 * keeps the previous call's bytes, and nothing read from it is ever older
 * than the current call's own uploads. iree_uk_mi355x_init resolves the
 * array's address ahead of the first call.
 * Under stream capture itself only the asynchronous mode can be used (a
 * synchronous call copies and synchronises, which capture forbids), and that
 * mode takes device operands only: nothing is staged there, and this entry
 * point then does exactly what iree_uk_mmt4d_p does, which allocates nothing
 * for device operands either. */
#define IREE_UK_MI355X_NOALLOC_MAX_STAGED_BYTES (16 * 1024 * 1024)
void iree_uk_mi355x_mmt4d_noalloc_p(const iree_uk_mmt4d_params_t* params);

/* Library version, MAJOR*10000 + MINOR*100 + PATCH. */
int iree_uk_mi355x_version(void);

/* Selects the HIP device for the calling thread's launches and checks that it
 * is a gfx950 part; a negative ordinal checks the thread's current device
 * without selecting another. Returns 0 on success, a HIP error code otherwise.
 * Calling it is optional: the first launch uses the current HIP device. */
int iree_uk_mi355x_init(int device_ordinal);

/* Per-thread launch mode.
 *   stream:  a hipStream_t cast to void* (NULL = the HIP null stream).
 *   asynchronous == 0 (default): each entry point returns after its results are
 *     visible, like the CPU microkernels. Operands whose `buffer + offset` is
 *     not a device address are staged: copied to device memory owned by the
 *     library, computed there, and the touched rows copied back.
 *   asynchronous != 0: entry points only enqueue work on `stream` and return;
 *     every operand must be device-accessible; nothing is staged or
 *     synchronised. */
void iree_uk_mi355x_set_stream(void* stream, int asynchronous);

/* Replaces the failure handler for the calling process (NULL restores
 * iree_uk_assert_fail). Meant for hosts that cannot provide a strong
 * iree_uk_assert_fail symbol at link time. */
typedef void (*iree_uk_mi355x_fail_handler_t)(const char* file, int line,
                                              const char* function,
                                              const char* condition);
void iree_uk_mi355x_set_fail_handler(iree_uk_mi355x_fail_handler_t handler);

/* Name of the kernel the calling thread's most recent entry point launched
 * ("" if it returned early). Static storage; do not free. */
const char* iree_uk_mi355x_last_kernel(void);

#ifdef __cplusplus
}
#endif

#endif /* IREE_UK_MI355X_H_ */
