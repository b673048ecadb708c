// LDS-staged pack / unpack for power-of-two tile sizes: HBM-bandwidth kernels.
//
// A workgroup owns a BR x BC block of the 2-D matrix (BR a multiple of the tile
// height T0, BC a multiple of the tile width T1). The block's image in the
// tiled buffer is a small number of long contiguous runs: with no outer
// transpose the BC/T1 tiles of one tile row follow each other, with an outer
// transpose the BR/T0 tiles of one tile column do. So both sides of the copy
// can be done with wide, fully coalesced accesses and the re-ordering happens
// in LDS:
//   pack:    2-D rows -> LDS (row-major, padded pitch) -> tiled runs (128-bit)
//   unpack:  tiled runs (128-bit) -> LDS -> 2-D rows
// The 2-D side uses 16-byte vectors whatever the alignment of the rows.
// Element values are never interpreted: the kernels move bytes, so results are
// bit-exact by construction; padding is the low bytes of padding_value
// (pack.h:15-24).
//
// With an inner transpose the tiled side's 16 contiguous bytes are 16 / E
// consecutive ROWS of one column. For 4-byte elements that is four 32-bit LDS
// reads per vector; for 1- and 2-byte elements it would be 16 or 8 narrow
// reads, which makes the kernel LDS-instruction bound (3.5 TB/s for int8). Pack
// with such elements goes through pack_transposing_kernel instead: a thread
// loads 16 bytes from each of 4 / E consecutive rows, transposes the 4x4 bytes
// (2x2 halfwords) blocks in registers (v_perm_b32), and writes dwords into an
// LDS image that is already in tiled order; the tiled side then is one 128-bit
// LDS read and one 128-bit store per vector.
//
// With an element stride on the 2-D side (in_stride1 / out_stride1 other than
// 1, which the reference handles in its tile path through a temporary row,
// pack.c:227) the 2-D side is accessed element by element, the stride apart;
// the LDS image and the tiled side stay as they are.
//
// Anything this file does not cover (non power-of-two tiles, unaligned tiled
// buffers) goes to the generic kernels.
#include <cstdlib>
#include <mutex>
#include <type_traits>
#include <vector>

#include "uk_internal.h"

namespace uk {

hipError_t launch_pack_generic(const PackArgs& a, hipStream_t stream, const char** name);
hipError_t launch_unpack_generic(const UnpackArgs& a, hipStream_t stream, const char** name);

namespace {

struct TiledArgs {
  const uint8_t* src;   // pack: 2-D buffer, unpack: tiled buffer
  uint8_t* dst;         // pack: tiled buffer, unpack: 2-D buffer
  int64_t flat_stride0;   // 2-D side row stride, elements
  int64_t flat_stride1;   // 2-D side element stride, elements (1: rows are contiguous)
  int64_t tiled_stride0;  // tiled side outer stride, elements
  int64_t size0, size1;   // 2-D sizes
  int64_t outer0, outer1; // tile counts along 2-D dims 0 / 1
  uint64_t padding_value;
  int32_t log2_t0, log2_t1;  // tile sizes along 2-D dims 0 / 1
  int32_t log2_s3;           // log2 of the tiled buffer's innermost size
  int32_t log2_br, log2_bc;  // block shape
  int32_t pitch_bytes;       // LDS row pitch
  int32_t blocks1;           // blocks along dim 1
  int32_t total_blocks;
  int32_t tr_inner, tr_outer;
  // pack_transposing_kernel only: consecutive lanes along a row before the next
  // row group starts, and the LDS image's skew (pad_bytes inserted every
  // 1 << log2_period bytes).
  int32_t log2_lpr, log2_period, pad_bytes;
  int32_t band;  // rows of blocks that are walked together (block_of)
  int32_t ext_cols;  // line-aligned unpack only: columns a block reads beyond its own
  // linear_block_of: consecutive blocks that one XCD takes, workgroups per XCD
  // that are dealt out that way, and blocks per XCD of the rest.
  int32_t group, grouped_slots, rest_per_xcd;
};

// Coordinates of an element of the tiled side within a block.
struct TiledCoord {
  int64_t global_elem;  // element offset in the tiled buffer
  int32_t row, col;     // position in the block (2-D side)
  bool in_range;        // tile exists in the tiled buffer
};

// Element `e` (in the block's tiled-side enumeration: runs in order, each run
// tile after tile, each tile in stored order) -> where it lives.
__device__ __forceinline__ TiledCoord tiled_coord(const TiledArgs& a, int32_t e, int64_t tile0_base,
                                                  int64_t tile1_base) {
  const int32_t log2_tile = a.log2_t0 + a.log2_t1;
  int32_t o0l, o1l, w;
  if (!a.tr_outer) {
    const int32_t log2_run = a.log2_bc + a.log2_t0;  // elements per run (one tile row of the block)
    o0l = e >> log2_run;
    const int32_t rem = e & ((1 << log2_run) - 1);
    o1l = rem >> log2_tile;
    w = rem & ((1 << log2_tile) - 1);
  } else {
    const int32_t log2_run = a.log2_br + a.log2_t1;  // one tile column of the block
    o1l = e >> log2_run;
    const int32_t rem = e & ((1 << log2_run) - 1);
    o0l = rem >> log2_tile;
    w = rem & ((1 << log2_tile) - 1);
  }
  const int32_t u2 = w >> a.log2_s3, u3 = w & ((1 << a.log2_s3) - 1);
  const int32_t t0 = a.tr_inner ? u3 : u2, t1 = a.tr_inner ? u2 : u3;
  TiledCoord c;
  c.row = (o0l << a.log2_t0) + t0;
  c.col = (o1l << a.log2_t1) + t1;
  const int64_t o0 = tile0_base + o0l, o1 = tile1_base + o1l;
  c.in_range = o0 < a.outer0 && o1 < a.outer1;
  const int64_t q0 = a.tr_outer ? o1 : o0, q1 = a.tr_outer ? o0 : o1;
  c.global_elem = q0 * a.tiled_stride0 + (q1 << log2_tile) + w;
  return c;
}

// Block number -> block coordinates. Blocks with consecutive numbers run at
// about the same time. Without an outer transpose they go along a row of
// blocks: each block's tiled side is one long run anyway, and neighbours read
// adjacent pieces of the same rows. With an outer transpose a block's tiled
// side is many short runs (one per tile column), and the next piece of each
// run belongs to the block BELOW: there `band` rows of blocks are walked
// together, down the rows first, so that neighbours in time extend each
// other's runs (measured on 16384^2 int8 into [n][k][16][16]: 4.9 TB/s with
// band 1, 5.9 TB/s with 16).
__device__ __forceinline__ void block_of(const TiledArgs& a, int32_t linear, int64_t* block0, int64_t* block1) {
  if (a.band <= 1) {
    *block0 = linear / a.blocks1;
    *block1 = linear % a.blocks1;
    return;
  }
  const int32_t blocks0 = a.total_blocks / a.blocks1;
  const int32_t g = linear / (a.band * a.blocks1), first = g * a.band;
  const int32_t rows_here = min(a.band, blocks0 - first);
  const int32_t i = linear - g * a.band * a.blocks1;
  *block0 = first + i % rows_here;
  *block1 = i / rows_here;
}

// Workgroup id -> block number. Consecutive workgroup ids land on different
// XCDs (separate L2s): workgroup 8 s + x runs on XCD x. Blocks are dealt to
// the XCDs in groups of a.group consecutive numbers: within a group,
// neighbours along a row share the cache lines at their common edge (rows
// need not be aligned to lines) and meet in one L2; across groups, the eight
// XCDs work side by side on one compact stretch of both buffers instead of
// on eight stretches an eighth of the matrix apart. Measured on f32
// [8191, 8190] with 16x1 tiles (32 blocks per row), group 1 / 16..128 / an
// eighth of all blocks: pack 5.77 / 6.01-6.04 / 5.92 TB/s, unpack 5.99 /
// 6.08-6.10 / 5.90, the copy-like pack into [8191, 512, 1, 16] 5.97 / 6.10-6.15
// / 5.68; walking bands of rows (block_of), one band's blocks per group:
// pack with both transposes 5.73 against 5.31-5.39 (groups of 16..256) and
// 5.54 (an eighth of all blocks).
// What does not fill eight whole groups any more is split into eight equal
// stretches, so that no XCD is left with a group more than the others.
__device__ __forceinline__ int32_t linear_block_of(const TiledArgs& a) {
  const uint32_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, group = (uint32_t)a.group;
  if (slot < (uint32_t)a.grouped_slots) {
    const uint32_t g = slot / group;
    return (int32_t)((g * 8 + xcd) * group + (slot - g * group));
  }
  const uint32_t r = slot - (uint32_t)a.grouped_slots;
  return (int32_t)((uint32_t)a.grouped_slots * 8 + xcd * (uint32_t)a.rest_per_xcd + r);
}

// 16 bytes without an alignment requirement: the hardware's multi-dword
// global accesses have none, the C++ type system would.
struct __attribute__((packed, aligned(1))) Dwords4 {
  uint32_t x, y, z, w;
};

constexpr int kBlockBytes = 16384;  // bytes of the 2-D matrix per workgroup

// E: element bytes. W: vector bytes on the 2-D side (16 needs 4-byte aligned
// rows). PL_BYTES: bytes of one contiguous LDS piece on the tiled side (16 when
// 16 output bytes come from one LDS row, down to E for column access).
//
// LINE_ALIGNED (unpack of 4-byte, and where rows are whole dwords apart 2-byte, elements into rows that do not start on
// 128-byte lines, blocks one tile row tall): each row's piece of a block is
// moved right to the next line boundary of THAT row, so a wavefront's 1 KiB
// store is eight whole lines and no line is written in two parts by two
// workgroups. Row r of block b then covers columns [b * BC + s(r), (b + 1) * BC
// + s(r)), s(r) < 128 / E being the distance from the block's first column to
// the row's next line boundary; the first block of a row starts at column 0
// and the last one ends with the row. A block therefore also reads the
// ext_cols columns of the tiles that follow its own. The LDS image is that of
// the block and those columns, unmoved; the 2-D side reads row r's vectors
// s(r) elements in (16-byte reads at element alignment). Measured on f32
// [512, 8190, 16, 1] -> [8191, 8190]: 5.60 -> 5.88 TB/s; with the stores moved
// but the extra columns not read (wrong results) 6.08: the 1/8 more lines
// requested on the tiled side cost what is left, whether or not the loads are
// masked down to the rows that are used, and although the lines shared by two
// blocks come from HBM only once.
template <int E, int W, int PL_BYTES, bool UNPACK, int LINE_ALIGNED = 0>  // (1: line-aligned unpack, 2: the same with an outer transpose)
__global__ __launch_bounds__(256) void tiled_kernel(const TiledArgs a) {
  static_assert(!LINE_ALIGNED || (UNPACK && W == 16), "line-aligned windows are for unpack");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  typedef typename std::conditional<E == 1, uint8_t,
          typename std::conditional<E == 2, uint16_t, uint32_t>::type>::type elem_t;
  typedef typename std::conditional<W == 16, Dwords4,
          typename std::conditional<W == 8, uint2,
          typename std::conditional<W == 4, uint32_t,
          typename std::conditional<W == 2, uint16_t, uint8_t>::type>::type>::type>::type flat_vec_t;
  typedef typename std::conditional<PL_BYTES == 16, uint4,
          typename std::conditional<PL_BYTES == 8, uint2,
          typename std::conditional<PL_BYTES == 4, uint32_t,
          typename std::conditional<PL_BYTES == 2, uint16_t, uint8_t>::type>::type>::type>::type piece_t;
  static_assert(sizeof(flat_vec_t) == W && W >= E, "2-D side vector type");
  constexpr int VE = 16 / E;          // elements per 128-bit tiled-side vector
  constexpr int PIECES = 16 / PL_BYTES;
  constexpr int PL = PL_BYTES / E;    // elements per piece
  constexpr int EPV = W / E;          // elements per 2-D side vector
  constexpr int FLAT_PER_THREAD = kBlockBytes / W / 256;
  constexpr int TILED_PER_THREAD = kBlockBytes / 16 / 256;
  constexpr int LOG2_E = E == 1 ? 0 : E == 2 ? 1 : 2;
  constexpr int LOG2_W = W == 16 ? 4 : W == 8 ? 3 : W == 4 ? 2 : W == 2 ? 1 : 0;

  const int tid = threadIdx.x;
  const int32_t linear = linear_block_of(a);
  if (linear >= a.total_blocks) return;
  int64_t block0, block1;
  block_of(a, linear, &block0, &block1);
  const int64_t row_base = block0 << a.log2_br, col_base = block1 << a.log2_bc;
  const int64_t tile0_base = row_base >> a.log2_t0, tile1_base = col_base >> a.log2_t1;
  const int32_t log2_vpr = a.log2_bc + LOG2_E - LOG2_W;  // 2-D side vectors per block row
  const int32_t vpr_mask = (1 << log2_vpr) - 1;

  union FlatVec {
    flat_vec_t vec;
    elem_t elem[EPV];
  };

  // ---- 2-D rows -> LDS (pack), all global loads issued before the LDS stores ----
  // (STRIDED: elements of a row lie flat_stride1 elements apart.)
  auto flat_load_phase = [&](auto strided) {
    constexpr bool STRIDED = decltype(strided)::value;
    constexpr int BATCH = FLAT_PER_THREAD < 8 ? FLAT_PER_THREAD : 8;
    for (int u0 = 0; u0 < FLAT_PER_THREAD; u0 += BATCH) {
      FlatVec regs[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int32_t v = tid + 256 * (u0 + u);
        const int32_t r = v >> log2_vpr, cv = v & vpr_mask;
        const int64_t row = row_base + r, col = col_base + (int64_t)cv * EPV;
        const uint8_t* g = a.src + (row * a.flat_stride0 + (STRIDED ? col * a.flat_stride1 : col)) * E;
        if (!STRIDED && row < a.size0 && col + EPV <= a.size1) {
          // Every byte is read once: streaming (non-temporal) accesses on both
          // sides leave the caches to the other side's partial lines.
          if constexpr (W == 16) {
            typedef int v4a4 __attribute__((ext_vector_type(4), aligned(1)));
            const v4a4 t = __builtin_nontemporal_load((const v4a4*)g);
            regs[u].vec = Dwords4{(uint32_t)t.x, (uint32_t)t.y, (uint32_t)t.z, (uint32_t)t.w};
          } else {
            regs[u].vec = *(const flat_vec_t*)g;
          }
        } else {
          // Edge: element by element, padding where the input ends.
#pragma unroll
          for (int i = 0; i < EPV; ++i) {
            elem_t x = (elem_t)a.padding_value;
            if (row < a.size0 && col + i < a.size1) x = ((const elem_t*)g)[STRIDED ? i * a.flat_stride1 : i];
            regs[u].elem[i] = x;
          }
        }
      }
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int32_t v = tid + 256 * (u0 + u);
        const int32_t r = v >> log2_vpr, cv = v & vpr_mask;
        *(flat_vec_t*)(lds + r * a.pitch_bytes + cv * W) = regs[u].vec;
      }
    }
  };

  // ---- LDS -> 2-D rows (unpack), nothing written outside size0 x size1 ----
  auto flat_store_phase = [&](auto strided) {
    constexpr bool STRIDED = decltype(strided)::value;
    constexpr int BATCH = FLAT_PER_THREAD < 8 ? FLAT_PER_THREAD : 8;
    for (int u0 = 0; u0 < FLAT_PER_THREAD; u0 += BATCH) {
      FlatVec regs[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int32_t v = tid + 256 * (u0 + u);
        regs[u].vec = *(const flat_vec_t*)(lds + (v >> log2_vpr) * a.pitch_bytes + (v & vpr_mask) * W);
      }
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int32_t v = tid + 256 * (u0 + u);
        const int32_t r = v >> log2_vpr, cv = v & vpr_mask;
        const int64_t row = row_base + r, col = col_base + (int64_t)cv * EPV;
        uint8_t* g = a.dst + (row * a.flat_stride0 + (STRIDED ? col * a.flat_stride1 : col)) * E;
        if (!STRIDED && row < a.size0 && col + EPV <= a.size1) {
          // Whole vectors inside the matrix: written once, not read here.
          if constexpr (W == 16) {
            typedef int v4a1 __attribute__((ext_vector_type(4), aligned(1)));
            __builtin_nontemporal_store(v4a1{(int)regs[u].vec.x, (int)regs[u].vec.y, (int)regs[u].vec.z, (int)regs[u].vec.w}, (v4a1*)g);
          } else if constexpr (W == 8) {
            typedef int v2 __attribute__((ext_vector_type(2)));
            __builtin_nontemporal_store(v2{(int)regs[u].vec.x, (int)regs[u].vec.y}, (v2*)g);
          } else if constexpr (W == 4) {
            __builtin_nontemporal_store(regs[u].vec, (flat_vec_t*)g);
          } else
          *(flat_vec_t*)g = regs[u].vec;
        } else if (row < a.size0) {
#pragma unroll
          for (int i = 0; i < EPV; ++i)
            if (col + i < a.size1) ((elem_t*)g)[STRIDED ? i * a.flat_stride1 : i] = regs[u].elem[i];
        }
      }
    }
  };

  union TiledVec {
    uint4 vec;
    piece_t piece[PIECES];
  };

  // ---- tiled side <-> LDS ----
  auto tiled_phase = [&]() {
    TiledVec regs[TILED_PER_THREAD];
    TiledCoord first[TILED_PER_THREAD];
#pragma unroll
    for (int u = 0; u < TILED_PER_THREAD; ++u) {
      const int32_t e = (tid + 256 * u) * VE;
      first[u] = tiled_coord(a, e, tile0_base, tile1_base);
      if constexpr (UNPACK) {
        if (first[u].in_range) {
          typedef int v4 __attribute__((ext_vector_type(4)));
          regs[u].vec = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4*)(a.src + first[u].global_elem * E)));
        }
      }
    }
#pragma unroll
    for (int u = 0; u < TILED_PER_THREAD; ++u) {
      if (!first[u].in_range) continue;
      const int32_t e = (tid + 256 * u) * VE;
#pragma unroll
      for (int q = 0; q < PIECES; ++q) {
        int32_t row = first[u].row, col = first[u].col;
        if (q > 0) {
          const TiledCoord c = tiled_coord(a, e + q * PL, tile0_base, tile1_base);
          row = c.row;
          col = c.col;
        }
        piece_t* l = (piece_t*)(lds + row * a.pitch_bytes + col * E);
        if constexpr (UNPACK) *l = regs[u].piece[q]; else regs[u].piece[q] = *l;
      }
      if constexpr (!UNPACK) {
        // Whole tiles, written once, never read back here: streaming store.
        typedef int v4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(v4, regs[u].vec), (v4*)(a.dst + first[u].global_elem * E));
      }
    }
  };

  if constexpr (LINE_ALIGNED) {
    constexpr int MAX_TILED = TILED_PER_THREAD + (LINE_ALIGNED == 2 ? 2 : 4);  // (the host keeps to these)
    const int32_t bc = 1 << a.log2_bc;
    const int32_t log2_tile = a.log2_t0 + a.log2_t1;
    const bool first_block = block1 == 0;
    // Distance (elements) from the block's first column to row r's next line.
    const uint32_t row_bytes = (uint32_t)((uint64_t)a.flat_stride0 * E) & 127u;
    const uint32_t to_line0 = (uint32_t)(0 - (uintptr_t)(a.dst + (row_base * a.flat_stride0 + col_base) * E)) & 127u;
    auto shift_of = [&](int32_t r) -> int32_t { return (int32_t)((to_line0 - (uint32_t)r * row_bytes) & 127u) / E; };
    // The tiled side: the block's own tiles and the ext_cols columns of tiles
    // after them, whole (which rows of those columns fall into this block's
    // windows is not looked at: a partly masked load touches the same lines,
    // and working it out ahead of the loads costs more than it saves). Nothing
    // of the window arithmetic comes before the loads: a workgroup lives for a
    // few microseconds, and what it computes first is time with nothing in
    // flight. The columns around a block's edge are read by two blocks: those
    // loads leave their lines in the cache for the other one, the rest stream.
    // A thread's vectors are 256 vectors apart, a whole number of tiles (the
    // host sees to that): all of them are the same pieces of their tiles.
    typedef int v4 __attribute__((ext_vector_type(4)));
    const int32_t e0 = tid * VE, w0 = e0 & ((1 << log2_tile) - 1);
    const uint8_t* const tile_row = a.src + (tile0_base * a.tiled_stride0 + w0) * E;
    const int32_t total_vecs = ((bc + a.ext_cols) << a.log2_br) / VE;
    TiledVec regs[MAX_TILED];
    bool wanted[MAX_TILED];
    if constexpr (LINE_ALIGNED == 2) {
      // Outer transpose: the tiled side is one run per tile column, and the columns after the block's own
      // are further runs; the block's enumeration simply goes on (tiled_coord).
      TiledCoord first[MAX_TILED];
#pragma unroll
      for (int u = 0; u < MAX_TILED; ++u) {
        const int32_t vec = tid + 256 * u;
        first[u] = tiled_coord(a, vec * VE, tile0_base, tile1_base);
        wanted[u] = vec < total_vecs && first[u].in_range;
        if (wanted[u]) {
          const uint8_t* g = a.src + first[u].global_elem * E;
          if (first[u].col < 128 / E || first[u].col >= bc)
            regs[u].vec = *(const uint4*)g;
          else
            regs[u].vec = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4*)g));
        }
      }
#pragma unroll
      for (int u = 0; u < MAX_TILED; ++u) {
        if (!wanted[u]) continue;
#pragma unroll
        for (int q = 0; q < PIECES; ++q) {
          int32_t row = first[u].row, col = first[u].col;
          if (q > 0) {
            const TiledCoord c = tiled_coord(a, (tid + 256 * u) * VE + q * PL, tile0_base, tile1_base);
            row = c.row;
            col = c.col;
          }
          *(piece_t*)(lds + row * a.pitch_bytes + col * E) = regs[u].piece[q];
        }
      }
    } else {
#pragma unroll
    for (int u = 0; u < MAX_TILED; ++u) {
      const int32_t vec = tid + 256 * u, o1l = (vec * VE) >> log2_tile, col0 = o1l << a.log2_t1;
      wanted[u] = vec < total_vecs && tile1_base + o1l < a.outer1;
      if (wanted[u]) {
        const uint8_t* g = tile_row + (((tile1_base + o1l) << log2_tile) * E);
        if (col0 < 128 / E || col0 >= bc)
          regs[u].vec = *(const uint4*)g;
        else
          regs[u].vec = __builtin_bit_cast(uint4, __builtin_nontemporal_load((const v4*)g));
      }
    }
    int32_t lds_base[PIECES];
#pragma unroll
    for (int q = 0; q < PIECES; ++q) {
      const int32_t w = w0 + q * PL, u2 = w >> a.log2_s3, u3 = w & ((1 << a.log2_s3) - 1);
      lds_base[q] = (a.tr_inner ? u3 : u2) * a.pitch_bytes + (a.tr_inner ? u2 : u3) * E;
    }
#pragma unroll
    for (int u = 0; u < MAX_TILED; ++u) {
      if (!wanted[u]) continue;
      const int32_t o1l = ((tid + 256 * u) * VE) >> log2_tile;
#pragma unroll
      for (int q = 0; q < PIECES; ++q) *(piece_t*)(lds + lds_base[q] + ((o1l << a.log2_t1) * E)) = regs[u].piece[q];
    }
    }
    __syncthreads();
    // Whole lines: vector cv of row r starts s(r) + cv * EPV columns into the block.
    {
      struct __attribute__((packed, aligned(4))) ShiftedVec {  // (the host sees to it that shifts are whole dwords)
        uint32_t x, y, z, w;
      };
      FlatVec out[FLAT_PER_THREAD];
#pragma unroll
      for (int u = 0; u < FLAT_PER_THREAD; ++u) {
        const int32_t v = tid + 256 * u, r = v >> log2_vpr;
        const ShiftedVec t = *(const ShiftedVec*)(lds + r * a.pitch_bytes + shift_of(r) * E + (v & vpr_mask) * W);
        out[u].vec = Dwords4{t.x, t.y, t.z, t.w};
      }
#pragma unroll
      for (int u = 0; u < FLAT_PER_THREAD; ++u) {
        const int32_t v = tid + 256 * u;
        const int32_t r = v >> log2_vpr, cv = v & vpr_mask;
        const int64_t row = row_base + r, col = col_base + shift_of(r) + (int64_t)cv * EPV;
        uint8_t* g = a.dst + (row * a.flat_stride0 + col) * E;
        if (row < a.size0 && col + EPV <= a.size1) {
          typedef int v4a1 __attribute__((ext_vector_type(4), aligned(1)));
          __builtin_nontemporal_store(v4a1{(int)out[u].vec.x, (int)out[u].vec.y, (int)out[u].vec.z, (int)out[u].vec.w}, (v4a1*)g);
        } else if (row < a.size0) {
#pragma unroll
          for (int i = 0; i < EPV; ++i)
            if (col + i < a.size1) ((elem_t*)g)[i] = out[u].elem[i];
        }
      }
    }
    // A row's first columns, up to its first line boundary.
    if (first_block) {
      constexpr int HEAD = 128 / E;
      for (int32_t i = tid; i < (HEAD << a.log2_br); i += 256) {
        const int32_t r = i / HEAD, c = i % HEAD;
        const int64_t row = row_base + r;
        if (c < shift_of(r) && row < a.size0 && c < a.size1)
          ((elem_t*)(a.dst + row * a.flat_stride0 * E))[c] = *(const elem_t*)(lds + r * a.pitch_bytes + c * E);
      }
    }
  } else if constexpr (!UNPACK) {
    if (a.flat_stride1 == 1) flat_load_phase(std::false_type()); else flat_load_phase(std::true_type());
    __syncthreads();
    tiled_phase();
  } else {
    tiled_phase();
    __syncthreads();
    if (a.flat_stride1 == 1) flat_store_phase(std::false_type()); else flat_store_phase(std::true_type());
  }
}

// Element (row, col) of a block -> its index in the block's tiled-side
// enumeration (the inverse of tiled_coord), for an inner transpose.
__host__ __device__ __forceinline__ int32_t tiled_index_tr_inner(const TiledArgs& a, int32_t row, int32_t col) {
  const int32_t log2_tile = a.log2_t0 + a.log2_t1;
  const int32_t o0l = row >> a.log2_t0, t0 = row & ((1 << a.log2_t0) - 1);
  const int32_t o1l = col >> a.log2_t1, t1 = col & ((1 << a.log2_t1) - 1);
  const int32_t w = (t1 << a.log2_t0) | t0;
  if (!a.tr_outer) return (o0l << (a.log2_bc + a.log2_t0)) | (o1l << log2_tile) | w;
  return (o1l << (a.log2_br + a.log2_t1)) | (o0l << log2_tile) | w;
}

__host__ __device__ __forceinline__ uint32_t skewed(const TiledArgs& a, uint32_t byte_offset) {
  return byte_offset + (byte_offset >> a.log2_period) * a.pad_bytes;
}

// Unit v (of the block's kBlockBytes / (RQ * 16)) -> its first row and column:
// 1 << log2_lpr units side by side along a row, then down all row groups, then
// the next stretch of columns.
__host__ __device__ __forceinline__ void transposing_unit(const TiledArgs& a, int32_t v, int rq, int ve, int32_t* row0,
                                                          int32_t* col0) {
  const int32_t log2_rg = a.log2_br - (rq == 4 ? 2 : 1);
  const int32_t cg_lo = v & ((1 << a.log2_lpr) - 1), rest = v >> a.log2_lpr;
  const int32_t rg = rest & ((1 << log2_rg) - 1), cg_hi = rest >> log2_rg;
  *row0 = rg * rq;
  *col0 = ((cg_hi << a.log2_lpr) | cg_lo) * ve;
}

// The same for tiles at least 16 bytes tall (T0 * E >= 16) and blocks at least
// 256 bytes wide: the four 16-lane rows of a wavefront load four consecutive
// groups of 4 / E rows of the same 256 bytes of columns and swap dwords among
// themselves (v_permlane32_swap, v_permlane16_swap: a 4x4 transpose of
// "register x lane row") so that each lane ends up with all 16 / E rows of 4 / E
// columns. After the byte transposes that is one whole 16-byte vector of the
// tiled side per column: 4 / E 128-bit LDS writes per lane instead of 16 / E
// dword writes, and a quarter of the address arithmetic.
template <int E>
__global__ __launch_bounds__(256) void pack_transposing_wide_kernel(const TiledArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  typedef typename std::conditional<E == 1, uint8_t, uint16_t>::type elem_t;
  constexpr int RQ = 4 / E;        // rows a lane loads; columns a lane ends up with
  constexpr int VE = 16 / E;       // columns per 16-byte vector; rows of a patch
  constexpr int PATCH_COLS = 256 / E;
  constexpr int UNITS = kBlockBytes / (VE * 256) / 4;  // patches per wavefront
  constexpr int TILED_PER_THREAD = kBlockBytes / 16 / 256;
  constexpr int LOG2_PATCH_COLS = E == 1 ? 8 : 7;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lane_row = lane >> 4, cg = lane & 15;
  const int32_t linear = linear_block_of(a);
  if (linear >= a.total_blocks) return;
  int64_t block0, block1;
  block_of(a, linear, &block0, &block1);
  const int64_t row_base = block0 << a.log2_br, col_base = block1 << a.log2_bc;
  const int64_t tile0_base = row_base >> a.log2_t0, tile1_base = col_base >> a.log2_t1;
  const int32_t log2_pcg = a.log2_bc - LOG2_PATCH_COLS;  // patches side by side in a block

  union RowVec {
    uint32_t dword[4];
    elem_t elem[VE];
  };
  RowVec regs[UNITS][RQ];
  int32_t patch_row[UNITS], patch_col[UNITS];
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    const int32_t patch = wave + 4 * u;
    patch_row[u] = (patch >> log2_pcg) * VE;
    patch_col[u] = (patch & ((1 << log2_pcg) - 1)) * PATCH_COLS;
#pragma unroll
    for (int j = 0; j < RQ; ++j) {
      const int64_t row = row_base + patch_row[u] + lane_row * RQ + j, col = col_base + patch_col[u] + cg * VE;
      const uint8_t* g = a.src + (row * a.flat_stride0 + col) * E;
      if (row < a.size0 && col + VE <= a.size1) {
        typedef int v4a4 __attribute__((ext_vector_type(4), aligned(1)));
        const v4a4 t = __builtin_nontemporal_load((const v4a4*)g);
        regs[u][j].dword[0] = t.x; regs[u][j].dword[1] = t.y; regs[u][j].dword[2] = t.z; regs[u][j].dword[3] = t.w;
      } else {
#pragma unroll
        for (int i = 0; i < VE; ++i) {
          elem_t x = (elem_t)a.padding_value;
          if (row < a.size0 && col + i < a.size1) x = ((const elem_t*)g)[i];
          regs[u][j].elem[i] = x;
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    // After this, dword k of regs[u][j] is what lane row k loaded as dword
    // `lane_row` of its row j: rows RQ*k + j of the patch, this lane's columns.
#pragma unroll
    for (int j = 0; j < RQ; ++j) {
      uint32_t* d = regs[u][j].dword;
      const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
      const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
      const auto s01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
      const auto s23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
      d[0] = s01[0]; d[1] = s01[1]; d[2] = s23[0]; d[3] = s23[1];
    }
    uint4 column[RQ];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      uint32_t out[RQ];
      if constexpr (E == 1) {
        const uint32_t ra = regs[u][0].dword[k], rb = regs[u][1].dword[k], rc = regs[u][2].dword[k], rd = regs[u][3].dword[k];
        const uint32_t ab_lo = __builtin_amdgcn_perm(rb, ra, 0x05010400u), ab_hi = __builtin_amdgcn_perm(rb, ra, 0x07030602u);
        const uint32_t cd_lo = __builtin_amdgcn_perm(rd, rc, 0x05010400u), cd_hi = __builtin_amdgcn_perm(rd, rc, 0x07030602u);
        out[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
        out[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
        out[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
        out[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
      } else {
        const uint32_t ra = regs[u][0].dword[k], rb = regs[u][1].dword[k];
        out[0] = __builtin_amdgcn_perm(rb, ra, 0x05040100u);
        out[1] = __builtin_amdgcn_perm(rb, ra, 0x07060302u);
      }
#pragma unroll
      for (int i = 0; i < RQ; ++i) {
        if (k == 0) column[i].x = out[i]; else if (k == 1) column[i].y = out[i]; else if (k == 2) column[i].z = out[i]; else column[i].w = out[i];
      }
    }
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      const int32_t e = tiled_index_tr_inner(a, patch_row[u], patch_col[u] + cg * VE + lane_row * RQ + i);
      *(uint4*)(lds + skewed(a, (uint32_t)e * E)) = column[i];
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < TILED_PER_THREAD; ++u) {
    const int32_t q = tid + 256 * u;
    const TiledCoord c = tiled_coord(a, q * VE, tile0_base, tile1_base);
    if (!c.in_range) continue;
    typedef int v4 __attribute__((ext_vector_type(4)));
    const v4 vec = *(const v4*)(lds + skewed(a, (uint32_t)q * 16));
    __builtin_nontemporal_store(vec, (v4*)(a.dst + c.global_elem * E));
  }
}

// Pack with an inner transpose for 1- and 2-byte elements (see the top of the
// file). A dword of the tiled side is RQ consecutive rows of 4 / (E * RQ)
// adjacent columns: RQ = 4 / E rows of one column for tiles at least that
// tall, or, for int8 tiles two rows tall (the [N0][2] layouts of the x86
// dot-product tiles), 2 rows of 2 columns.
template <int E, int RQ>
__global__ __launch_bounds__(256) void pack_transposing_kernel(const TiledArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  typedef typename std::conditional<E == 1, uint8_t, uint16_t>::type elem_t;
  static_assert((E == 1 && (RQ == 4 || RQ == 2)) || (E == 2 && RQ == 2), "rows per dword");
  constexpr int CQ = 4 / (E * RQ);  // columns per dword
  constexpr int NOUT = 4 / E / CQ;  // dwords made from one dword of each of the RQ rows
  constexpr int VE = 16 / E;        // columns per 16-byte vector
  constexpr int UNITS = kBlockBytes / (RQ * 16) / 256;
  constexpr int TILED_PER_THREAD = kBlockBytes / 16 / 256;

  const int tid = threadIdx.x;
  const int32_t linear = linear_block_of(a);
  if (linear >= a.total_blocks) return;
  int64_t block0, block1;
  block_of(a, linear, &block0, &block1);
  const int64_t row_base = block0 << a.log2_br, col_base = block1 << a.log2_bc;
  const int64_t tile0_base = row_base >> a.log2_t0, tile1_base = col_base >> a.log2_t1;

  union RowVec {
    uint32_t dword[4];
    elem_t elem[VE];
  };
  RowVec regs[UNITS][RQ];
  int32_t row0[UNITS], col0[UNITS];
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    transposing_unit(a, tid + 256 * u, RQ, VE, &row0[u], &col0[u]);
#pragma unroll
    for (int j = 0; j < RQ; ++j) {
      const int64_t row = row_base + row0[u] + j, col = col_base + col0[u];
      const uint8_t* g = a.src + (row * a.flat_stride0 + col) * E;
      if (row < a.size0 && col + VE <= a.size1) {
        typedef int v4a4 __attribute__((ext_vector_type(4), aligned(1)));
        const v4a4 t = __builtin_nontemporal_load((const v4a4*)g);
        regs[u][j].dword[0] = t.x; regs[u][j].dword[1] = t.y; regs[u][j].dword[2] = t.z; regs[u][j].dword[3] = t.w;
      } else {
#pragma unroll
        for (int i = 0; i < VE; ++i) {
          elem_t x = (elem_t)a.padding_value;
          if (row < a.size0 && col + i < a.size1) x = ((const elem_t*)g)[i];
          regs[u][j].elem[i] = x;
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      uint32_t out[NOUT];
      if constexpr (E == 1 && RQ == 4) {
        const uint32_t ra = regs[u][0].dword[k], rb = regs[u][1].dword[k], rc = regs[u][2].dword[k], rd = regs[u][3].dword[k];
        const uint32_t ab_lo = __builtin_amdgcn_perm(rb, ra, 0x05010400u), ab_hi = __builtin_amdgcn_perm(rb, ra, 0x07030602u);
        const uint32_t cd_lo = __builtin_amdgcn_perm(rd, rc, 0x05010400u), cd_hi = __builtin_amdgcn_perm(rd, rc, 0x07030602u);
        out[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
        out[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
        out[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
        out[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
      } else if constexpr (E == 1) {
        // Two rows: bytes (column c, row 0), (c, 1), (c + 1, 0), (c + 1, 1).
        const uint32_t ra = regs[u][0].dword[k], rb = regs[u][1].dword[k];
        out[0] = __builtin_amdgcn_perm(rb, ra, 0x05010400u);
        out[1] = __builtin_amdgcn_perm(rb, ra, 0x07030602u);
      } else {
        const uint32_t ra = regs[u][0].dword[k], rb = regs[u][1].dword[k];
        out[0] = __builtin_amdgcn_perm(rb, ra, 0x05040100u);
        out[1] = __builtin_amdgcn_perm(rb, ra, 0x07060302u);
      }
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        const int32_t e = tiled_index_tr_inner(a, row0[u], col0[u] + (4 / E) * k + CQ * i);
        *(uint32_t*)(lds + skewed(a, (uint32_t)e * E)) = out[i];
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < TILED_PER_THREAD; ++u) {
    const int32_t q = tid + 256 * u;
    const TiledCoord c = tiled_coord(a, q * VE, tile0_base, tile1_base);
    if (!c.in_range) continue;
    typedef int v4 __attribute__((ext_vector_type(4)));
    const v4 vec = *(const v4*)(lds + skewed(a, (uint32_t)q * 16));
    __builtin_nontemporal_store(vec, (v4*)(a.dst + c.global_elem * E));
  }
}

int log2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int l = 0;
  while ((1ll << l) < v) ++l;
  return l;
}

int largest_pow2_dividing(uint64_t v, int cap) {
  int w = 1;
  while (w < cap && (v % (2 * w)) == 0) w *= 2;
  return w;
}

// Host copy of tiled_coord's (row, col) for the bank-conflict search below.
void host_row_col(const TiledArgs& a, int32_t e, int32_t* row, int32_t* col) {
  const int32_t log2_tile = a.log2_t0 + a.log2_t1;
  int32_t o0l, o1l, w;
  if (!a.tr_outer) {
    const int32_t log2_run = a.log2_bc + a.log2_t0;
    o0l = e >> log2_run;
    const int32_t rem = e & ((1 << log2_run) - 1);
    o1l = rem >> log2_tile;
    w = rem & ((1 << log2_tile) - 1);
  } else {
    const int32_t log2_run = a.log2_br + a.log2_t1;
    o1l = e >> log2_run;
    const int32_t rem = e & ((1 << log2_run) - 1);
    o0l = rem >> log2_tile;
    w = rem & ((1 << log2_tile) - 1);
  }
  const int32_t u2 = w >> a.log2_s3, u3 = w & ((1 << a.log2_s3) - 1);
  const int32_t t0 = a.tr_inner ? u3 : u2, t1 = a.tr_inner ? u2 : u3;
  *row = (o0l << a.log2_t0) + t0;
  *col = (o1l << a.log2_t1) + t1;
}

// LDS row pitch: the block width plus the padding (in 16-byte steps) that
// spreads one wavefront's tiled-side accesses over the most of the 64 banks.
// (extra_cols: columns of the following tiles that the image holds as well.)
int choose_pitch(const TiledArgs& a, int elem_bytes, int piece_bytes, int extra_cols = 0) {
  const int row_bytes = ((1 << a.log2_bc) + extra_cols) * elem_bytes;
  const int ve = 16 / elem_bytes;
  int best_pitch = row_bytes, best_cost = 1 << 30;
  for (int pad = 0; pad <= 256; pad += 16) {
    const int pitch = row_bytes + pad;
    int hits[64] = {0};
    for (int lane = 0; lane < 64; ++lane) {
      int32_t row, col;
      host_row_col(a, lane * ve, &row, &col);
      const int addr = row * pitch + col * elem_bytes;
      const int words = piece_bytes < 4 ? 1 : piece_bytes / 4;
      for (int w = 0; w < words; ++w) hits[((addr / 4) + w) & 63]++;
    }
    int cost = 0;
    for (int b = 0; b < 64; ++b) cost = hits[b] > cost ? hits[b] : cost;
    if (cost < best_cost) {
      best_cost = cost;
      best_pitch = pitch;
    }
  }
  return best_pitch;
}

struct Plan {
  TiledArgs args;
  bool line_aligned;
  int elem_bytes, flat_vec_bytes, piece_bytes;
  unsigned grid;
  size_t lds_bytes;
};

// Common planning for pack and unpack. `flat` is the 2-D side, `tiled` the
// 4-D side; returns false if the generic kernel has to take the call.
bool make_plan(const uint8_t* flat, const uint8_t* tiled, int64_t flat_stride0, int64_t flat_stride1,
               int64_t tiled_stride0, int64_t size0, int64_t size1, int64_t tsize0, int64_t tsize1,
               int64_t tsize2, int64_t tsize3, bool tr_inner, bool tr_outer, int elem_bytes,
               bool for_unpack, Plan* plan) {
  if (flat_stride1 < 1) return false;  // (0: every element of a row the same one; left to the generic kernel)
  const int l2 = log2_exact(tsize2), l3 = log2_exact(tsize3);
  if (l2 < 0 || l3 < 0) return false;
  const int64_t tile_bytes = tsize2 * tsize3 * elem_bytes;
  if (tile_bytes % 16 || tile_bytes > 16384) return false;
  if ((uintptr_t)tiled % 16 || (tsize0 > 1 && (tiled_stride0 * elem_bytes) % 16)) return false;
  if ((uintptr_t)flat % elem_bytes) return false;
  if (size0 <= 0 || size1 <= 0) return false;  // nothing but padding: generic

  TiledArgs& a = plan->args;
  a.tr_inner = tr_inner;
  a.tr_outer = tr_outer;
  a.log2_s3 = l3;
  a.log2_t0 = tr_inner ? l3 : l2;
  a.log2_t1 = tr_inner ? l2 : l3;
  a.outer0 = tr_outer ? tsize1 : tsize0;
  a.outer1 = tr_outer ? tsize0 : tsize1;
  a.flat_stride0 = flat_stride0;
  a.flat_stride1 = flat_stride1;
  a.tiled_stride0 = tiled_stride0;
  a.size0 = size0;
  a.size1 = size1;
  const int64_t T0 = 1ll << a.log2_t0, T1 = 1ll << a.log2_t1;

  // Block shape: kBlockBytes of the 2-D matrix. Without an outer transpose one
  // tile row (the tiled side is then a single contiguous run); with it, row
  // pieces of 256 bytes to 1 KiB and as many rows as fit (runs grow with rows).
  const int E = elem_bytes;
  int64_t br, bc;
  if (!tr_outer) {
    br = T0;
    bc = kBlockBytes / (br * E);
  } else {
    // 1 KiB row pieces where the tile height allows (measured best of 128 B .. 4 KiB:
    // shorter pieces waste more of their first and last cache line, longer ones
    // shorten the contiguous runs on the tiled side).
    bc = 1024 / E;
    while (bc * E > 256 && kBlockBytes / (bc * E) < T0) bc /= 2;
    // The runs on the tiled side (rows x tile width) must be whole cache lines:
    // with narrow tiles a 16-row block has runs of 16 to 64 bytes, and each
    // 128-byte line is then written in pieces by several blocks (int8 8x2
    // tiles: 1.8 TB/s; with 64 rows x 256 bytes instead 4.7 TB/s). Longer runs
    // than a line at the price of shorter row pieces measured slower again.
    while (bc * E > 128 && (kBlockBytes / (bc * E)) * T1 * E < 128) bc /= 2;
    if (bc < T1) bc = T1;
    br = kBlockBytes / (bc * E);
  }
  if (br < T0 || bc < T1 || br * bc * E != kBlockBytes) return false;
  a.log2_br = log2_exact(br);
  a.log2_bc = log2_exact(bc);

  // 2-D side: 16-byte vectors whatever the alignment of the rows (global memory
  // accesses need none; for loads this is worth up to 1.6x on rows that are
  // only byte aligned, for stores 4-9 % over the widest aligned vector).
  // Elements themselves must be aligned: edges are handled element by element.
  {
    int w = largest_pow2_dividing((uintptr_t)flat, 4);
    if (size0 > 1) {
      const int ws = largest_pow2_dividing((uint64_t)(flat_stride0 * E), 4);
      w = ws < w ? ws : w;
    }
    if (w < E) return false;
  }
  plan->flat_vec_bytes = 16;

  // Contiguous LDS piece on the tiled side.
  int piece = tr_inner ? E : (int)((T1 * E) < 16 ? (T1 * E) : 16);
  plan->piece_bytes = piece;
  plan->elem_bytes = E;

  // Unpack of 4-byte elements into rows that are not whole 128-byte lines apart
  // (or do not start on one): every row's windows are moved to its own line
  // boundaries (tiled_kernel, LINE_ALIGNED).
  // (2-byte elements where the shifts are whole dwords; tiles that divide a thread's stride through the block.)
  const bool dword_shifts = E == 4 || (E == 2 && (uintptr_t)flat % 4 == 0 && (size0 == 1 || (flat_stride0 * E) % 4 == 0));
  plan->line_aligned = for_unpack && dword_shifts && flat_stride1 == 1 && size1 > bc && T0 * T1 * E <= 4096 &&
                       ((uintptr_t)flat % 128 != 0 || (size0 > 1 && (flat_stride0 * E) % 128 != 0));
  a.ext_cols = 0;
  if (plan->line_aligned) a.ext_cols = (int32_t)(T1 > 128 / E ? T1 : 128 / E);
  if (plan->line_aligned && tr_outer && a.ext_cols * br * E / 16 > 512) plan->line_aligned = false, a.ext_cols = 0;
  a.pitch_bytes = choose_pitch(a, E, piece, a.ext_cols);
  a.blocks1 = (int32_t)((size1 + bc - 1) / bc);
  // Blocks must cover every tile of the tiled side, not only the 2-D extent
  // (pack writes whole tiles of padding beyond it).
  const int64_t rows_needed = a.outer0 << a.log2_t0, cols_needed = a.outer1 << a.log2_t1;
  const int64_t blocks0 = (rows_needed + br - 1) / br;
  a.blocks1 = (int32_t)((cols_needed + bc - 1) / bc);
  if (blocks0 * a.blocks1 >= (1ll << 31)) return false;
  a.total_blocks = (int32_t)(blocks0 * a.blocks1);
  // Bytes of one contiguous run on the tiled side when runs are short.
  const int64_t run_bytes = (br / T0) * T0 * T1 * E;
  a.band = !tr_outer ? 1 : (run_bytes <= 128 ? 32 : 16);
  // With an outer transpose the runs of neighbouring tile columns lie tiled_stride0 apart, and a band writes (or
  // reads) the same few KiB of all of them at about the same time. Where that distance is a multiple of 127 or
  // 129 times 4 KiB, these pieces fall on few memory channels (measured: streams 512 KiB -+ 4 KiB, 1 MiB -+ 8 KiB,
  // 1.5 MiB -+ 12 KiB, 2 MiB -+ 16 KiB apart run a quarter slower than at any other distance, as an address hash
  // that folds bits 19.. onto bits 12..18 would have it), and f32 [8256, 8190] with both transposes packed at 0.58
  // of the HBM peak against 0.73-0.76 a few rows either side. A band four times as tall has each column's piece
  // span sixteen channel granules instead of four: 0.73 there. Elsewhere the taller band is 0 to 12 % slower, so it is
  // taken within 2.5 KiB of these distances only, for 4-byte elements (the kernels measured) and four bands or more.
  if (tr_outer && E == 4 && a.band == 16 && blocks0 >= 4 * 64) {
    const int64_t distance = tiled_stride0 * E;
    for (int64_t m = 1; m <= 8 && a.band == 16; ++m)
      for (int64_t granules = 127; granules <= 129; granules += 2)
        if (std::llabs(distance - m * granules * 4096) <= 2560) a.band = 64;
  }
  // Groups of blocks per XCD (linear_block_of): 64 blocks, or one band's.
  {
    const int64_t group = a.band > 1 ? (int64_t)a.band * a.blocks1 : 64;
    const int64_t grouped_slots = a.total_blocks / (8 * group) * group;
    const int64_t rest = a.total_blocks - 8 * grouped_slots;
    a.group = (int32_t)group;
    a.grouped_slots = (int32_t)grouped_slots;
    a.rest_per_xcd = (int32_t)((rest + 7) / 8);
    plan->grid = (unsigned)((grouped_slots + a.rest_per_xcd) * 8);
  }
  plan->lds_bytes = (size_t)br * a.pitch_bytes;
  return plan->lds_bytes <= 49152;
}

// Lane arrangement and LDS skew for pack_transposing_kernel: the combination
// with the fewest bank conflicts among the dword writes of one wavefront
// (32 lanes per pass over 32 banks), found by trying them on the host. The
// search takes about a millisecond, so results are kept per block geometry.
struct TransposingChoice {
  uint32_t key;
  int32_t log2_lpr, log2_period, pad_bytes;
};

void choose_transposing(TiledArgs* a, int elem_bytes, int rq) {
  static std::mutex mutex;
  static std::vector<TransposingChoice> known;
  const uint32_t key = (uint32_t)elem_bytes | (uint32_t)a->log2_t0 << 4 | (uint32_t)a->log2_t1 << 8 |
                       (uint32_t)a->log2_br << 12 | (uint32_t)a->log2_bc << 17 | (uint32_t)a->tr_outer << 22 |
                       (uint32_t)rq << 23;
  std::lock_guard<std::mutex> lock(mutex);
  for (const TransposingChoice& c : known) {
    if (c.key == key) {
      a->log2_lpr = c.log2_lpr; a->log2_period = c.log2_period; a->pad_bytes = c.pad_bytes;
      return;
    }
  }
  const int ve = 16 / elem_bytes;
  const int cq = 4 / (elem_bytes * rq);
  const int log2_cg = a->log2_bc + (elem_bytes == 2 ? 1 : 0) - 4;
  TransposingChoice best{key, 0, 14, 0};
  long best_cost = -1;
  TiledArgs t = *a;
  for (t.log2_lpr = log2_cg < 2 ? log2_cg : 2; t.log2_lpr <= log2_cg; ++t.log2_lpr) {
    for (t.log2_period = 6; t.log2_period <= 14; ++t.log2_period) {
      for (t.pad_bytes = 0; t.pad_bytes <= 64; t.pad_bytes += 16) {
        if (t.log2_period == 14 && t.pad_bytes) break;  // one period: padding changes nothing
        long cost = 0;
        for (int i = 0; i < ve; i += cq) {
          for (int half = 0; half < 2; ++half) {
            int hits[32] = {0};
            int worst = 0;
            for (int lane = 32 * half; lane < 32 * half + 32; ++lane) {
              int32_t row0, col0;
              transposing_unit(t, lane, rq, ve, &row0, &col0);
              const uint32_t addr = skewed(t, (uint32_t)tiled_index_tr_inner(t, row0, col0 + i) * elem_bytes);
              const int h = ++hits[(addr >> 2) & 31];
              worst = h > worst ? h : worst;
            }
            cost += worst;
          }
        }
        // Fewest conflicts; then the longest contiguous stretch of a row per
        // load instruction; then the least padding.
        const long ranked = cost * 1000 - t.log2_lpr * 10 + t.pad_bytes / 16;
        if (best_cost < 0 || ranked < best_cost) {
          best_cost = ranked;
          best.log2_lpr = t.log2_lpr; best.log2_period = t.log2_period; best.pad_bytes = t.pad_bytes;
        }
      }
    }
  }
  known.push_back(best);
  a->log2_lpr = best.log2_lpr; a->log2_period = best.log2_period; a->pad_bytes = best.pad_bytes;
}

// The LDS skew for pack_transposing_wide_kernel: fewest bank conflicts among a
// wavefront's 128-bit writes (8 lanes per pass, 4 of the 32 banks each).
void choose_transposing_wide(TiledArgs* a, int elem_bytes) {
  static std::mutex mutex;
  static std::vector<TransposingChoice> known;
  const uint32_t key = (uint32_t)elem_bytes | (uint32_t)a->log2_t0 << 4 | (uint32_t)a->log2_t1 << 8 |
                       (uint32_t)a->log2_br << 12 | (uint32_t)a->log2_bc << 17 | (uint32_t)a->tr_outer << 22;
  std::lock_guard<std::mutex> lock(mutex);
  for (const TransposingChoice& c : known) {
    if (c.key == key) {
      a->log2_lpr = 0; a->log2_period = c.log2_period; a->pad_bytes = c.pad_bytes;
      return;
    }
  }
  const int rq = 4 / elem_bytes, ve = 16 / elem_bytes;
  TransposingChoice best{key, 0, 14, 0};
  long best_cost = -1;
  TiledArgs t = *a;
  for (t.log2_period = 6; t.log2_period <= 14; ++t.log2_period) {
    for (t.pad_bytes = 0; t.pad_bytes <= 64; t.pad_bytes += 16) {
      if (t.log2_period == 14 && t.pad_bytes) break;
      long cost = 0;
      for (int pass = 0; pass < 8; ++pass) {
        int hits[32] = {0};
        int worst = 0;
        for (int lane = 8 * pass; lane < 8 * pass + 8; ++lane) {
          const int32_t col = (lane & 15) * ve + (lane >> 4) * rq;
          const uint32_t addr = skewed(t, (uint32_t)tiled_index_tr_inner(t, 0, col) * elem_bytes);
          for (int w = 0; w < 4; ++w) {
            const int h = ++hits[((addr >> 2) + w) & 31];
            worst = h > worst ? h : worst;
          }
        }
        cost += worst;
      }
      const long ranked = cost * 1000 + t.pad_bytes / 16;
      if (best_cost < 0 || ranked < best_cost) {
        best_cost = ranked;
        best.log2_period = t.log2_period; best.pad_bytes = t.pad_bytes;
      }
    }
  }
  known.push_back(best);
  a->log2_lpr = 0; a->log2_period = best.log2_period; a->pad_bytes = best.pad_bytes;
}

// Whether one of the transposing kernels takes the planned call (0: no,
// 1: pack_transposing_kernel, 2: pack_transposing_wide_kernel, 3:
// pack_transposing_kernel for int8 tiles two rows tall); sets it up.
int plan_transposing(Plan* p) {
  TiledArgs& a = p->args;
  const int E = p->elem_bytes;
  if (!a.tr_inner || E > 2 || p->flat_vec_bytes != 16 || a.flat_stride1 != 1) return 0;
  const int log2_e = E == 2 ? 1 : 0;
  const int log2_rq = 2 - log2_e, log2_ve = 4 - log2_e;
  if (a.log2_bc + log2_e < 4) return 0;
  if (E == 1 && a.log2_t0 == 1 && a.log2_t1 >= 1 && a.log2_br >= 1) {
    choose_transposing(&a, E, 2);
    p->lds_bytes = skewed(a, kBlockBytes - 16) + 16;
    return 3;
  }
  if (a.log2_t0 < log2_rq) return 0;
  int which = 1;
  if (a.log2_t0 >= log2_ve && a.log2_bc + log2_e >= 8 && a.log2_br >= log2_ve) {
    which = 2;
    choose_transposing_wide(&a, E);
  } else {
    choose_transposing(&a, E, 4 / E);
  }
  p->lds_bytes = skewed(a, kBlockBytes - 16) + 16;
  return which;
}

// Workgroups resident per compute unit, for 4-byte elements and more than 128 MiB per side. A block's LDS image
// is 16 to 20 KiB and its four wavefronts let eight workgroups share a unit; with LDS asked for as if the image
// were 32 KiB, five do, and large f32 matrices move faster: [8191, 8190] with 16x1 tiles pack 6.04 -> 6.17 TB/s, with
// both transposes 5.74 -> 5.83 (six or four workgroups: in between; three or two: 5.0-5.8), unpack 6.06 -> 6.17. Over
// tiles 16x1, 8x8, 16x16, the four transpose combinations and [2048, 16384] ... [1024, 65536], buffers rotated
// so that the last-level cache does not hold them: pack -3 to +8 %, unpack -6 to +12 %, about +2 % in the mean for
// both. Not for 1- and 2-byte elements (-1 to -19 %) and not for matrices the last-level cache holds (4096^2:
// -1 to -5 %, 3000^2: -2 to -8 %).
void limit_resident_blocks(Plan* p) {
  constexpr size_t kLdsAskedFor = 32 * 1024;
  if (p->elem_bytes == 4 && p->args.total_blocks >= 8192 && p->lds_bytes < kLdsAskedFor) p->lds_bytes = kLdsAskedFor;
}

template <int E, int W, bool UNPACK>
hipError_t launch_pw(const Plan& p, hipStream_t stream) {
  const dim3 grid(p.grid), block(256);
  switch (p.piece_bytes) {
#define UK_PIECE(PB)                                                                         \
  case PB:                                                                                   \
    if constexpr (PB >= E) {                                                                 \
      hipLaunchKernelGGL((tiled_kernel<E, W, PB, UNPACK>), grid, block, p.lds_bytes, stream, \
                         p.args);                                                            \
      return hipGetLastError();                                                              \
    }                                                                                        \
    return hipErrorInvalidValue
    UK_PIECE(16);
    UK_PIECE(8);
    UK_PIECE(4);
    UK_PIECE(2);
    UK_PIECE(1);
#undef UK_PIECE
    default:
      return hipErrorInvalidValue;
  }
}

template <int E, bool UNPACK>
hipError_t launch_e(const Plan& p, hipStream_t stream) {
  if (p.flat_vec_bytes != 16) return hipErrorInvalidValue;
  return launch_pw<E, 16, UNPACK>(p, stream);
}

template <bool UNPACK>
hipError_t launch_plan(const Plan& p, hipStream_t stream) {
  switch (p.elem_bytes) {
    case 1: return launch_e<1, UNPACK>(p, stream);
    case 2: return launch_e<2, UNPACK>(p, stream);
    case 4: return launch_e<4, UNPACK>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t launch_pack(const PackArgs& original, hipStream_t stream, const char** name) {
  Plan plan;
  PackArgs a = original;
  bool tr_inner = a.flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER;
  const bool tr_outer = a.flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER;
  // Tiles one column wide are consecutive rows of that column whichever way the
  // inner dimensions are ordered; and int8 tiles two columns wide are tiles one
  // column wide of 2-byte elements when everything else is even. Both are put
  // in the inner-transposed form, which for 1- and 2-byte elements has the
  // register-transposing kernels (int8 [M1][K1][16][2] lhs layouts: 4.8 ->
  // 5.5 TB/s).
  if (!tr_inner && a.elem_bytes == 1 && a.out_size3 == 2 && a.in_stride1 == 1 && a.in_size1 % 2 == 0 &&
      a.in_stride0 % 2 == 0 && a.out_stride0 % 2 == 0 && (uintptr_t)a.in % 2 == 0) {
    a.elem_bytes = 2;
    a.in_size1 /= 2;
    a.in_stride0 /= 2;
    a.out_stride0 /= 2;
    a.out_size3 = 1;
    a.padding_value = (a.padding_value & 0xFF) * 0x0101u;
  }
  if (!tr_inner && a.out_size3 == 1 && a.elem_bytes <= 2) {
    a.out_size3 = a.out_size2;
    a.out_size2 = 1;
    tr_inner = true;
  }
  // The other way round: a tile one ROW tall stored inner-transposed ([T1][1])
  // is that row's T1 consecutive elements, i.e. the untransposed [1][T1]; as
  // such its 16-byte vectors are whole pieces of a row in LDS instead of
  // separate elements (int8 [16383, 16382] into 1x16 tiles: 3.6 -> 5.4 TB/s).
  if (tr_inner && a.out_size3 == 1) {
    a.out_size3 = a.out_size2;
    a.out_size2 = 1;
    tr_inner = false;
  }
  // Tiles of 8 bytes with a unit dimension (int8 8x1, the Arm tiles for K0 = 1,
  // arch/arm_64/pack_arm_64_entry_point.c:24-26): the vectors of the tiled side
  // are 16 bytes, i.e. two tiles that follow each other along out dimension 1,
  // and two such tiles are one 16-byte tile: [1][n] twice along the direction
  // of n is [1][2n]; along the other direction it is [2][n]. With an odd
  // number of tiles along that dimension the last one is left to the generic
  // kernel (a slice of the source and one column of tiles).
  PackArgs last_tiles;
  bool have_last_tiles = false;
  if (a.out_size2 * a.out_size3 * a.elem_bytes == 8 && (a.out_size2 == 1 || a.out_size3 == 1) &&
      a.out_size1 >= 2 && a.in_stride1 == 1) {
    if (a.out_size3 == 1) {  // [n][1] is [1][n] with the other inner order
      a.out_size3 = a.out_size2;
      a.out_size2 = 1;
      tr_inner = !tr_inner;
    }
    const int merge_dim = tr_outer ? 0 : 1;   // source dimension that out dimension 1 walks along
    const int long_dim = tr_inner ? 0 : 1;    // source dimension of the tile's n elements
    const int64_t tile_extent = merge_dim == long_dim ? a.out_size3 : 1;
    if (a.out_size1 & 1) {
      const int64_t start = (a.out_size1 - 1) * tile_extent;  // first source coordinate of the last tiles
      int64_t& size_along = merge_dim == 0 ? a.in_size0 : a.in_size1;
      last_tiles = a;
      last_tiles.flags = (a.flags & ~(uint32_t)IREE_UK_FLAG_PACK_TRANSPOSE_INNER) |
                         (tr_inner ? IREE_UK_FLAG_PACK_TRANSPOSE_INNER : 0u);
      last_tiles.in = a.in + start * (merge_dim == 0 ? a.in_stride0 : a.in_stride1) * a.elem_bytes;
      (merge_dim == 0 ? last_tiles.in_size0 : last_tiles.in_size1) = size_along > start ? size_along - start : 0;
      last_tiles.out = a.out + (a.out_size1 - 1) * 8;
      last_tiles.out_size1 = 1;
      have_last_tiles = true;
      size_along = size_along < start ? size_along : start;
      a.out_size1 -= 1;
    }
    a.out_size1 /= 2;
    if (merge_dim == long_dim) a.out_size3 *= 2; else a.out_size2 = 2;
  }
  if (!make_plan(a.in, a.out, a.in_stride0, a.in_stride1, a.out_stride0, a.in_size0, a.in_size1,
                 a.out_size0, a.out_size1, a.out_size2, a.out_size3, tr_inner, tr_outer,
                 a.elem_bytes, /*for_unpack=*/false, &plan))
    return launch_pack_generic(original, stream, name);
  if (have_last_tiles) {
    const hipError_t e = launch_pack_generic(last_tiles, stream, name);
    if (e != hipSuccess) return e;
  }
  plan.args.src = a.in;
  plan.args.dst = a.out;
  plan.args.padding_value = a.padding_value;
  const int which = plan_transposing(&plan);
  limit_resident_blocks(&plan);
  if (which) {
    *name = "pack_transposing";
    const dim3 grid(plan.grid), block(256);
    if (which == 2 && plan.elem_bytes == 1) {
      hipLaunchKernelGGL(pack_transposing_wide_kernel<1>, grid, block, plan.lds_bytes, stream, plan.args);
    } else if (which == 2) {
      hipLaunchKernelGGL(pack_transposing_wide_kernel<2>, grid, block, plan.lds_bytes, stream, plan.args);
    } else if (which == 3) {
      hipLaunchKernelGGL((pack_transposing_kernel<1, 2>), grid, block, plan.lds_bytes, stream, plan.args);
    } else if (plan.elem_bytes == 1) {
      hipLaunchKernelGGL((pack_transposing_kernel<1, 4>), grid, block, plan.lds_bytes, stream, plan.args);
    } else {
      hipLaunchKernelGGL((pack_transposing_kernel<2, 2>), grid, block, plan.lds_bytes, stream, plan.args);
    }
    return hipGetLastError();
  }
  *name = "pack_tiled";
  return launch_plan<false>(plan, stream);
}

hipError_t launch_unpack(const UnpackArgs& original, hipStream_t stream, const char** name) {
  Plan plan;
  UnpackArgs a = original;
  bool tr_inner = a.flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER;
  const bool tr_outer = a.flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER;
  // A tile one row tall stored inner-transposed is the untransposed [1][T1]
  // (see launch_pack).
  if (tr_inner && a.in_size3 == 1) {
    a.in_size3 = a.in_size2;
    a.in_size2 = 1;
    tr_inner = false;
  }
  if (!make_plan(a.out, a.in, a.out_stride0, a.out_stride1, a.in_stride0, a.out_size0, a.out_size1,
                 a.in_size0, a.in_size1, a.in_size2, a.in_size3, tr_inner, tr_outer, a.elem_bytes,
                 /*for_unpack=*/true, &plan))
    return launch_unpack_generic(original, stream, name);
  plan.args.src = a.in;
  plan.args.dst = a.out;
  plan.args.padding_value = 0;
  limit_resident_blocks(&plan);
  *name = "unpack_tiled";
  if (plan.line_aligned) {
    const dim3 grid(plan.grid), block(256);
    void (*kernel)(const TiledArgs) = nullptr;
#define UK_LINE_ALIGNED_KERNEL(E, MODE)                                                                        \
  (plan.piece_bytes == 16 ? tiled_kernel<E, 16, 16, true, MODE>                                                 \
   : plan.piece_bytes == 8 ? tiled_kernel<E, 16, 8, true, MODE>                                                 \
   : (plan.piece_bytes == 4 || E == 4) ? tiled_kernel<E, 16, 4, true, MODE> : tiled_kernel<E, 16, E, true, MODE>)
    if (plan.elem_bytes == 4) kernel = tr_outer ? UK_LINE_ALIGNED_KERNEL(4, 2) : UK_LINE_ALIGNED_KERNEL(4, 1);
    else kernel = tr_outer ? UK_LINE_ALIGNED_KERNEL(2, 2) : UK_LINE_ALIGNED_KERNEL(2, 1);
#undef UK_LINE_ALIGNED_KERNEL
    hipLaunchKernelGGL(kernel, grid, block, plan.lds_bytes, stream, plan.args);
    return hipGetLastError();
  }
  return launch_plan<true>(plan, stream);
}

}  // namespace uk
