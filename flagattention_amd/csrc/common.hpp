// Shared pieces of the attention kernels: launch helper, tile movers and MFMA operand readers.
//
// Conventions used by every kernel in this directory
//   * tensors are (batch, head, token, D) views with unit stride on D; strides are in elements;
//   * a "tile" is a row-major patch of tokens x D held in LDS with a padded row stride (LD);
//   * one wavefront multiplies 32x32 blocks with mfma32 (hw.hpp); its lane l owns column l % 32 of a
//     block and the half h = l / 32 selects which rows / which 8 of the 16 contraction indices.
#pragma once
#include "hw.hpp"

namespace fa {

using hw::u32x4;
using hw::f32x16;
using hw::short4v;

constexpr int kThreads = 256;  // 4 wavefronts per workgroup
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

FA_DEVICE int cdiv(int a, int b) { return (a + b - 1) / b; }
FA_DEVICE int imin(int a, int b) { return a < b ? a : b; }
FA_DEVICE int imax(int a, int b) { return a > b ? a : b; }
FA_DEVICE float neg_inf() { return -__builtin_inff(); }

// ---------------------------------------------------------------------------------------------
// global -> registers -> LDS movement of a ROWS x COLS tile (16 bytes per thread per step)
// ---------------------------------------------------------------------------------------------
template <int ROWS, int COLS>
struct TileRegs {
  static constexpr int kChunks = ROWS * COLS / 8;
  static constexpr int kPerThread = (kChunks + kThreads - 1) / kThreads;
  u32x4 r[kPerThread];
};

// Rows at or beyond `row_limit` are filled with zeros (a masked probability times a stray NaN
// would otherwise poison the accumulators).
template <class T, int ROWS, int COLS>
FA_DEVICE void tile_fetch(TileRegs<ROWS, COLS>& t, const T* base, int64_t row_stride, int row0,
                          int row_limit, int tid) {
  constexpr int kCPR = COLS / 8;  // 16-byte chunks per row
#pragma unroll
  for (int i = 0; i < TileRegs<ROWS, COLS>::kPerThread; ++i) {
    int c = tid + i * kThreads;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (c < TileRegs<ROWS, COLS>::kChunks) {
      int r = c / kCPR, col = (c % kCPR) * 8;
      if (row0 + r < row_limit) v = *(const u32x4*)(base + (int64_t)(row0 + r) * row_stride + col);
    }
    t.r[i] = v;
  }
}

template <class T, int ROWS, int COLS, int LD>
FA_DEVICE void tile_commit(const TileRegs<ROWS, COLS>& t, T* lds_tile, int tid) {
  constexpr int kCPR = COLS / 8;
#pragma unroll
  for (int i = 0; i < TileRegs<ROWS, COLS>::kPerThread; ++i) {
    int c = tid + i * kThreads;
    if (c < TileRegs<ROWS, COLS>::kChunks) {
      int r = c / kCPR, col = (c % kCPR) * 8;
      *(u32x4*)(lds_tile + r * LD + col) = t.r[i];
    }
  }
}

// Loop-invariant plan of one thread's share of a ROWS x COLS tile: byte offsets inside the global
// tile are computed once, so that a steady-state fetch is one load per chunk from a uniform tile
// base plus a 32-bit lane offset, and the LDS destination is a fixed offset from the tile start.
template <class T, int ROWS, int COLS>
struct TileMover {
  static constexpr int CPR = COLS / 8;          // 16-byte chunks per row
  static constexpr int RPP = kThreads / CPR;    // rows covered by one pass of the workgroup
  static constexpr int PASSES = (ROWS + RPP - 1) / RPP;
  static constexpr bool kExact = (PASSES * RPP == ROWS);
  u32x4 r[PASSES];
  uint32_t goff[PASSES];
  int row0, col0;

  FA_DEVICE void init(int tid, int64_t row_stride) {
    row0 = tid / CPR;
    col0 = (tid % CPR) * 8;
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      goff[i] = (uint32_t)(((int64_t)(row0 + i * RPP) * row_stride + col0) * (int64_t)sizeof(T));
  }
  // every row of the tile exists
  FA_DEVICE void fetch_full(const T* tile_base) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (kExact || row0 + i * RPP < ROWS) v = *(const u32x4*)((const char*)tile_base + goff[i]);
      r[i] = v;
    }
  }
  // only the first rows_valid rows exist; the rest is filled with zeros
  FA_DEVICE void fetch_rows(const T* tile_base, int rows_valid) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      u32x4 v = {0u, 0u, 0u, 0u};
      const int row = row0 + i * RPP;
      if ((kExact || row < ROWS) && row < rows_valid) v = *(const u32x4*)((const char*)tile_base + goff[i]);
      r[i] = v;
    }
  }
  FA_DEVICE void fetch(const T* tile_base, int rows_valid) {
    if (rows_valid >= ROWS) fetch_full(tile_base); else fetch_rows(tile_base, rows_valid);
  }
  template <int LD>
  FA_DEVICE void commit(T* lds_tile) const {
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      if (kExact || row0 + i * RPP < ROWS) *(u32x4*)(lds_tile + (row0 + i * RPP) * LD + col0) = r[i];
  }
};

// ---------------------------------------------------------------------------------------------
// MFMA operand readers
// ---------------------------------------------------------------------------------------------
// Operand whose contraction index runs along D: element (row = row0 + l % 32, k = k0 + 8h + 0..7)
// of a row-major tile, one 16-byte LDS read.
template <class T, int LD>
FA_DEVICE typename hw::Elem<T>::v8 operand_rowmajor(const T* lds_tile, int row0, int k0, int lane) {
  const T* p = lds_tile + (row0 + (lane & 31)) * LD + k0 + 8 * (lane >> 5);
  return hw::as_v8<T>(*(const u32x4*)p);
}

// Operand whose contraction index runs along the tile's rows (tokens) and whose free index runs
// along D: the lane needs, for column c0 + l % 32, the 8 rows
//     t0 + 4h + {0,1,2,3}  and  t0 + 8 + 4h + {0,1,2,3}
// which is exactly the order in which an mfma32 result holds rows 0..15 of a block (registers
// 0..7) -- so a 16-row slice of a result block can be multiplied against this operand directly.
// Two transposing reads fetch them from the row-major tile.
template <class T, int LD>
FA_DEVICE typename hw::Elem<T>::v8 operand_transposed(const T* lds_tile, int t0, int c0, int lane) {
  int i = lane & 15, dhalf = (lane >> 4) & 1, h = lane >> 5;
  const T* p = lds_tile + (t0 + 4 * h + (i >> 2)) * LD + c0 + 16 * dhalf + 4 * (i & 3);
  short4v lo = hw::lds_read_tr16(p);
  short4v hi = hw::lds_read_tr16(p + 8 * LD);
  return hw::join_v8<T>(lo, hi);
}

// Work distribution of the tiled kernels: a 1-D grid of (tile rank) x (batch * head) workgroups with
// the (batch, head) index running fastest.  Workgroups are dispatched in id order, so ranking tiles
// from most to least work puts every head's longest tiles first and leaves the shortest for the
// tail (balanced finish under the causal mask); and because consecutive ids go to consecutive XCDs,
// a given (batch, head) -- whose K/V or Q/dO every one of its tiles re-reads -- stays on one XCD's
// L2 whenever batch * heads is a multiple of the XCD count.
struct TileId { int rank, head, batch; };
FA_DEVICE TileId tile_of_workgroup(int H, int B) {
  const int lin = hw::block_x(), bh = lin % (H * B);
  TileId t;
  t.rank = lin / (H * B);
  t.head = bh % H;
  t.batch = bh / H;
  return t;
}

// Row index inside a 32-row result block of register r for the lane's half h.
FA_DEVICE int block_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// Packs registers 8c..8c+7 of a result block into an operand (rounded to T).
template <class T>
FA_DEVICE typename hw::Elem<T>::v8 pack_half_block(const f32x16& s, int c) {
  typename hw::Elem<T>::v8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (T)s[8 * c + e];
  return v;
}

// ---------------------------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------------------------
#ifdef FLAGATTN_HOST_SIM
template <class P>
int launch(void (*kern)(P), dim3 grid, size_t lds_bytes, hipStream_t, const P& p) {
  hwsim::run_grid(grid, kThreads, lds_bytes, [&]() { kern(p); });
  return 0;
}
#else
template <class P>
int launch(void (*kern)(P), dim3 grid, size_t lds_bytes, hipStream_t stream, const P& p) {
  if (lds_bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, stream, p);
  return (int)hipGetLastError();
}
#endif

// error codes of the C entry points (positive values are hipError_t)
constexpr int kOk = 0;
constexpr int kBadArgument = -1;
constexpr int kUnsupported = -2;

constexpr int kDtypeF16 = 0;
constexpr int kDtypeBF16 = 1;

}  // namespace fa
