// Shared pieces of the attention kernels: launch helper, tile movers and MFMA operand readers.
//
// Conventions used by every kernel in this directory
//   * tensors are (batch, head, token, D) views with unit stride on D; strides are in elements;
//   * a "tile" is a row-major patch of tokens x D held in LDS with a padded row stride (LD);
//   * one wavefront multiplies 32x32 blocks with mfma32 (hw.hpp); its lane l owns column l % 32 of a
//     block and the half h = l / 32 selects which rows / which 8 of the 16 contraction indices.
#pragma once
#include <atomic>
#include <mutex>
#include <type_traits>
#include <unordered_map>
#include <utility>

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
// Loop-invariant plan of one thread's share of a ROWS x COLS tile: byte offsets inside the global
// tile are computed once, so that a steady-state fetch is one load per chunk from a uniform tile
// base plus a 32-bit lane offset, and the LDS destination is a fixed offset from the tile start.
//
// fetch() is branch-free on purpose.  With a branch per load (or per tile kind) the compiler puts
// loads in separate basic blocks and waits for ALL outstanding loads at their boundaries -- a full
// memory latency per tile.  Rows that do not exist are therefore read from the last row that does
// (always valid memory) and replaced by zeros when the tile is committed to LDS.
template <class T, int ROWS, int COLS>
struct TileMover {
  static constexpr int CPR = COLS / 8;          // 16-byte chunks per row
  static constexpr int RPP = kThreads / CPR;    // rows covered by one pass of the workgroup
  static constexpr int PASSES = (ROWS + RPP - 1) / RPP;
  static constexpr bool kExact = (PASSES * RPP == ROWS);
  u32x4 r[PASSES];
  uint32_t goff[PASSES];
  uint32_t stride_bytes, col_bytes;
  int row0, col0;
  int valid;  // rows of the fetched tile that exist
  uint32_t last_off;

  FA_DEVICE void init(int tid, int64_t row_stride) {
    row0 = tid / CPR;
    col0 = (tid % CPR) * 8;
    stride_bytes = (uint32_t)(row_stride * (int64_t)sizeof(T));
    col_bytes = (uint32_t)(col0 * (int)sizeof(T));
    valid = ROWS;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) goff[i] = (uint32_t)(row0 + i * RPP) * stride_bytes + col_bytes;
  }
  // rows_valid >= 1 rows of the tile exist; rows past them load a copy of the last one
  FA_DEVICE void fetch(const T* tile_base, int rows_valid) {
    fetch_begin(rows_valid);
#pragma unroll
    for (int i = 0; i < PASSES; ++i) fetch_pass(tile_base, i);
  }
  // the same in pieces, for callers that place the loads themselves
  FA_DEVICE void fetch_begin(int rows_valid) {
    valid = rows_valid < ROWS ? rows_valid : ROWS;
    last_off = (uint32_t)(valid - 1) * stride_bytes + col_bytes;
  }
  FA_DEVICE void fetch_pass(const T* tile_base, int i) {
    const uint32_t off = (row0 + i * RPP < valid) ? goff[i] : last_off;
    r[i] = *(const u32x4*)((const char*)tile_base + off);
  }
  // one pass of commit(), without the zeroes for rows past the end: those keep the copies of the
  // last row that fetch() loaded
  template <int LD>
  FA_DEVICE void commit_pass(T* lds_tile, int i) const {
    static_assert(kExact, "whole passes only");
    *(u32x4*)(lds_tile + (row0 + i * RPP) * LD + col0) = r[i];
  }
  template <int LD>
  FA_DEVICE void commit(T* lds_tile) {
    if (valid < ROWS) {  // tail tile only (uniform): rows past the end become zeros
      hw::keep_branch();
#pragma unroll
      for (int i = 0; i < PASSES; ++i)
        if (row0 + i * RPP >= valid) r[i] = u32x4{0u, 0u, 0u, 0u};
    }
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
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order: a loop whose index is a
// constant expression inside the body
template <int... I, class F>
FA_DEVICE void static_for_each(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
FA_DEVICE void static_for(F&& f) {
  static_for_each(std::make_integer_sequence<int, N>{}, f);
}

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
// dropout mask
// ---------------------------------------------------------------------------------------------
// The reference draws one number per score element with Triton's tl.rand(seed, offs, n_rounds=6)
// (src/flag_attn/flash.py:367-371, 454-457): Philox-4x32 with counter (lo(c), hi(c), 0, 0),
// c = offset + ((b * H + h) * M + m) * N + n, key (lo(seed), hi(seed)), 6 rounds, first output word;
// the word, read as int32 with negative values folded by -x - 1, times 4.6566127342e-10 is the
// uniform number, and the probability is kept when it exceeds dropout_p.
FA_DEVICE uint32_t philox6_first_word(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1) {
  uint32_t c2 = 0u, c3 = 0u;
#pragma unroll
  for (int round = 0; round < 6; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}
FA_DEVICE bool dropout_keeps(uint64_t counter, uint64_t seed, float dropout_p) {
  const uint32_t x = philox6_first_word((uint32_t)counter, (uint32_t)(counter >> 32), (uint32_t)seed,
                                        (uint32_t)(seed >> 32));
  int32_t v = (int32_t)x;
  v = v < 0 ? ~v : v;  // -v - 1
  return (float)v * 4.6566127342e-10f > dropout_p;
}

// ---------------------------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------------------------
constexpr int kMaxDevices = 64;   // devices whose per-device facts are remembered

// A kernel that needs more than 48 KB of LDS has to be given the limit before its first launch, once per
// device (the attribute belongs to the device's copy of the function).  The runtime call costs about as
// much as a launch, so the devices on which it has been made are remembered per kernel.
template <class P>
int allow_lds(void (*kern)(P), size_t lds_bytes) {
  static std::mutex lock;
  static std::unordered_map<const void*, uint64_t> done;   // kernel -> bit per device
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) dev = kMaxDevices;
  const uint64_t bit = dev < kMaxDevices ? (uint64_t)1 << dev : 0;
  if (bit) {
    std::lock_guard<std::mutex> g(lock);
    auto it = done.find((const void*)kern);
    if (it != done.end() && (it->second & bit)) return 0;
  }
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return (int)e;
  if (bit) {
    std::lock_guard<std::mutex> g(lock);
    done[(const void*)kern] |= bit;
  }
  return 0;
}

template <class P>
int launch(void (*kern)(P), dim3 grid, size_t lds_bytes, hipStream_t stream, const P& p) {
  if (lds_bytes > 48 * 1024) {
    const int rc = allow_lds(kern, lds_bytes);
    if (rc) return rc;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, stream, p);
  return (int)hipGetLastError();
}

// error codes of the C entry points (positive values are hipError_t)
constexpr int kOk = 0;
constexpr int kBadArgument = -1;
constexpr int kUnsupported = -2;

constexpr int kDtypeF16 = 0;
constexpr int kDtypeBF16 = 1;

}  // namespace fa
