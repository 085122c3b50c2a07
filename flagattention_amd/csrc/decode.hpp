// Core of the decode-shaped kernels (few query rows against a long key/value stream): dense split-KV
// flash decoding and paged attention share it.  These kernels are bound by HBM bandwidth, so the
// structure is built around keeping many 16-byte loads in flight rather than around MFMA occupancy:
//
//   * a workgroup serves up to 32 query rows that share one key/value head (all query heads of a
//     GQA group, times the few query positions), so K and V are read once per kv head;
//   * each of its 4 wavefronts walks its own interleaved sequence of 32-key steps with no workgroup
//     barrier inside the loop: coalesced 16-byte global loads into registers, a private LDS patch to
//     re-layout them, S^T = K Q^T and O^T += V^T P^T on the MFMA (one query row per lane), and the
//     next step's global loads are issued before the current step's arithmetic;
//   * at the end the 4 wavefronts merge their (max, sum, O) triples through LDS.
#pragma once
#include "common.hpp"

namespace fa {

template <class T, int D>
struct DecCfg {
  static constexpr int TK = 32;  // keys per wavefront step
  static constexpr int DV = D < 32 ? 32 : D;
  static constexpr int KSTEPS = D / 16;
  static constexpr int CPR = D / 8;               // 16-byte chunks per row
  static constexpr int CH = (TK * CPR + 63) / 64;  // chunks per lane per tile
  static constexpr int K_LD = D + 8;
  static constexpr int V_LD = DV + 32;
  static constexpr int WAVE_ELEMS = TK * K_LD + TK * V_LD;
  static constexpr size_t STAGING_BYTES = 4 * WAVE_ELEMS * sizeof(T);
  // merge area: per wavefront 32 rows x (DV + 2) floats
  static constexpr size_t MERGE_BYTES = 4 * 32 * (DV + 2) * sizeof(float);
  static constexpr size_t LDS_BYTES = STAGING_BYTES > MERGE_BYTES ? STAGING_BYTES : MERGE_BYTES;
};

// Result of the per-workgroup pass, valid in every thread after decode_block():
// thread t owns output elements (row = idx / DV, d = idx % DV) for idx = t, t + 256, ...
template <int DV>
struct DecodeOut {
  static constexpr int kPerThread = 32 * DV / kThreads;
  float o[kPerThread];     // un-normalised sum_j p_j v_j, relative to row_max
  float row_max[kPerThread];  // running maximum of the raw (unscaled) scores, -inf if no key seen
  float row_sum[kPerThread];  // sum_j exp(scale * (s_j - row_max))
};

// Src must provide:
//   struct Ids;                                  per-lane lookup state for one tile
//   void lookup(Ids&, int n0, int lane) const;   start resolving rows of the tile at key n0
//   const T* k_row(const Ids&, int i, int n) const;   row pointer of key n (chunk slot i of the lane)
//   const T* v_row(const Ids&, int i, int n) const;
template <class T, int D, class Src>
FA_DEVICE void decode_block(const Src& src, const T* q_row /* this lane's query row or nullptr */,
                            int n_begin, int n_end, int lane_limit /* keys n < lane_limit are visible */,
                            float c2, unsigned char* smem, DecodeOut<DecCfg<T, D>::DV>& out) {
  using C = DecCfg<T, D>;
  using V8 = typename hw::Elem<T>::v8;
  const int tid = hw::thread_id(), lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  T* sK = (T*)smem + wave * C::WAVE_ELEMS;
  T* sV = sK + C::TK * C::K_LD;

  V8 qreg[C::KSTEPS];
#pragma unroll
  for (int kk = 0; kk < C::KSTEPS; ++kk) {
    u32x4 z = {0u, 0u, 0u, 0u};
    if (q_row) z = *(const u32x4*)(q_row + 16 * kk + 8 * hh);
    qreg[kk] = hw::as_v8<T>(z);
  }

  if (C::DV != D) {  // columns D..DV-1 of the value patch are never written by loads
    for (int i = lane; i < C::TK * C::V_LD; i += 64) sV[i] = (T)0.f;
  }

  const int limit = imin(lane_limit, n_end);
  float m_i = neg_inf(), l_i = 0.f;
  f32x16 oacc[C::DV / 32];
#pragma unroll
  for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;

  const int total_tiles = n_end > n_begin ? cdiv(n_end - n_begin, C::TK) : 0;
  const int my_tiles = total_tiles > wave ? (total_tiles - wave + 3) / 4 : 0;
  auto tile_start = [&](int j) { return n_begin + (wave + 4 * j) * C::TK; };

  u32x4 kst[C::CH], vst[C::CH];
  typename Src::Ids ids;
  auto fetch = [&](int n0) {
#pragma unroll
    for (int i = 0; i < C::CH; ++i) {
      const int c = lane + 64 * i;
      const int row = c / C::CPR, col = (c % C::CPR) * 8;
      const int n = n0 + row;
      u32x4 a = {0u, 0u, 0u, 0u}, b = a;
      if (row < C::TK && n < n_end) {
        a = *(const u32x4*)(src.k_row(ids, i, n) + col);
        b = *(const u32x4*)(src.v_row(ids, i, n) + col);
      }
      kst[i] = a;
      vst[i] = b;
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < C::CH; ++i) {
      const int c = lane + 64 * i;
      const int row = c / C::CPR, col = (c % C::CPR) * 8;
      if (row < C::TK) {
        *(u32x4*)(sK + row * C::K_LD + col) = kst[i];
        *(u32x4*)(sV + row * C::V_LD + col) = vst[i];
      }
    }
  };

  if (my_tiles > 0) {
    src.lookup(ids, tile_start(0), n_end, lane);
    fetch(tile_start(0));
    if (my_tiles > 1) src.lookup(ids, tile_start(1), n_end, lane);
  }

  for (int j = 0; j < my_tiles; ++j) {
    const int n0 = tile_start(j);
    hw::wave_sync();
    commit();
    if (j + 1 < my_tiles) {
      fetch(tile_start(j + 1));
      if (j + 2 < my_tiles) src.lookup(ids, tile_start(j + 2), n_end, lane);
    }
    hw::wave_sync();

    f32x16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk)
      s = hw::mfma32(operand_rowmajor<T, C::K_LD>(sK, 0, 16 * kk, lane), qreg[kk], s);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int n = n0 + block_row(r, hh);
      s[r] = (n < limit) ? s[r] : neg_inf();
    }
    float mx = neg_inf();
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
    mx = fmaxf(mx, hw::xor32(mx));
    const float m_new = fmaxf(m_i, mx);
    const float m_use = (m_new == neg_inf()) ? 0.f : m_new;
    const float alpha = hw::exp2_fast((m_i - m_use) * c2);
    const float shift = -m_use * c2;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float e = hw::exp2_fast(fmaf(s[r], c2, shift));
      s[r] = e;
      psum += e;
    }
    l_i = l_i * alpha + psum;
    m_i = m_new;
#pragma unroll
    for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      V8 pb = pack_half_block<T>(s, c);
#pragma unroll
      for (int db = 0; db < C::DV / 32; ++db)
        oacc[db] = hw::mfma32(operand_transposed<T, C::V_LD>(sV, 16 * c, db * 32, lane), pb, oacc[db]);
    }
  }

  // ---- merge the 4 wavefronts: area[w][row][0..DV-1] = O, [DV] = max, [DV+1] = sum ----
  l_i += hw::xor32(l_i);
  hw::block_sync();  // every wavefront is done with its staging patch
  float* area = (float*)smem;
  constexpr int RS = C::DV + 2;
  {
    float* mine = area + (wave * 32 + l32) * RS;
#pragma unroll
    for (int db = 0; db < C::DV / 32; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) mine[db * 32 + block_row(r, hh)] = oacc[db][r];
    if (hh == 0) { mine[C::DV] = m_i; mine[C::DV + 1] = l_i; }
  }
  hw::block_sync();
#pragma unroll
  for (int e = 0; e < DecodeOut<C::DV>::kPerThread; ++e) {
    const int idx = tid + e * kThreads;
    const int row = idx / C::DV, d = idx % C::DV;
    float mw[4], mm = neg_inf();
#pragma unroll
    for (int w = 0; w < 4; ++w) { mw[w] = area[(w * 32 + row) * RS + C::DV]; mm = fmaxf(mm, mw[w]); }
    const float m_use = (mm == neg_inf()) ? 0.f : mm;
    float acc = 0.f, sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = hw::exp2_fast((mw[w] - m_use) * c2);  // -inf -> 0
      acc += f * area[(w * 32 + row) * RS + d];
      sum += f * area[(w * 32 + row) * RS + C::DV + 1];
    }
    out.o[e] = acc;
    out.row_max[e] = mm;
    out.row_sum[e] = sum;
  }
}

}  // namespace fa
