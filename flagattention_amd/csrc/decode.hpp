// Core of the decode-shaped kernels (few query rows against a long key/value stream): dense split-KV
// flash decoding and paged attention share it.  These kernels are bound by HBM bandwidth, so the
// structure is built around keeping many 16-byte loads in flight rather than around MFMA occupancy:
//
//   * a workgroup serves up to 16 query rows that share one key/value head (all query heads of a
//     GQA group, times the few query positions), so K and V are read once per kv head;
//   * the products use the 16x16x32 MFMA: with 16 query rows the output accumulator O^T (D x 16)
//     needs D/4 registers and the scores of a 32-key step 8, which leaves room for a register set
//     of key/value loads -- while one 32-key step is computed the loads of the next one are in
//     flight (NSETS = 1: 16 KB per wavefront at D = 128, 128 KB per CU with two wavefronts per
//     SIMD; the code also carries a second set, NSETS = 2, which is not switched on);
//   * each of the 4 wavefronts walks its own interleaved sequence of 32-key steps with no workgroup
//     barrier inside the loop: coalesced 16-byte global loads into registers, a private LDS patch to
//     re-layout them, S^T = K Q^T (keys x queries, one query row per lane of each 16-lane group) and
//     O^T += V^T P^T with V read through the transposing LDS read;
//   * at the end the 4 wavefronts merge their (max, sum, O) triples through LDS.
//
// Layouts of mfma16 (hw.hpp): lane l = 16 g + i.  A operand: row i, contraction indices 8g..8g+7;
// B operand: column i, contraction indices 8g..8g+7; result: column i, rows 4g..4g+3.
// A score block S^T (16 keys x 16 queries) therefore leaves keys 4g..4g+3 of query i in lane (g, i).
// Two such blocks (keys 0..15 and 16..31 of a step) are used, as they are, as the B operand of the
// second product, with contraction slot (g, e) standing for key 4g + e (e < 4) or 16 + 4g + e - 4;
// the matching A operand V^T is fetched with two transposing reads per 16-wide slice of D.
#pragma once
#include "common.hpp"

namespace fa {

template <class T, int D>
struct DecCfg {
  // keys per wavefront step: two 16-key score blocks fill the contraction of the second product; at
  // head size 512 a 32-key step would not fit registers (loads in flight) or LDS (4 patches), so the
  // step is one block and the other half of the contraction multiplies zeros (the kernel is HBM-bound)
  static constexpr int TK = D > 256 ? 16 : 32;
  static constexpr int KB = TK / 16;  // 16-key score blocks per step
  static constexpr int ROWS = 16;  // query rows per workgroup
  static constexpr int DK = D < 32 ? 32 : D;  // contraction width of the first product (zero padded)
  static constexpr int KSTEPS = DK / 32;
  static constexpr int NDB = D / 16;          // 16-wide slices of the output
  static constexpr int CPR = D / 8;           // 16-byte chunks per row
  static constexpr int CH = (TK * CPR + 63) / 64;  // chunks per lane per step
  static constexpr int NSETS = 1;   // register sets of loads in flight
  static constexpr int K_LD = DK + 8;
  static constexpr int V_LD = D + 32;  // 64 B of padding: the 4 rows of a transposing read fall in disjoint banks
  static constexpr int WAVE_ELEMS = TK * K_LD + TK * V_LD;
  static constexpr size_t STAGING_BYTES = 4 * WAVE_ELEMS * sizeof(T);
  // merge area: per wavefront ROWS x (D + 2) floats
  static constexpr size_t MERGE_BYTES = 4 * ROWS * (D + 2) * sizeof(float);
  static constexpr size_t WORK_BYTES = STAGING_BYTES > MERGE_BYTES ? STAGING_BYTES : MERGE_BYTES;
  // at head size 512 the query rows (64 registers as an MFMA operand) live in LDS behind the work area
  static constexpr bool Q_IN_LDS = D > 256;
  static constexpr int Q_LD = DK + 8;
  static constexpr size_t LDS_BYTES = WORK_BYTES + (Q_IN_LDS ? ROWS * Q_LD * sizeof(T) : 0);
};

// Result of the per-workgroup pass, valid in every thread after decode_block():
// thread t owns output elements (row = idx / D, d = idx % D) for idx = t, t + 256, ... < 16 * D.
template <int D>
struct DecodeOut {
  static constexpr int kPerThread = (16 * D + kThreads - 1) / kThreads;
  float o[kPerThread];        // un-normalised sum_j p_j v_j, relative to row_max
  float row_max[kPerThread];  // running maximum of the raw (unscaled) scores, -inf if no key seen
  float row_sum[kPerThread];  // sum_j exp(scale * (s_j - row_max))
};

// Src must provide:
//   struct Ids;                                             per-lane lookup state for one step
//   void lookup(Ids&, int n0, int n_end, int lane) const;   start resolving the rows of the step at key n0
//   const T* k_row(const Ids&, int i, int n) const;         row pointer of key n (chunk slot i of the lane)
//   const T* v_row(const Ids&, int i, int n) const;
template <class T, int D, class Src>
FA_DEVICE void decode_block(const Src& src, const T* q_row /* query row of lane % 16, or nullptr */,
                            int n_begin, int n_end, int lane_limit /* keys n < lane_limit are visible */,
                            float c2, unsigned char* smem, DecodeOut<D>& out) {
  using C = DecCfg<T, D>;
  using V8 = typename hw::Elem<T>::v8;
  const int tid = hw::thread_id(), lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, g = lane >> 4;
  T* sK = (T*)smem + wave * C::WAVE_ELEMS;
  T* sV = sK + C::TK * C::K_LD;

  // this lane's query row as B operand: contraction indices 32 ks + 8 g + 0..7
  V8 qreg[C::Q_IN_LDS ? 1 : C::KSTEPS];
  T* sQ = (T*)(smem + C::WORK_BYTES);
  if (C::Q_IN_LDS) {  // wavefront w stores every fourth 32-wide slice of the 16 rows
    for (int ks = wave; ks < C::KSTEPS; ks += 4) {
      u32x4 z = {0u, 0u, 0u, 0u};
      if (q_row) z = *(const u32x4*)(q_row + 32 * ks + 8 * g);
      *(u32x4*)(sQ + li * C::Q_LD + 32 * ks + 8 * g) = z;
    }
    hw::block_sync();
  } else {
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      if (q_row && 32 * ks + 8 * g < D) z = *(const u32x4*)(q_row + 32 * ks + 8 * g);
      qreg[ks] = hw::as_v8<T>(z);
    }
  }
  if (C::DK != D) {  // columns D..DK-1 of the key patch are read by the first product, never loaded
    for (int i = lane; i < C::TK * C::K_LD; i += 64) sK[i] = (T)0.f;
  }

  const int limit = imin(lane_limit, n_end);
  float m_i = neg_inf(), l_i = 0.f;
  hw::f32x4 oacc[C::NDB];
#pragma unroll
  for (int i = 0; i < C::NDB; ++i) oacc[i] = hw::f32x4{0.f, 0.f, 0.f, 0.f};

  const int total_tiles = n_end > n_begin ? cdiv(n_end - n_begin, C::TK) : 0;
  const int my_tiles = total_tiles > wave ? (total_tiles - wave + 3) / 4 : 0;
  auto tile_start = [&](int j) { return n_begin + (wave + 4 * j) * C::TK; };

  u32x4 kst0[C::CH], vst0[C::CH];
  u32x4 kst1[C::NSETS == 2 ? C::CH : 1], vst1[C::NSETS == 2 ? C::CH : 1];
  typename Src::Ids ids;
  // Branch-free on purpose: a guarded load would put every chunk in its own basic block, and the
  // compiler then waits for ALL outstanding loads before each one.  Rows past the end are read from
  // the last valid row instead; their scores are masked, and finite values times zero stay zero.
  // Precondition that follows: the value rows of every key in [n_begin, n_end) are finite, including
  // keys that only the causal limit hides from some query row -- they enter the second product with
  // probability 0.  The reference's kernels form the same product p @ v with p = 0 at those
  // positions (flash.py:448-461, split_kv.py:137), so a non-finite value there gives NaN in both.
  static_assert(C::TK * C::CPR == 64 * C::CH, "a step is a whole number of 64-lane load instructions");
  auto fetch = [&](int n0, u32x4* kst, u32x4* vst) {
#pragma unroll
    for (int i = 0; i < C::CH; ++i) {
      const int c = lane + 64 * i;
      const int row = c / C::CPR, col = (c % C::CPR) * 8;
      const int n = imin(n0 + row, n_end - 1);
      kst[i] = *(const u32x4*)(src.k_row(ids, i, n) + col);
      vst[i] = *(const u32x4*)(src.v_row(ids, i, n) + col);
    }
  };
  auto commit = [&](const u32x4* kst, const u32x4* vst) {
#pragma unroll
    for (int i = 0; i < C::CH; ++i) {
      const int c = lane + 64 * i;
      const int row = c / C::CPR, col = (c % C::CPR) * 8;
      *(u32x4*)(sK + row * C::K_LD + col) = kst[i];
      *(u32x4*)(sV + row * C::V_LD + col) = vst[i];
    }
  };

  // loads of the first NSETS steps, and the block-table rows of the step after them
  if (my_tiles > 0) {
    src.lookup(ids, tile_start(0), n_end, lane);
    fetch(tile_start(0), kst0, vst0);
  }
  if (C::NSETS == 2 && my_tiles > 1) {
    src.lookup(ids, tile_start(1), n_end, lane);
    fetch(tile_start(1), kst1, vst1);
  }
  if (my_tiles > C::NSETS) src.lookup(ids, tile_start(C::NSETS), n_end, lane);

  auto step = [&](int j, u32x4* kst, u32x4* vst) {
    const int n0 = tile_start(j);
    hw::wave_sync();
    commit(kst, vst);
    if (j + C::NSETS < my_tiles) {
      fetch(tile_start(j + C::NSETS), kst, vst);
      if (j + C::NSETS + 1 < my_tiles) src.lookup(ids, tile_start(j + C::NSETS + 1), n_end, lane);
    }
    hw::wave_sync();

    // ---- S^T: blocks of 16 keys x 16 queries ----
    hw::f32x4 s[C::KB];
#pragma unroll
    for (int kb = 0; kb < C::KB; ++kb) s[kb] = hw::f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int kKGroup = C::KSTEPS < 8 ? C::KSTEPS : 8;
#pragma unroll
    for (int k0 = 0; k0 < C::KSTEPS; k0 += kKGroup) {
      V8 ka[C::KB][kKGroup];  // operands requested before the first product of the group: one exposed LDS latency
      V8 qb[kKGroup];
#pragma unroll
      for (int ks = 0; ks < kKGroup; ++ks)
      {
        if constexpr (C::Q_IN_LDS) qb[ks] = hw::as_v8<T>(*(const u32x4*)(sQ + li * C::Q_LD + 32 * (k0 + ks) + 8 * g));
        else qb[ks] = qreg[k0 + ks];
      }
#pragma unroll
      for (int kb = 0; kb < C::KB; ++kb)
#pragma unroll
        for (int ks = 0; ks < kKGroup; ++ks)
          ka[kb][ks] = hw::as_v8<T>(*(const u32x4*)(sK + (16 * kb + li) * C::K_LD + 32 * (k0 + ks) + 8 * g));
      hw::sched_fence();
#pragma unroll
      for (int kb = 0; kb < C::KB; ++kb)
#pragma unroll
        for (int ks = 0; ks < kKGroup; ++ks) s[kb] = hw::mfma16(ka[kb][ks], qb[ks], s[kb]);
    }
    float mx = neg_inf();
#pragma unroll
    for (int kb = 0; kb < C::KB; ++kb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = n0 + 16 * kb + 4 * g + r;
        s[kb][r] = (n < limit) ? s[kb][r] : neg_inf();
        mx = fmaxf(mx, s[kb][r]);
      }
    {  // the 4 lane groups of a query row: three independent exchanges, one exposed latency
      const float a = hw::shfl_xor(mx, 16), b = hw::shfl_xor(mx, 32), c = hw::shfl_xor(mx, 48);
      mx = fmaxf(fmaxf(mx, a), fmaxf(b, c));
    }
    const float m_new = fmaxf(m_i, mx);
    const float m_use = (m_new == neg_inf()) ? 0.f : m_new;
    const float alpha = hw::exp2_fast((m_i - m_use) * c2);
    const float shift = -m_use * c2;
    float psum = 0.f;
    V8 pb;
#pragma unroll
    for (int i = 0; i < 8; ++i) pb[i] = (T)0.f;
#pragma unroll
    for (int kb = 0; kb < C::KB; ++kb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = hw::exp2_fast(fmaf(s[kb][r], c2, shift));
        psum += e;
        pb[4 * kb + r] = (T)e;
      }
    l_i = l_i * alpha + psum;
    m_i = m_new;
    // ---- O^T += V^T P^T, one 16-wide slice of D at a time ----
    constexpr int kGroup = C::NDB < 8 ? C::NDB : 8;  // operands requested ahead of their products
#pragma unroll
    for (int d0 = 0; d0 < C::NDB; d0 += kGroup) {
      V8 va[kGroup];
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const T* pv = sV + (4 * g + (li >> 2)) * C::V_LD + 16 * (d0 + u) + 4 * (li & 3);
        const hw::short4v lo = hw::lds_read_tr16(pv);
        va[u] = hw::join_v8<T>(lo, C::KB == 2 ? hw::lds_read_tr16(pv + (C::KB - 1) * 16 * C::V_LD) : hw::short4v{0, 0, 0, 0});
      }
      hw::sched_fence();
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        hw::f32x4 o = oacc[d0 + u];
        o *= alpha;
        oacc[d0 + u] = hw::mfma16(va[u], pb, o);
      }
    }
  };

  if (C::NSETS == 2) {
    for (int j = 0; j < my_tiles; j += 2) {
      step(j, kst0, vst0);
      if (j + 1 < my_tiles) step(j + 1, kst1, vst1);
    }
  } else {
    for (int j = 0; j < my_tiles; ++j) step(j, kst0, vst0);
  }

  // ---- merge the 4 wavefronts: area[w][row][0..D-1] = O, [D] = max, [D+1] = sum ----
  l_i += hw::shfl_xor(l_i, 16);
  l_i += hw::shfl_xor(l_i, 32);
  hw::block_sync();  // every wavefront is done with its staging patch
  float* area = (float*)smem;
  constexpr int RS = D + 2;
  {
    float* mine = area + (wave * C::ROWS + li) * RS;
#pragma unroll
    for (int db = 0; db < C::NDB; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[16 * db + 4 * g + r] = oacc[db][r];
    if (g == 0) { mine[D] = m_i; mine[D + 1] = l_i; }
  }
  hw::block_sync();
#pragma unroll
  for (int e = 0; e < DecodeOut<D>::kPerThread; ++e) {
    const int idx = tid + e * kThreads;
    const int row = (idx / D) % C::ROWS, d = idx % D;  // idx >= 16 * D occurs only when 16 * D < 256; callers skip it
    float mw[4], mm = neg_inf();
#pragma unroll
    for (int w = 0; w < 4; ++w) { mw[w] = area[(w * C::ROWS + row) * RS + D]; mm = fmaxf(mm, mw[w]); }
    const float m_use = (mm == neg_inf()) ? 0.f : mm;
    float acc = 0.f, sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = hw::exp2_fast((mw[w] - m_use) * c2);  // -inf -> 0
      acc += f * area[(w * C::ROWS + row) * RS + d];
      sum += f * area[(w * C::ROWS + row) * RS + D + 1];
    }
    out.o[e] = acc;
    out.row_max[e] = mm;
    out.row_sum[e] = sum;
  }
}

}  // namespace fa
