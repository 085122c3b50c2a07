// Total attention: column sums of the softmax matrix, recomputed from Q, K and the saved
// log-normalizer.  Replaces `_total_attention_kernel` (src/flag_attn/total.py:50-142).
//
// A wavefront owns 32 keys whose K rows sit in registers as the B operand of S = Q K^T
// (queries x keys, one key per lane); P = exp2(S * scale * log2e - L * log2e) is summed over the
// query index, which runs along registers and the two lane halves, so the column sum needs no
// shared memory.  Query tiles of 64 rows (and their L values) are double buffered through LDS.
#include "common.hpp"
#include "params.hpp"

namespace fa {

template <class T, int D>
struct TotCfg {
  static constexpr int BN = 128, BM = 64;
  static constexpr int KSTEPS = D / 16;
  static constexpr int LD = D + 8;
  static constexpr int TILE = BM * LD;
  static constexpr size_t STAGE_BYTES = TILE * sizeof(T) + BM * sizeof(float);
  static constexpr size_t LDS_BYTES = 2 * STAGE_BYTES;
};

template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS(kThreads) fa_total_kernel(TotalParams p) {
  using C = TotCfg<T, D>;
  using V8 = typename hw::Elem<T>::v8;
  FA_LDS_DECL(smem);

  const int tid = hw::thread_id(), lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const TileId wg = tile_of_workgroup(p.H, p.B);  // key blocks in ascending order: most queries first
  const int head = wg.head, batch = wg.batch;
  const int hk = head / p.group;
  const int M = p.M, N = p.N, pseq = N - M;
  const int n0 = wg.rank * C::BN, nw = n0 + wave * 32, my_n = nw + l32;

  const T* qb = (const T*)p.q.ptr + batch * p.q.sb + head * p.q.sh;
  const T* kb = (const T*)p.k.ptr + batch * p.k.sb + hk * p.k.sh;
  const float* lse = p.lse + ((int64_t)batch * p.H + head) * M;

  V8 kreg[C::KSTEPS];
#pragma unroll
  for (int kk = 0; kk < C::KSTEPS; ++kk) {
    u32x4 a = {0u, 0u, 0u, 0u};
    if (my_n < N) a = *(const u32x4*)(kb + (int64_t)my_n * p.k.st + 16 * kk + 8 * hh);
    kreg[kk] = hw::as_v8<T>(a);
  }

  int m_lo = 0;
  if (p.causal) m_lo = (imax(0, n0 - pseq) / C::BM) * C::BM;
  const int n_tiles = m_lo < M ? cdiv(M - m_lo, C::BM) : 0;

  TileMover<T, C::BM, D> qr;
  qr.init(tid, p.q.st);
  float l_reg = 0.f;
  int l_row = 0;
  auto fetch = [&](int m0) {
    qr.fetch(qb + (int64_t)m0 * p.q.st, M - m0);
    // branch-free, and nothing consumes the load here (the wait would cover the tile loads too)
    l_row = m0 + (tid & (C::BM - 1));
    l_reg = lse[imin(l_row, M - 1)];
  };
  auto commit = [&](int stage) {
    unsigned char* base = smem + stage * C::STAGE_BYTES;
    qr.template commit<C::LD>((T*)base);
    // rows past M: P = 0
    if (tid < C::BM) ((float*)(base + C::TILE * sizeof(T)))[tid] = l_row < M ? l_reg * kLog2e : __builtin_inff();
  };

  if (n_tiles > 0) { fetch(m_lo); commit(0); }
  hw::block_sync();
  hw::wait_global_loads();  // K rows

  const float c2 = p.sm_scale * kLog2e;
  float colsum = 0.f;

  for (int it = 0; it < n_tiles; ++it) {
    const int m0 = m_lo + it * C::BM;
    const bool more = it + 1 < n_tiles;
    if (more) fetch(m0 + C::BM);
    const unsigned char* base = smem + (it & 1) * C::STAGE_BYTES;
    const T* sQ = (const T*)base;
    const float* sL = (const float*)(base + C::TILE * sizeof(T));
#pragma unroll
    for (int sb = 0; sb < C::BM / 32; ++sb) {
      const int mr0 = m0 + sb * 32;
      if (p.causal && (mr0 + 31 + pseq < nw)) continue;
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
      for (int kk = 0; kk < C::KSTEPS; ++kk)
        s = hw::mfma32(operand_rowmajor<T, C::LD>(sQ, sb * 32, 16 * kk, lane), kreg[kk], s);
      const bool need_mask = p.causal && (mr0 + pseq < nw + 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int ml = sb * 32 + block_row(r, hh);
        float pv = hw::exp2_fast(fmaf(s[r], c2, -sL[ml]));
        if (need_mask) pv = (m0 + ml + pseq >= my_n) ? pv : 0.f;
        colsum += pv;
      }
    }
    if (more) commit((it + 1) & 1);
    hw::block_sync();
  }

  colsum += hw::xor32(colsum);
  if (hh == 0 && my_n < N) p.total[((int64_t)batch * p.H + head) * N + my_n] = colsum;
}

template <class T>
static int launch_total(const TotalParams& p, hipStream_t stream) {
  dim3 grid(((p.N + 127) / 128) * p.H * p.B, 1, 1);
  switch (p.D) {
    case 16: return launch(fa_total_kernel<T, 16>, grid, TotCfg<T, 16>::LDS_BYTES, stream, p);
    case 32: return launch(fa_total_kernel<T, 32>, grid, TotCfg<T, 32>::LDS_BYTES, stream, p);
    case 64: return launch(fa_total_kernel<T, 64>, grid, TotCfg<T, 64>::LDS_BYTES, stream, p);
    case 128: return launch(fa_total_kernel<T, 128>, grid, TotCfg<T, 128>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

int run_total(const TotalParams& p, hipStream_t stream) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0 || p.N <= 0 || p.group <= 0) return kBadArgument;
  if (p.dtype == kDtypeF16) return launch_total<hw::half_t>(p, stream);
  if (p.dtype == kDtypeBF16) return launch_total<hw::bf16_t>(p, stream);
  return kUnsupported;
}

}  // namespace fa
