// FlashAttention-2 forward for gfx950, and its piecewise (two score regimes) variant.
//
// Replaces the reference's Triton kernels `_fwd_kernel` (src/flag_attn/flash.py:325-489) and the
// piecewise `_fwd_kernel` (src/flag_attn/piecewise.py:223-370).
//
// Work decomposition: one workgroup (4 wavefronts) owns 128 query rows of one (batch, head); each
// wavefront owns 32 of them and keeps, for the whole kernel,
//   * its Q rows as the B operand of S^T = K Q^T (registers, never in LDS),
//   * O^T (D x 32) as fp32 accumulators,
//   * the running row maximum and the lane-partial row sum of the online softmax.
// Working on S^T puts one query row in one lane (and its lane^32 twin), so the row maximum and row
// sum are register reductions plus one cross-lane exchange, and the probabilities come out of the
// first product already in the operand layout of the second (O^T = V^T P^T) -- no LDS round trip.
// K/V tiles of 64 keys are staged global -> registers -> LDS, double buffered, with the next tile's
// global loads in flight during the current tile's matrix work.  V is read from LDS through the
// transposing 64-bit read.
#include "common.hpp"
#include "params.hpp"

namespace fa {

template <class T, int D, bool PW>
struct FwdCfg {
  static constexpr int BM = 128, BN = 64;
  static constexpr int DV = D < 32 ? 32 : D;  // value/output width rounded up to one MFMA block
  static constexpr int KSTEPS = D / 16;
  static constexpr int WAVES_PER_SIMD = 2;  // register budget per wavefront
  static constexpr int K_LD = D + 8;    // 16 B of padding: conflict-free 16-byte row reads
  static constexpr int V_LD = DV + 32;  // 64 B of padding: the 4 rows of a transposing read fall in disjoint banks
  static constexpr int K_TILE = BN * K_LD, V_TILE = BN * V_LD;
  static constexpr int STAGE = K_TILE + V_TILE;  // elements per pipeline stage
  static constexpr size_t LDS_BYTES = 2 * STAGE * sizeof(T);
};

// DROP: dropout as in the reference (flash.py:450-457, 479-482): the row sum is taken before the mask,
// dropped probabilities do not enter the second product, the output is scaled by 1 / (1 - dropout_p).
template <class T, int D, bool PW, bool DROP = false>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, (FwdCfg<T, D, PW>::WAVES_PER_SIMD)) fa_fwd_kernel(FwdParams p) {
  static_assert(!(PW && DROP), "piecewise attention has no dropout");
  using C = FwdCfg<T, D, PW>;
  using V8 = typename hw::Elem<T>::v8;
  FA_LDS_DECL(smem);
  T* lds = (T*)smem;

  const int tid = hw::thread_id(), lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const TileId wg = tile_of_workgroup(p.H, p.B);
  const int mb = (p.M + C::BM - 1) / C::BM - 1 - wg.rank;  // long rows first under the causal mask
  const int head = wg.head, batch = wg.batch;
  const int hk = head / p.group;
  const int M = p.M, N = p.N, pseq = N - M;
  const int m0 = mb * C::BM, mw = m0 + wave * 32, my_m = mw + l32;

  const T* qb = (const T*)p.q.ptr + batch * p.q.sb + head * p.q.sh;
  const T* kb = (const T*)p.k.ptr + batch * p.k.sb + hk * p.k.sh;
  const T* vb = (const T*)p.v.ptr + batch * p.v.sb + hk * p.v.sh;
  const T* q2b = PW ? (const T*)p.q2.ptr + batch * p.q2.sb + head * p.q2.sh : nullptr;
  const T* k2b = PW ? (const T*)p.k2.ptr + batch * p.k2.sb + hk * p.k2.sh : nullptr;

  // ---- Q rows of this lane as B operands: k = 16 * kk + 8 * hh + 0..7 ----
  V8 qreg[C::KSTEPS];
  auto load_q = [&](const T* base, int64_t row_stride) {
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk) {
      u32x4 z = {0u, 0u, 0u, 0u};
      if (my_m < M) z = *(const u32x4*)(base + (int64_t)my_m * row_stride + 16 * kk + 8 * hh);
      qreg[kk] = hw::as_v8<T>(z);
    }
  };

  // ---- key range of this workgroup ----
  int hi = N;
  if (p.causal) hi = imin(N, pseq + m0 + C::BM);
  const int n_tiles = hi > 0 ? cdiv(hi, C::BN) : 0;

  // When D < 32 the value tile has columns D..31 that no load ever writes: clear both stages once.
  if (C::DV != D) {
    for (int i = tid; i < 2 * C::STAGE; i += kThreads) lds[i] = (T)0.f;
    hw::block_sync();
  }

  const float c2 = p.sm_scale * kLog2e;
  constexpr float kLazyBits = 8.f;
  const float lazy_tau = c2 > 0.f ? kLazyBits / c2 : 0.f;   // in units of raw scores; a non-positive scale keeps the exact maximum
  // dropout counter of (my_m, key 0)
  const uint64_t drop_row = DROP ? p.offset + (((uint64_t)batch * p.H + head) * M + (uint64_t)(my_m < M ? my_m : 0)) * N : 0;
  float m_i = neg_inf(), l_i = 0.f;
  f32x16 oacc[C::DV / 32];
#pragma unroll
  for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;

  // Piecewise: the score of (m, n) comes from (q2, k2) when the distance m + pseq - n is >= w and
  // from (q1, k1) otherwise.  The two regimes are two passes of the same loop -- first the keys far
  // from this workgroup's rows with (q2, k2), then the near ones with (q1, k1) -- each masking the
  // entries that belong to the other; the online softmax does not care that a key tile crossed by
  // the threshold is visited twice.  So the variant needs no more registers or LDS than plain flash.
  bool far_phase = false;
  const T* k_src = kb;
  int64_t k_stride = p.k.st;
  TileMover<T, C::BN, D> kr, vr;
  vr.init(tid, p.v.st);
  auto fetch = [&](int n0) {
    const int rows = N - n0;
    kr.fetch(k_src + (int64_t)n0 * k_stride, rows);
    vr.fetch(vb + (int64_t)n0 * p.v.st, rows);
  };
  auto commit = [&](int stage) {
    T* s = lds + stage * C::STAGE;
    kr.template commit<C::K_LD>(s);
    vr.template commit<C::V_LD>(s + C::K_TILE);
  };

  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // One key tile.  `plain`: no mask touches the tile for any row of this wavefront, so the body has none of the
  // mask branches and the compiler sees one basic block from the first product to the second (the rare rescale
  // branch aside).  The two variants run in loops of their own.
  auto step = [&](auto plain_tag, int it, int t_end, int kStage) {
    constexpr bool plain = decltype(plain_tag)::value;
    const int n0 = it * C::BN;
    const bool more = it + 1 < t_end;
    if (more) fetch(n0 + C::BN);

    const T* sK = lds + kStage * C::STAGE;
    const T* sV = sK + C::K_TILE;

    // A tile that the causal mask hides from all 32 rows of this wavefront (the last tiles of a
    // workgroup, for its upper wavefronts) only takes part in the data movement.
    if (plain || !(p.causal && (mw + 31 + pseq < n0))) {
    // ---- S^T = K Q^T : BN/32 blocks of (32 keys x 32 queries) ----
    // the two blocks advance together: consecutive matrix instructions never wait for each other
    f32x16 s[C::BN / 32];
#pragma unroll
    for (int nb = 0; nb < C::BN / 32; ++nb) s[nb] = zero16;
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk)
#pragma unroll
      for (int nb = 0; nb < C::BN / 32; ++nb)
        s[nb] = hw::mfma32(operand_rowmajor<T, C::K_LD>(sK, nb * 32, 16 * kk, lane), qreg[kk], s[nb]);
    hw::sched_prefetched_operands<(C::BN / 32) * C::KSTEPS, (C::KSTEPS >= 4 ? 4 : C::KSTEPS)>();

    // ---- masks (key tail, causal, the other regime's entries) only on tiles that need them ----
    bool need_mask = !plain && ((n0 + C::BN > N) || (p.causal && (n0 + C::BN - 1 > pseq + mw)));
    if (PW && !plain) need_mask = need_mask || (far_phase ? (mw + pseq - (n0 + C::BN - 1) < p.w) : (mw + 31 + pseq - n0 >= p.w));
    if (need_mask) {
#pragma unroll
      for (int nb = 0; nb < C::BN / 32; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          int n = n0 + nb * 32 + block_row(r, hh);
          bool keep = (n < N) && (!p.causal || (my_m + pseq >= n));
          if (PW) keep = keep && ((my_m + pseq - n >= p.w) == far_phase);
          s[nb][r] = keep ? s[nb][r] : neg_inf();
        }
    }

    // ---- online softmax (base 2); a query row lives in lanes l and l ^ 32 ----
    float mx = neg_inf();
#pragma unroll
    for (int nb = 0; nb < C::BN / 32; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[nb][r]);
    mx = fmaxf(mx, hw::xor32(mx));
    // The reference of the exponentials (m_i) is raised only when the tile's maximum exceeds it by more than
    // 2^kLazyBits in the base-2 domain: softmax does not depend on the reference, probabilities up to 2^8 are
    // exact in fp32 and in range for fp16 and bf16, and the accumulators are then rescaled a few times per
    // row instead of in most tiles (the running maximum of 32 rows moves in every second tile of a long row).
    const bool grow = mx > m_i + lazy_tau;   // always true for the first visible key (m_i = -inf)
    const float m_new = grow ? mx : m_i;
    const float m_use = (m_new == neg_inf()) ? 0.f : m_new;  // row with no visible key so far
    const float shift = -m_use * c2;
    float psum = 0.f;
#pragma unroll
    for (int nb = 0; nb < C::BN / 32; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float e = hw::exp2_fast(fmaf(s[nb][r], c2, shift));
        psum += e;
        if (DROP) e = dropout_keeps(drop_row + (uint64_t)(n0 + nb * 32 + block_row(r, hh)), p.seed, p.dropout_p) ? e : 0.f;
        s[nb][r] = e;
      }
    // The accumulators are rescaled only when some row of the wavefront raised its maximum;
    // after the first few tiles that is rare.
    if (hw::wave_any(grow)) {
      hw::keep_branch();
      const float alpha = hw::exp2_fast((m_i - m_use) * c2);
      l_i *= alpha;
#pragma unroll
      for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
    }
    l_i += psum;
    m_i = m_new;

    // ---- O^T += V^T P^T ; P is rounded to the input dtype as the reference does ----
#pragma unroll
    for (int nb = 0; nb < C::BN / 32; ++nb)
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        V8 pb = pack_half_block<T>(s[nb], c);
#pragma unroll
        for (int db = 0; db < C::DV / 32; ++db)
          oacc[db] = hw::mfma32(operand_transposed<T, C::V_LD>(sV, nb * 32 + 16 * c, db * 32, lane), pb, oacc[db]);
      }

    }
    if (more) commit(kStage ^ 1);
    hw::block_sync();
  };

  int stage = 0;
#pragma unroll 1
  for (int ph = 0; ph < (PW ? 2 : 1); ++ph) {
    int t_begin = 0, t_end = n_tiles;
    far_phase = PW && ph == 0;
    if (PW) {
      if (far_phase) {  // keys n <= m0 + BM - 1 + pseq - w are far from some row of the workgroup
        const int far_hi = imin(hi, m0 + C::BM + pseq - p.w);
        t_end = far_hi > 0 ? cdiv(far_hi, C::BN) : 0;
      } else {          // keys n > m0 + pseq - w are near some row
        t_begin = imax(0, m0 + pseq - p.w + 1) / C::BN;
      }
    }
    if (t_begin >= t_end) continue;
    k_src = far_phase ? k2b : kb;
    k_stride = far_phase ? p.k2.st : p.k.st;
    kr.init(tid, k_stride);
    load_q(far_phase ? q2b : qb, far_phase ? p.q2.st : p.q.st);
    fetch(t_begin * C::BN);
    commit(stage);
    hw::block_sync();
    hw::wait_global_loads();  // Q rows
    // Tiles [plain_lo, plain_hi): complete (64 keys exist), visible to the wavefront's first row under the causal
    // mask and, for piecewise attention, wholly inside this pass's regime for all 32 rows.
    int plain_lo = t_begin, plain_hi = imin(t_end, N / C::BN);
    if (p.causal) plain_hi = imin(plain_hi, imax(0, mw + pseq + 1) / C::BN);
    if (PW) {
      if (far_phase) plain_hi = imin(plain_hi, imax(0, mw + pseq - p.w + 1) / C::BN);   // 64 it + 63 <= mw + pseq - w
      else plain_lo = imax(plain_lo, imax(-1, (mw + 31 + pseq - p.w) >> 6) + 1);          // 64 it > mw + 31 + pseq - w
    }
    plain_lo = hw::uniform(imin(plain_lo, t_end));
    plain_hi = hw::uniform(imax(plain_hi, plain_lo));
    int it = t_begin;
#pragma unroll 1
    for (; it < plain_lo; ++it) { step(std::false_type{}, it, t_end, stage); stage ^= 1; }
#pragma unroll 1
    for (; it < plain_hi; ++it) { step(std::true_type{}, it, t_end, stage); stage ^= 1; }
#pragma unroll 1
    for (; it < t_end; ++it) { step(std::false_type{}, it, t_end, stage); stage ^= 1; }
  }

  // ---- epilogue: O = acc / l, L = m * scale + ln(l); rows that saw no key give O = 0, L = -inf ----
  const float l_tot = l_i + hw::xor32(l_i);
  const bool empty = !(l_tot > 0.f);
  const float inv = empty ? 0.f : (DROP ? 1.f / ((1.f - p.dropout_p) * l_tot) : 1.f / l_tot);
  if (my_m < M) {
    T* ob = (T*)p.o.ptr + batch * p.o.sb + head * p.o.sh + (int64_t)my_m * p.o.st;
#pragma unroll
    for (int db = 0; db < C::DV / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        int d = db * 32 + 8 * g + 4 * hh;
        if (d < D) {
          hw::u32x2 w;
          w[0] = (uint32_t)hw::bits16<T>(oacc[db][4 * g + 0] * inv) | ((uint32_t)hw::bits16<T>(oacc[db][4 * g + 1] * inv) << 16);
          w[1] = (uint32_t)hw::bits16<T>(oacc[db][4 * g + 2] * inv) | ((uint32_t)hw::bits16<T>(oacc[db][4 * g + 3] * inv) << 16);
          *(hw::u32x2*)(ob + d) = w;
        }
      }
    if (hh == 0)
      p.lse[((int64_t)batch * p.H + head) * M + my_m] = empty ? neg_inf() : m_i * p.sm_scale + hw::log_nat(l_tot);
  }
}

template <class T, bool PW, bool DROP>
static int launch_fwd(const FwdParams& p, hipStream_t stream) {
  dim3 grid(((p.M + 127) / 128) * p.H * p.B, 1, 1);
  switch (p.D) {
    case 16: return launch(fa_fwd_kernel<T, 16, PW, DROP>, grid, FwdCfg<T, 16, PW>::LDS_BYTES, stream, p);
    case 32: return launch(fa_fwd_kernel<T, 32, PW, DROP>, grid, FwdCfg<T, 32, PW>::LDS_BYTES, stream, p);
    case 64: return launch(fa_fwd_kernel<T, 64, PW, DROP>, grid, FwdCfg<T, 64, PW>::LDS_BYTES, stream, p);
    case 128: return launch(fa_fwd_kernel<T, 128, PW, DROP>, grid, FwdCfg<T, 128, PW>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

template <class T>
static int dispatch_fwd(const FwdParams& p, bool piecewise, hipStream_t stream) {
  if (piecewise) return launch_fwd<T, true, false>(p, stream);
  return p.dropout_p > 0.f ? launch_fwd<T, false, true>(p, stream) : launch_fwd<T, false, false>(p, stream);
}

// Which kernel a launch without an explicit tile takes: the 256-row kernel is the faster one per tile,
// but its workgroups hold a compute unit alone, so it needs at least one workgroup per compute unit.
static bool prefer_wide(const FwdParams& p) {
  const int num_cus = num_cus_of_current_device();
  return num_cus > 0 && (int64_t)((p.M + 255) / 256) * p.H * p.B >= num_cus;
}

int run_fwd(const FwdParams& p, bool piecewise, hipStream_t stream) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0 || p.N < 0 || p.group <= 0) return kBadArgument;
  if (!(p.dropout_p >= 0.f && p.dropout_p < 1.f) || (piecewise && p.dropout_p > 0.f)) return kBadArgument;
  if (p.block_m != 0 && p.block_m != 128 && p.block_m != 256) return kUnsupported;
  if (p.block_m == 256 && (piecewise || !fwd_wide_supported(p))) return kUnsupported;
  if (!piecewise && (p.block_m == 256 || (p.block_m == 0 && fwd_wide_supported(p) && prefer_wide(p)))) return run_fwd_wide(p, stream);
  if (p.dtype == kDtypeF16) return dispatch_fwd<hw::half_t>(p, piecewise, stream);
  if (p.dtype == kDtypeBF16) return dispatch_fwd<hw::bf16_t>(p, piecewise, stream);
  return kUnsupported;
}

}  // namespace fa
