// FlashAttention-2 backward for gfx950 (and the piecewise variant): the row-dot preprocess, a
// kernel that owns a block of keys and produces dK/dV, and a kernel that owns a block of queries and
// produces dQ.  As in the reference there is no atomic read-modify-write: every output tile has
// exactly one writer.
//
// Replaces `_bwd_preprocess` (src/flag_attn/flash.py:522-568), `_bwd_kv_kernel` (flash.py:571-745),
// `_bwd_q_kernel` (flash.py:748-909) and their piecewise counterparts
// (src/flag_attn/piecewise.py:407-447, 450-627, 630-792).
//
// Shared scheme: P is recomputed as exp2(S * scale * log2e - L * log2e) from the saved
// log-normalizer; masked entries are removed by select (never by multiplying), because a row that
// saw no key has L = -inf and would give inf * 0.
//
//  dK/dV kernel: a wavefront owns 32 keys; K and V rows sit in registers as B operands of
//    S = Q K^T and dP = dO V^T (queries x keys, one key per lane).  P and dS then come out of the MFMA
//    in the A-operand layout of dV += P^T dO and dK += dS^T Q, whose B operands (dO, Q with the
//    query index as contraction index) are fetched from the LDS tiles with the transposing read.
//  dQ kernel: a wavefront owns 32 queries; Q and dO rows sit in registers as B operands of
//    S^T = K Q^T and dP^T = V dO^T (keys x queries, one query per lane, so L and delta are per-lane
//    scalars); dS^T is the B operand of dQ^T += K^T dS^T, with K^T read transposed from LDS.
#include "common.hpp"
#include "params.hpp"

namespace fa {

// ------------------------------------------------------------------------------ preprocess ----
template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS(kThreads) fa_bwd_delta_kernel(BwdParams p) {
  constexpr int kLanesPerRow = D / 8;
  constexpr int kRows = kThreads / kLanesPerRow;
  const int tid = hw::thread_id();
  const int row = hw::block_x() * kRows + tid / kLanesPerRow;
  const int col = (tid % kLanesPerRow) * 8;
  const int head = hw::block_y(), batch = hw::block_z();
  float acc = 0.f;
  if (row < p.M) {
    const T* o = (const T*)p.o.ptr + batch * p.o.sb + head * p.o.sh + (int64_t)row * p.o.st + col;
    const T* g = (const T*)p.dout.ptr + batch * p.dout.sb + head * p.dout.sh + (int64_t)row * p.dout.st + col;
    auto ov = hw::as_v8<T>(*(const u32x4*)o);
    auto gv = hw::as_v8<T>(*(const u32x4*)g);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += (float)ov[e] * (float)gv[e];
  }
#pragma unroll
  for (int s = 1; s < kLanesPerRow; s <<= 1) acc += hw::shfl_xor(acc, s);
  if (row < p.M && (tid % kLanesPerRow) == 0)
    p.delta[((int64_t)batch * p.H + head) * p.M + row] = acc;
}

template <class T>
static int launch_delta(const BwdParams& p, hipStream_t stream) {
  auto rows = [](int D) { return kThreads / (D / 8); };
  switch (p.D) {
    case 16: return launch(fa_bwd_delta_kernel<T, 16>, dim3((p.M + rows(16) - 1) / rows(16), p.H, p.B), 0, stream, p);
    case 32: return launch(fa_bwd_delta_kernel<T, 32>, dim3((p.M + rows(32) - 1) / rows(32), p.H, p.B), 0, stream, p);
    case 64: return launch(fa_bwd_delta_kernel<T, 64>, dim3((p.M + rows(64) - 1) / rows(64), p.H, p.B), 0, stream, p);
    case 128: return launch(fa_bwd_delta_kernel<T, 128>, dim3((p.M + rows(128) - 1) / rows(128), p.H, p.B), 0, stream, p);
  }
  return kUnsupported;
}

int run_bwd_delta(const BwdParams& p, hipStream_t stream) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0) return kBadArgument;
  if (p.dtype == kDtypeF16) return launch_delta<hw::half_t>(p, stream);
  if (p.dtype == kDtypeBF16) return launch_delta<hw::bf16_t>(p, stream);
  return kUnsupported;
}

// ------------------------------------------------------------------------------- dK and dV ----
template <class T, int D, bool PW>
struct KvCfg {
  static constexpr int BN = 128;  // keys per workgroup (32 per wavefront)
  static constexpr int BM = 64;   // queries per pipeline step
  static constexpr int DV = D < 32 ? 32 : D;
  static constexpr int KSTEPS = D / 16;
  static constexpr int LD = DV + (DV == 128 ? 24 : 40);  // 16-byte row reads and transposing reads both conflict-free
  static constexpr int TILE = BM * LD;
  // register budget the compiler may use: 256 registers (two wavefronts per SIMD) at the small head sizes; at 64
  // and 128 the slot-structured body gets all 512 (at 64 it needs 229, so two workgroups still share a CU)
  static constexpr int WAVES_PER_SIMD = D < 64 ? 2 : 1;
  // one wavefront per SIMD: overlap of matrix and element-wise work has to come from the instruction order
  static constexpr bool SLOTTED = WAVES_PER_SIMD == 1 && BM == 64 && (D == 128 || D == 64);
  static constexpr size_t STAGE_BYTES = 2 * TILE * sizeof(T) + 2 * BM * sizeof(float);  // Q, dO, L, delta
  // the slot-structured body writes the next tile into LDS and passes the barrier before its last
  // matrix instructions, which still read the current tile: three stages
  static constexpr int STAGES = SLOTTED ? 3 : 2;
  static constexpr size_t LDS_BYTES = STAGES * STAGE_BYTES;
};

// PW (piecewise): the score of (m, n) comes from (q2, k2) when the distance m + pseq - n is >= w and
// from (q1, k1) otherwise.  The two regimes are two passes over the query tiles -- the near rows
// with (q1, k1) accumulating dK1, then the far rows with (q2, k2) accumulating dK2 in the same
// registers -- each masking the entries of the other; dV accumulates over both.
//
// DS: also leave dS (rounded to T, as it enters dK += dS^T Q) in the workspace p.ds for
// fa_bwd_dq_from_ds_kernel, one 2 KB chunk per 32 x 32 block in the order the MFMA result holds it:
// chunk[c][lane] = 8 elements, queries 16c + 8g + 4(lane / 32) + e at position 4g + e, key lane % 32.
// Chunks are indexed (batch * H + head, key block, query block); both counts padded to 4.
//
// DROP: dropout as in the reference (flash.py:697-721): dV takes the masked P and is scaled by
// 1 / (1 - dropout_p); dP is masked and scaled likewise; dS = P (dP - delta) with the unmasked P.
//
// GROUPED: the workgroup walks more than one query head (see below); a separate instantiation,
// because the extra loop level costs the single-head kernel 10 % through register allocation alone.
template <class T, int D, bool PW, bool DS = false, bool DROP = false, bool GROUPED = false>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, (DROP ? 1 : KvCfg<T, D, PW>::WAVES_PER_SIMD)) fa_bwd_dkdv_kernel(BwdParams p) {
  static_assert(!(GROUPED && (PW || DROP)), "grouped accumulation is built for plain attention without dropout");
  static_assert(!(PW && DROP), "piecewise attention has no dropout");
  using C = KvCfg<T, D, PW>;
  using V8 = typename hw::Elem<T>::v8;
  FA_LDS_DECL(smem);

  const int tid = hw::thread_id(), lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  // One workgroup per (key block, chunk of query heads that share a kv head): it walks the heads of
  // the chunk one after the other and accumulates their dK / dV in the same registers, so the sum
  // over the chunk costs nothing.  chunk = group gives dK/dV per kv head; smaller chunks (more
  // workgroups, for launches that would not fill the device) leave group / chunk slices to add.
  const int chunk = GROUPED ? (p.chunk > 0 ? p.chunk : p.group) : 1;
  const TileId wg = tile_of_workgroup(p.H / chunk, p.B);  // key blocks in ascending order: most queries first
  const int slice = wg.head, batch = wg.batch;             // output slice = chunk index
  const int hk = slice * chunk / p.group;
  const int M = p.M, N = p.N, pseq = N - M;
  const int n0 = wg.rank * C::BN, nw = n0 + wave * 32, my_n = nw + l32;

  int head = slice * chunk;  // query head being processed
  const T* gb = nullptr;
  const T* vb = (const T*)p.v.ptr + batch * p.v.sb + hk * p.v.sh;
  const float* lse = nullptr;
  const float* dlt = nullptr;

  // K (of the current regime) and V rows of this lane as B operands (k = 16 kk + 8 hh + 0..7)
  V8 kreg[C::KSTEPS], vreg[C::KSTEPS];
  auto load_rows = [&](V8* dst, const T* base, int64_t row_stride) {
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk) {
      u32x4 a = {0u, 0u, 0u, 0u};
      if (my_n < N) a = *(const u32x4*)(base + (int64_t)my_n * row_stride + 16 * kk + 8 * hh);
      dst[kk] = hw::as_v8<T>(a);
    }
  };
  load_rows(vreg, vb, p.v.st);

  // first query tile that can see a key of this block under the causal mask
  int m_lo = 0;
  if (p.causal) m_lo = (imax(0, n0 - pseq) / C::BM) * C::BM;

  if (C::DV != D) {
    T* z = (T*)smem;
    for (int i = tid; i < (int)(C::LDS_BYTES / sizeof(T)); i += kThreads) z[i] = (T)0.f;
    hw::block_sync();
  }

  f32x16 dk[C::DV / 32], dv[C::DV / 32];
#pragma unroll
  for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dk[i][r] = 0.f; dv[i][r] = 0.f; }

  // dS chunks of this wavefront's key block: one row of the (key block, query block) chunk grid
  T* ds_row = nullptr;

  bool far_phase = false;
  const T* q_src = nullptr;
  int64_t q_stride = 0;
  TileMover<T, C::BM, D> qr, gr;
  gr.init(tid, p.dout.st);
  float l_reg = 0.f, d_reg = 0.f;
  int l_row = 0;
  // In the instantiation with the slot-structured body, LDS holds -L / sm_scale and -delta per row:
  // the score and dP accumulators start from them, so that P = exp2(c2 (q.k - L / sm_scale)) and
  // dS = P (dO.v - delta) take one multiplication each in the slots.
  constexpr bool FOLDED = C::SLOTTED && !DROP;
  const float inv_scale = 1.f / p.sm_scale;
  auto fetch_stats = [&](int m0) {
    l_row = m0 + (tid & (C::BM - 1));
    const int mc = imin(l_row, M - 1);
    l_reg = lse[mc];
    d_reg = dlt[mc];
  };
  auto fetch = [&](int m0) {
    const int rows = M - m0;
    qr.fetch(q_src + (int64_t)m0 * q_stride, rows);
    gr.fetch(gb + (int64_t)m0 * p.dout.st, rows);
    // L and delta of row m0 + tid (threads 0..63), read branch-free from a clamped row and fixed up
    // at commit: nothing may consume a load here, or the wait would cover the tile loads as well
    fetch_stats(m0);
  };
  auto commit = [&](int stage) {
    unsigned char* base = smem + stage * C::STAGE_BYTES;
    T* s = (T*)base;
    qr.template commit<C::LD>(s);
    gr.template commit<C::LD>(s + C::TILE);
    float* f = (float*)(base + 2 * C::TILE * sizeof(T));
    // rows past M get L = +inf, hence P = 0
    if (tid < C::BM) {
      if constexpr (FOLDED) {  // what the accumulators of q.k and dO.v start from
        f[tid] = l_row < M ? -l_reg * inv_scale : -__builtin_inff();
        f[C::BM + tid] = l_row < M ? -d_reg : 0.f;
      } else {
        f[tid] = l_row < M ? l_reg * kLog2e : __builtin_inff();
        f[C::BM + tid] = l_row < M ? d_reg : 0.f;
      }
    }
  };

  const float c2 = p.sm_scale * kLog2e;
  const float rp = DROP ? 1.f / (1.f - p.dropout_p) : 1.f;
  uint64_t drop_col = 0;  // dropout counter of (query 0, my_n) of the current head

  // Result block (32 keys x D) of a wavefront: in the accumulators D runs along the lanes and the keys along the
  // registers, so a direct store would be 2 bytes per lane, 64 instructions per block.  The tiles in LDS are dead
  // by then: the wavefront rounds its block into a patch there and stores it from the patch as whole rows, 16
  // bytes per lane (8 instructions at head size 128).  Same values, same rounding.
  auto store_keys = [&](const f32x16* acc, const View4& dst, float scale) {
    constexpr int PLD = C::DV + 8;                       // elements per patch row: 16-byte multiples, rows 4 apart in distinct banks
    static_assert(4 * 32 * PLD * sizeof(T) <= C::LDS_BYTES && (PLD * sizeof(T)) % 16 == 0, "four patches fit the tile stages");
    T* patch = (T*)smem + wave * 32 * PLD;
    hw::block_sync();                                    // every wavefront has read the last operands of its last tile
#pragma unroll
    for (int db = 0; db < C::DV / 32; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) patch[block_row(r, hh) * PLD + db * 32 + l32] = (T)(acc[db][r] * scale);
    hw::wave_sync();
    T* base = (T*)dst.ptr + batch * dst.sb + slice * dst.sh;
    constexpr int CPR = C::DV / 8, RPI = 64 / CPR;       // 16-byte chunks per row, rows per store instruction
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
      const int row = i * RPI + lane / CPR, d0 = (lane % CPR) * 8;
      const int n = nw + row;
      if (n < N && d0 < D) *(u32x4*)(base + (int64_t)n * dst.st + d0) = *(const u32x4*)(patch + row * PLD + d0);
    }
    hw::block_sync();                                    // the patches are read out before a next pass writes tiles again
  };

  int stage = 0;
#pragma unroll 1
  for (int gi = 0; gi < chunk; ++gi) {
  head = slice * chunk + gi;
  gb = (const T*)p.dout.ptr + batch * p.dout.sb + head * p.dout.sh;
  lse = p.lse + ((int64_t)batch * p.H + head) * M;
  dlt = p.delta + ((int64_t)batch * p.H + head) * M;
  T* ds_near = nullptr;
  int64_t ds_regime_stride = 0;  // piecewise: the far regime's chunk grid follows the near regime's
  if (DS) {
    const int64_t nqb = 4 * (int64_t)cdiv(M, 128), nkb = 4 * (int64_t)cdiv(N, 128);
    ds_near = (T*)p.ds + ((((int64_t)batch * p.H + head) * nkb + (n0 / 32 + wave)) * nqb) * 1024 + lane * 8;
    ds_regime_stride = (int64_t)p.B * p.H * nkb * nqb * 1024;
    ds_row = ds_near;
  }
  if (DROP) drop_col = p.offset + ((uint64_t)batch * p.H + head) * M * (uint64_t)N + (uint64_t)(my_n < N ? my_n : 0);
#pragma unroll
  for (int ph = 0; ph < (PW ? 2 : 1); ++ph) {
    far_phase = PW && ph == 1;
    if (DS && PW) ds_row = ds_near + (far_phase ? ds_regime_stride : 0);
    // query tiles [t_begin, t_end) of 64 rows that hold an entry of this regime for some key of the block
    int t_begin = m_lo / C::BM, t_end = cdiv(M, C::BM);
    if (PW) {
      if (far_phase) t_begin = imax(t_begin, imax(0, n0 + p.w - pseq) / C::BM);
      else t_end = imin(t_end, cdiv(imax(0, imin(M, n0 + C::BN - 1 + p.w - pseq)), C::BM));
    }
    if (t_begin < t_end) {
      q_src = (const T*)(far_phase ? p.q2.ptr : p.q.ptr) + batch * (far_phase ? p.q2.sb : p.q.sb) +
              head * (far_phase ? p.q2.sh : p.q.sh);
      q_stride = far_phase ? p.q2.st : p.q.st;
      qr.init(tid, q_stride);
      if (far_phase) load_rows(kreg, (const T*)p.k2.ptr + batch * p.k2.sb + hk * p.k2.sh, p.k2.st);
      else load_rows(kreg, (const T*)p.k.ptr + batch * p.k.sb + hk * p.k.sh, p.k.st);
      fetch(t_begin * C::BM);
      commit(stage);
      hw::block_sync();
    }
    hw::wait_global_loads();  // K and V rows
    if constexpr (FOLDED) {
#pragma unroll
      for (int kk = 0; kk < C::KSTEPS; ++kk) { hw::keep_in_agprs(kreg[kk]); hw::keep_in_agprs(vreg[kk]); }
    }
    // the tile loop starts with the rows of the second tile on their way to registers: every tile
    // commits its successor to LDS and then requests the tile after that
    if (t_begin + 1 < t_end) fetch((t_begin + 1) * C::BM);

    // Tiles [plain_lo, plain_hi) are touched by no mask for this wavefront's 32 keys and run the slot-structured
    // body without selects (the same answer in every lane: kept in scalar registers, so that the loops below are
    // scalar loops).  A block with keys past N has no such tile: its P and dS must be exact zeroes for those keys
    // (K and V rows are zero, so the score is just -L and exp2 of it can be huge).
    int plain_lo = t_end, plain_hi = t_end;
    if (FOLDED && nw + 31 < N) {
      auto ceil64 = [](int a) { return (a + 63) >> 6; };   // also for negative a
      plain_lo = t_begin;
      // under the causal mask every row of the tile sees every key of the block: 64 it + pseq >= nw + 31
      if (p.causal) plain_lo = imax(plain_lo, ceil64(nw + 31 - pseq));
      // piecewise: every entry of the 64 x 32 tile belongs to this pass's regime --
      // far: 64 it + pseq - (nw + 31) >= w;  near: 64 it + 63 + pseq - nw < w
      if (PW && far_phase) plain_lo = imax(plain_lo, ceil64(p.w + nw + 31 - pseq));
      if (PW && !far_phase) plain_hi = imin(plain_hi, ceil64(p.w + nw - 63 - pseq));
      plain_lo = imin(plain_lo, t_end);
      plain_hi = imax(plain_hi, plain_lo);
    }
    plain_lo = hw::uniform(plain_lo);
    plain_hi = hw::uniform(plain_hi);
    // Registers of the slot-structured body that live from one tile into the next: the score and dP accumulators
    // of the two 32-query blocks and the ring of matrix operands read from LDS.  A tile's last slots already read
    // the next tile's first operands and the values its first accumulator starts from, so that the first matrix
    // instruction of a tile follows the last one of the tile before it without a trip to LDS in between.
    f32x16 sx[2], dpx[2];
    constexpr int kDepth = 4;
    V8 ring[kDepth];
    // operand of A-phase instruction j of block sb (rows of Q for j < KSTEPS, of dO behind) in the stage at `base`
    auto a_operand_in = [&](const unsigned char* base, int sb, int j) {
      const T* tq = (const T*)base;
      return operand_rowmajor<T, C::LD>(j < C::KSTEPS ? tq : tq + C::TILE, sb * 32, 16 * (j % C::KSTEPS), lane);
    };
    auto start_scores_in = [&](const unsigned char* base, int sb) {
      const float* tl = (const float*)(base + 2 * C::TILE * sizeof(T));
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const hw::f32x4 l4 = *(const hw::f32x4*)(tl + sb * 32 + 8 * g + 4 * hh);
#pragma unroll
        for (int e = 0; e < 4; ++e) sx[sb][4 * g + e] = l4[e];
      }
    };
    // what a slot-structured tile expects to find when it starts: block 0's score accumulator at its rows'
    // values and the first kDepth operands on their way (the first tile of a run; later ones get them from
    // their predecessor's last slots)
    auto preload = [&](int st) {
      const unsigned char* base = smem + st * C::STAGE_BYTES;
      start_scores_in(base, 0);
#pragma unroll
      for (int k = 0; k < kDepth; ++k) ring[k] = a_operand_in(base, 0, k);
    };
    // One query tile.  The bodies are separate instantiations, run from loops of their own (below): with
    // two inside one loop the compiler carries the flags that tell them apart through every iteration and
    // allocates registers for the union of the two.
    //   kPhases       S and dP, then the element-wise work, then dV and dK, one 32 x 32 block after the other; masks
    //                 by select, blocks that are masked as a whole skipped.  Every instantiation can run it.
    //   kSlotsPlain   the slot-structured body for tiles that no mask touches
    //   kSlotsMasked  the same slots with one select per element of P behind its exponential, for a mask that begins
    //                 inside the tile: rows from a per-lane bound on are kept (causal mask, keys past N); blocks
    //                 masked as a whole are computed and come out as zeroes
    //   kSlotsBand    likewise with two selects per element, for the regimes of piecewise attention: rows from one
    //                 per-lane bound up to another are kept
    constexpr int kPhases = 0, kSlotsPlain = 1, kSlotsMasked = 2, kSlotsBand = 3;
    // Per-lane bounds of those masks as rows counted from row 0 (the tile subtracts its m0), minus the 4 rows by
    // which the upper half of the lanes is ahead in every register: element (block sb, register r) is row
    // 32 sb + 8 (r / 4) + r % 4 + 4 hh.  first_seen_row: first row that sees key my_n under the causal mask;
    // first_far_row: first row whose distance to key my_n reaches the piecewise threshold.  A key past N is seen
    // by no row.
    constexpr int kNoRow = 1 << 29;
    const int first_seen_row = (my_n < N ? (p.causal ? my_n - pseq : -kNoRow) : kNoRow) - 4 * hh;
    const int first_far_row = PW ? my_n + imax(-kNoRow, imin(p.w, kNoRow)) - pseq - 4 * hh : 0;
    // rows [keep_from, keep_below) of this pass's regime: far = visible and at least the threshold away
    const int keep_from = (PW && far_phase) ? imax(first_far_row, first_seen_row) : first_seen_row;
    const int keep_below = (PW && !far_phase) ? first_far_row : kNoRow;
    auto tile = [&](auto kind_tag, int it) {
      constexpr int kind = decltype(kind_tag)::value;
      constexpr bool plain_tile = kind != kPhases;          // the slot-structured body
      constexpr bool select_in_slots = kind == kSlotsMasked || kind == kSlotsBand;
      const int m0 = it * C::BM;
      const bool more = it + 1 < t_end;

      const unsigned char* base = smem + stage * C::STAGE_BYTES;
      const T* sQ = (const T*)base;
      const T* sG = sQ + C::TILE;
      const float* sL = (const float*)(base + 2 * C::TILE * sizeof(T));
      const float* sDl = sL + C::BM;
      const int next_stage = stage + 1 == C::STAGES ? 0 : stage + 1;
      constexpr bool committed_in_slots = plain_tile, synced_in_slots = plain_tile, fetched_in_slots = plain_tile;

      // The slot-structured body.  Nothing else would issue under this wavefront's matrix instructions (the
      // launch bounds leave the kernel one wavefront per SIMD), so the element-wise work of one 32 x 32 block is
      // written BETWEEN the matrix instructions of the other, one element per matrix instruction at head size
      // 128 and two at head size 64, in the order
      //   A0 | A1 with E0 | C0 with E1 | C1      (A: S and dP, E: P and dS, C: dV and dK)
      // and a scheduling fence after every such slot keeps the compiler from regrouping them.
      if constexpr (plain_tile) {
      {
        constexpr int NA = 2 * C::KSTEPS;       // matrix instructions of an A phase (16 at head size 128, 8 at 64)
        constexpr int DB = C::DV / 32;          // 32-column blocks of dV and dK
        constexpr int NC = 4 * DB;              // matrix instructions of a C phase (16 / 8)
        static_assert(NA == NC && (NA == 16 || NA == 8), "a block's 16 elements per lane spread evenly over the slots of a phase");
        constexpr int kRate = 16 / NA;          // elements of a block per matrix instruction
        // operand of A-phase instruction j of block sb, and of C-phase instruction j
        auto a_operand = [&](int sb, int j) {
          return operand_rowmajor<T, C::LD>(j < C::KSTEPS ? sQ : sG, sb * 32, 16 * (j % C::KSTEPS), lane);
        };
        auto c_operand = [&](int sb, int j) {   // j = 2 DB c + DB which + db: per 16-query half c, DB products of dV, then DB of dK
          return operand_transposed<T, C::LD>(((j / DB) & 1) ? sQ : sG, sb * 32 + 16 * (j / (2 * DB)), (j % DB) * 32, lane);
        };
        auto a_issue = [&](int sb, int j, const V8& op) {
          if (j < C::KSTEPS) sx[sb] = hw::mfma32_vacc(op, kreg[j], sx[sb]);
          else dpx[sb] = hw::mfma32_vacc(op, vreg[j - C::KSTEPS], dpx[sb]);
        };
        // the tile's matrix instructions in issue order: A0, A1, C0, C1 (16 each at head size 128: slots 0-15, 16-31, 32-47, 48-63)
        constexpr int kSlots = 2 * NA + 2 * NC;
        auto operand = [&](int k) {
          if (k < NA) return a_operand(0, k);
          if (k < 2 * NA) return a_operand(1, k - NA);
          if (k < 2 * NA + NC) return c_operand(0, k - 2 * NA);
          return c_operand(1, k - 2 * NA - NC);
        };
        // accumulators start from the per-row values
        auto start_scores = [&](int sb) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const hw::f32x4 l4 = *(const hw::f32x4*)(sL + sb * 32 + 8 * g + 4 * hh);
#pragma unroll
            for (int e = 0; e < 4; ++e) sx[sb][4 * g + e] = l4[e];
          }
        };
        auto start_dp = [&](int sb) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const hw::f32x4 d4 = *(const hw::f32x4*)(sDl + sb * 32 + 8 * g + 4 * hh);
#pragma unroll
            for (int e = 0; e < 4; ++e) dpx[sb][4 * g + e] = d4[e];
          }
        };
        // element r of a block in two steps, each as early as its inputs exist, so that the element-wise
        // work spreads over as many slots as the data dependencies allow: p = exp2(c s) of block 0 from
        // the slot after its S chain ended (kP0), dS = p dP eight slots behind it, block 1 likewise a
        // phase later.  The multiplications and exponentials are assembly statements that stay in their
        // slot (left to the compiler they drift towards the matrix instruction that produced their input,
        // closer than the hardware allows); step t multiplies element t, exponentiates element t - 1 and
        // packs the pair that was complete a step ago, so that nothing reads an exponential in the slot
        // that issued it.
        u32x4 pa[2][2], da[2][2];   // [block][half of its 16 elements]: 8 values rounded to T, the A operand of a C-phase product
        float pr[2][16];
        float p_arg[2] = {0.f, 0.f};
        // the rows of this tile at which this lane's mask begins and (kSlotsBand) ends
        const int mask_row = keep_from - m0, mask_end = keep_below - m0;
        auto elem_p = [&](auto sb_tag, auto t_tag) {   // t = 0 .. 17
          constexpr int sb = decltype(sb_tag)::value, t = decltype(t_tag)::value;
          if constexpr (select_in_slots && t >= 2) {   // element t - 2, exponentiated a step ago, before its pair is packed
            constexpr int r = t - 2;
            pr[sb][r] = hw::slot_keep_if_at_least<32 * sb + 8 * (r / 4) + r % 4>(pr[sb][r], mask_row);
            if constexpr (kind == kSlotsBand) pr[sb][r] = hw::slot_keep_if_below<32 * sb + 8 * (r / 4) + r % 4>(pr[sb][r], mask_end);
          }
          if (t >= 3 && (t & 1)) {
            const int r = t - 2;             // pair (r - 1, r), r odd
            pa[sb][r >> 3][(r & 7) >> 1] = hw::slot_pack2(T{}, pr[sb][r - 1], pr[sb][r]);
          }
          if (t >= 1 && t <= 16) pr[sb][t - 1] = hw::slot_exp2(p_arg[sb]);
          if (t <= 15) p_arg[sb] = hw::slot_mul(sx[sb][t], c2);
        };
        float dsr[2][16];
        auto elem_ds = [&](int sb, int t) {   // t = 0 .. 16: multiplies element t, packs the pair finished a step ago
          if (t >= 2 && !(t & 1)) {
            const int r = t - 1;             // pair (r - 1, r), r odd
            da[sb][r >> 3][(r & 7) >> 1] = hw::slot_pack2(T{}, dsr[sb][r - 1], dsr[sb][r]);
          }
          if (t <= 15) dsr[sb][t] = hw::slot_mul(pr[sb][t], dpx[sb][t]);
        };
        constexpr int kP0 = C::KSTEPS + 1, kD0 = NA + 1, kP1 = NA + C::KSTEPS + 1, kD1 = 2 * NA + 1;
        // hw::mfma32_vacc hides its result registers from the compiler's hazard handling, so the slot
        // order itself has to keep a vector-ALU read of sx / dpx behind the matrix instruction that
        // wrote them last.  A 32x32x16 product occupies the matrix pipe for 8 passes of 4 cycles and its
        // result may be read 12 wait states (the passes plus 4) after its issue; a slot issues its matrix
        // instruction first and its element-wise work after it.  If the chain's last product sits in
        // slot w, the product of slot w + 1 cannot issue before w has left the pipe's front and the
        // product of slot w + 2 cannot issue before w has written back, so element-wise work of slot
        // r >= w + 2 reads finished registers: one whole other matrix instruction lies in between.
        constexpr int kLastS0 = C::KSTEPS - 1, kLastDp0 = NA - 1, kLastS1 = NA + C::KSTEPS - 1, kLastDp1 = 2 * NA - 1;
        constexpr int kHazardSlots = 2;
        static_assert(kP0 >= kLastS0 + kHazardSlots, "exp2 of block 0 reads S before its last product has written back");
        static_assert(kD0 >= kLastDp0 + kHazardSlots, "dS of block 0 reads dP before its last product has written back");
        static_assert(kP1 >= kLastS1 + kHazardSlots, "exp2 of block 1 reads S before its last product has written back");
        static_assert(kD1 >= kLastDp1 + kHazardSlots, "dS of block 1 reads dP before its last product has written back");
        // A slot runs kRate steps of each element stream that is active in it, the dS streams before the P streams.
        // Element r of P is final after step r + 2 of its stream (exponential in step r + 1, select in r + 2);
        // dS of element r is step r of the dS stream.
        constexpr auto slot_of = [](int first_slot, int step) constexpr { return first_slot + step / kRate; };
        static_assert(slot_of(kD0, 0) > slot_of(kP0, 2) && slot_of(kD0, 15) > slot_of(kP0, 17) &&
                      slot_of(kD1, 0) > slot_of(kP1, 2) && slot_of(kD1, 15) > slot_of(kP1, 17),
                      "dS = p * dP reads p of the same element in a later slot than the one that finished it");
        // operands are packed in pairs as soon as their second element exists (half c of P complete in step 8 c + 9,
        // of dS in step 8 c + 8); half c of block sb feeds C-phase slots 2 DB c .. (dV) and 2 DB c + DB .. (dK), and
        // the first of them also stores the half block of dS
        constexpr auto first_dv_slot = [](int sb, int c) constexpr { return 2 * NA + sb * NC + 2 * DB * c; };
        static_assert(slot_of(kP0, 9) < first_dv_slot(0, 0) && slot_of(kP0, 17) < first_dv_slot(0, 1) &&
                      slot_of(kP1, 9) < first_dv_slot(1, 0) && slot_of(kP1, 17) < first_dv_slot(1, 1),
                      "P is packed before dV takes it");
        static_assert(slot_of(kD0, 8) < first_dv_slot(0, 0) && slot_of(kD0, 16) < first_dv_slot(0, 1) &&
                      slot_of(kD1, 8) < first_dv_slot(1, 0) && slot_of(kD1, 16) < first_dv_slot(1, 1),
                      "a half block of dS is packed before the slot that stores it (dK takes it DB slots later)");
        // the accumulators of block 1 are re-initialised while block 1's own chains have not started (S: slots NA ..,
        // dP: NA + KSTEPS ..) and after the tile before has read them for the last time (its slots up to
        // slot_of(kP1, 15) and slot_of(kD1, 15)); block 0's likewise (start_dp(0) in slot 1, the scores in the
        // tile before)
        constexpr int kStartS1 = NA - 6, kStartDp1 = NA == 16 ? NA + 2 : 4;
        static_assert(kStartS1 >= 0 && kStartS1 < NA - 2 && kStartDp1 < NA + C::KSTEPS - 1 && 1 < C::KSTEPS - 1,
                      "a block starts from its rows' values before its chains run");
        static_assert(slot_of(kP1, 17) < 2 * NA + 2 * NC && slot_of(kD1, 16) < 2 * NA + 2 * NC,
                      "every element stream ends inside the tile");

        // The next tile's rows (in registers since the previous tile) go to the next stage during the
        // C1 slots, the workgroup's barrier follows them there, and the loads of the tile after the
        // next take over the registers one slot after they are free: nothing but the loop edge stands
        // between this tile's last matrix instruction and the next tile's first.  All of it is
        // unconditional, because a branch would end the basic block whose order the fences keep: past
        // the last tile the writes store stale registers into a stage that nobody reads before its
        // next commit, and the loads fetch the last tile once more.  Rows past M hold copies of row
        // M - 1 instead of commit()'s zeroes: their P and dS are exact zeroes (L = +inf), and row M - 1
        // itself is in the same products.
        constexpr int kPasses = TileMover<T, C::BM, D>::PASSES;
        // (head size 64 has 8 slots per phase: there the hand-over starts with C0, so that the barrier is passed
        // before the last kDepth slots, which read the next tile's first operands)
        constexpr int kCommitSlot = NA == 16 ? 2 * NA + NC : 2 * NA, kSyncSlot = kCommitSlot + 2 * kPasses + 1;
        constexpr int kFetchSlot = kCommitSlot + kPasses;   // Q registers are free from here on
        static_assert(TileMover<T, C::BM, D>::kExact && kFetchSlot + 2 * kPasses < kSlots, "fits the tile's last slots");
        const int m_ahead = imin(it + 2, t_end - 1) * C::BM;
        const T* q_ahead = q_src + (int64_t)m_ahead * q_stride;
        const T* g_ahead = gb + (int64_t)m_ahead * p.dout.st;
        T* nQ = (T*)(smem + next_stage * C::STAGE_BYTES);
        T* nG = nQ + C::TILE;
        float* nf = (float*)(nG + C::TILE);

        // slots in which the tile's tail reads for its successor: the successor's stage is complete behind the
        // barrier of slot kSyncSlot; block 0's score accumulator has been free since its last element (kP0 + 15)
        constexpr int kNextScoresSlot = kSyncSlot + 1, kNextRingSlot = kSlots - kDepth;
        static_assert(kNextScoresSlot > slot_of(kP0, 15) && kNextScoresSlot < kSlots && kNextRingSlot > kSyncSlot,
                      "the next tile's first reads follow the barrier and find their registers free");
        const unsigned char* next_base = smem + next_stage * C::STAGE_BYTES;
        // LDS accesses a slot issues: the reads of the operand kDepth slots ahead (one 16-byte read for an A-phase
        // operand, also the successor's; two transposing reads for a C-phase operand) and whatever else is
        // placed in it (sl < 0: a slot of the tile before)
        auto lds_accesses_of = [](int sl) constexpr {
          if (sl < 0) sl += kSlots;
          const int ahead = sl + kDepth;
          int n = (ahead >= 2 * NA && ahead < kSlots) ? 2 : 1;
          if (sl == 1 || sl == kStartS1 || sl == kStartDp1 || sl == kNextScoresSlot) n += 4;   // per-row starting values
          if (sl >= kCommitSlot && sl <= kCommitSlot + 2 * kPasses) n += 1;              // the successor's rows
          return n;
        };
        hw::sched_fence();
        static_for<kSlots>([&](auto slot) {
          constexpr int k = decltype(slot)::value;
          // one wait per pair of slots: an even slot waits for its own operand and for the next slot's, i.e. until
          // only the accesses of the last two slots are outstanding, and the odd slot finds its operand complete
          if constexpr ((k & 1) == 0) {
            hw::wait_lds_pending<lds_accesses_of(k - 2) + lds_accesses_of(k - 1)>();
            hw::sched_fence();   // or the scheduler lifts the matrix instruction over the wait and the compiler adds one of its own
          }
          const V8 op = ring[k % kDepth];
          if constexpr (k < 2 * NA) {
            a_issue(k / NA, k % NA, op);
          } else {
            constexpr int sb = (k - 2 * NA) / NC, j = (k - 2 * NA) % NC, c = j / (2 * DB), db = j % DB;
            if constexpr (((j / DB) & 1) != 0) dk[db] = hw::mfma32(hw::as_v8<T>(da[sb][c]), op, dk[db]);
            else dv[db] = hw::mfma32(hw::as_v8<T>(pa[sb][c]), op, dv[db]);
            if (DS && (j % (2 * DB)) == 0)
              hw::store_streaming(ds_row + (int64_t)(m0 / 32 + sb) * 1024 + c * 512,
                                  da[sb][c]);
          }
          if constexpr (k + kDepth < kSlots) ring[k % kDepth] = operand(k + kDepth);
          else ring[k % kDepth] = a_operand_in(next_base, 0, k + kDepth - kSlots);   // the successor's first operands
          if constexpr (k == 1) start_dp(0);            // needed by slot KSTEPS
          if constexpr (k == kNextScoresSlot) start_scores_in(next_base, 0);
          if constexpr (k == kStartS1) start_scores(1);
          if constexpr (k == kStartDp1) start_dp(1);
          static_for<kRate>([&](auto sub) {
            constexpr int t0 = (k - kD0) * kRate + decltype(sub)::value, t1 = (k - kD1) * kRate + decltype(sub)::value;
            if constexpr (k >= kD0 && t0 < 17) elem_ds(0, t0);
            if constexpr (k >= kD1 && t1 < 17) elem_ds(1, t1);
          });
          static_for<kRate>([&](auto sub) {
            constexpr int t0 = (k - kP0) * kRate + decltype(sub)::value, t1 = (k - kP1) * kRate + decltype(sub)::value;
            if constexpr (k >= kP0 && t0 < 18) elem_p(std::integral_constant<int, 0>{}, std::integral_constant<int, (k >= kP0 ? t0 : 0)>{});
            if constexpr (k >= kP1 && t1 < 18) elem_p(std::integral_constant<int, 1>{}, std::integral_constant<int, (k >= kP1 ? t1 : 0)>{});
          });
          if constexpr (k >= kCommitSlot && k < kCommitSlot + kPasses)
            qr.template commit_pass<C::LD>(nQ, k - kCommitSlot);
          if constexpr (k >= kCommitSlot + kPasses && k < kCommitSlot + 2 * kPasses)
            gr.template commit_pass<C::LD>(nG, k - kCommitSlot - kPasses);
          if constexpr (k == kCommitSlot + 2 * kPasses) {  // every wavefront writes the same 64 + 64 values
            nf[tid & (C::BM - 1)] = l_row < M ? -l_reg * inv_scale : -__builtin_inff();
            nf[C::BM + (tid & (C::BM - 1))] = l_row < M ? -d_reg : 0.f;
          }
          if constexpr (k == kSyncSlot) hw::block_sync();
          if constexpr (k == kFetchSlot) { qr.fetch_begin(M - m_ahead); gr.fetch_begin(M - m_ahead); }
          if constexpr (k >= kFetchSlot && k < kFetchSlot + kPasses) qr.fetch_pass(q_ahead, k - kFetchSlot);
          if constexpr (k >= kFetchSlot + kPasses && k < kFetchSlot + 2 * kPasses)
            gr.fetch_pass(g_ahead, k - kFetchSlot - kPasses);
          if constexpr (k == kFetchSlot + 2 * kPasses) fetch_stats(m_ahead);
          hw::sched_fence();
        });
      }
      }
      if constexpr (!plain_tile) {
#pragma unroll
      for (int sb = 0; sb < C::BM / 32; ++sb) {
        const int mr0 = m0 + sb * 32;
        // every (m, n) of this 32 x 32 block is masked, or belongs to the other regime: nothing to add
        if (p.causal && (mr0 + 31 + pseq < nw)) continue;
        if (PW && (far_phase ? (mr0 + 31 + pseq - nw < p.w) : (mr0 + pseq - (nw + 31) >= p.w))) continue;
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < C::KSTEPS; ++kk)
          s = hw::mfma32(operand_rowmajor<T, C::LD>(sQ, sb * 32, 16 * kk, lane), kreg[kk], s);
#pragma unroll
        for (int kk = 0; kk < C::KSTEPS; ++kk)
          dp = hw::mfma32(operand_rowmajor<T, C::LD>(sG, sb * 32, 16 * kk, lane), vreg[kk], dp);
        hw::sched_prefetched_operands<2 * C::KSTEPS, (C::KSTEPS >= 8 ? 8 : 2)>();

        bool need_mask = (nw + 31 >= N) || (p.causal && (mr0 + pseq < nw + 31));
        if (PW) need_mask = need_mask || (far_phase ? (mr0 + pseq - (nw + 31) < p.w) : (mr0 + 31 + pseq - nw >= p.w));
        // L * log2e and delta of this lane's 16 query rows: rows 8g + 4h + 0..3 are contiguous
        hw::f32x4 lrow[4], drow[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          lrow[g] = *(const hw::f32x4*)(sL + sb * 32 + 8 * g + 4 * hh);
          drow[g] = *(const hw::f32x4*)(sDl + sb * 32 + 8 * g + 4 * hh);
        }
        f32x16 pr, ds;
        if (need_mask) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = mr0 + block_row(r, hh);
            bool keep = (my_n < N) && (!p.causal || (m + pseq >= my_n));
            if (PW) keep = keep && ((m + pseq - my_n >= p.w) == far_phase);
            float pv = FOLDED ? hw::exp2_fast((s[r] + lrow[r >> 2][r & 3]) * c2)
                              : hw::exp2_fast(fmaf(s[r], c2, -lrow[r >> 2][r & 3]));
            pv = keep ? pv : 0.f;
            float pd = pv, dpv = dp[r];
            if (DROP) {
              const bool kd = dropout_keeps(drop_col + (uint64_t)m * N, p.seed, p.dropout_p);
              pd = kd ? pv : 0.f;
              dpv = kd ? dp[r] * rp : 0.f;
            }
            pr[r] = pd;
            ds[r] = FOLDED ? pv * (dpv + drow[r >> 2][r & 3]) : pv * (dpv - drow[r >> 2][r & 3]);
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float pv = FOLDED ? hw::exp2_fast((s[r] + lrow[r >> 2][r & 3]) * c2)
                                    : hw::exp2_fast(fmaf(s[r], c2, -lrow[r >> 2][r & 3]));
            float pd = pv, dpv = dp[r];
            if (DROP) {
              const bool kd = dropout_keeps(drop_col + (uint64_t)(mr0 + block_row(r, hh)) * N, p.seed, p.dropout_p);
              pd = kd ? pv : 0.f;
              dpv = kd ? dp[r] * rp : 0.f;
            }
            pr[r] = pd;
            ds[r] = FOLDED ? pv * (dpv + drow[r >> 2][r & 3]) : pv * (dpv - drow[r >> 2][r & 3]);
          }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          V8 pa = pack_half_block<T>(pr, c);
#pragma unroll
          for (int db = 0; db < C::DV / 32; ++db)
            dv[db] = hw::mfma32(pa, operand_transposed<T, C::LD>(sG, sb * 32 + 16 * c, db * 32, lane), dv[db]);
          V8 da = pack_half_block<T>(ds, c);
          if (DS) hw::store_streaming(ds_row + (int64_t)(mr0 / 32) * 1024 + c * 512, __builtin_bit_cast(u32x4, da));
#pragma unroll
          for (int db = 0; db < C::DV / 32; ++db)
            dk[db] = hw::mfma32(da, operand_transposed<T, C::LD>(sQ, sb * 32 + 16 * c, db * 32, lane), dk[db]);
        }
        // each of these products takes an operand made of two transposing reads
        hw::sched_prefetched_operands<4 * (C::DV / 32), (C::DV >= 128 ? 5 : 1), 2>();
      }
      }

      if constexpr (!committed_in_slots) { if (more) commit(next_stage); }
      if constexpr (!synced_in_slots) hw::block_sync();
      if constexpr (!fetched_in_slots) { if (it + 2 < t_end) fetch(m0 + 2 * C::BM); }
      stage = next_stage;
    };
    using Phases = std::integral_constant<int, kPhases>;
    using SlotsPlain = std::integral_constant<int, kSlotsPlain>;
    using SlotsMasked = std::integral_constant<int, kSlotsMasked>;
    using SlotsBand = std::integral_constant<int, kSlotsBand>;
    if constexpr (FOLDED) {   // every tile in slots; the ones a mask crosses (before and behind the plain range) with selects
      using Crossed = std::conditional_t<PW, SlotsBand, SlotsMasked>;
      int it = t_begin;
      if (it < t_end) preload(stage);
#pragma unroll 1
      for (; it < plain_lo; ++it) tile(Crossed{}, it);
#pragma unroll 1
      for (; it < plain_hi; ++it) tile(SlotsPlain{}, it);
      if constexpr (PW) {   // (without regimes the plain range runs to the end)
#pragma unroll 1
        for (; it < t_end; ++it) tile(Crossed{}, it);
      }
    } else {
#pragma unroll 1
      for (int it = t_begin; it < t_end; ++it) tile(Phases{}, it);
    }

    if (PW) {  // this regime's dK is complete (piecewise has no grouped heads)
      store_keys(dk, far_phase ? p.dk2 : p.dk, p.sm_scale);
      if (!far_phase) {
#pragma unroll
        for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) dk[i][r] = 0.f;
      }
    }
  }
  }
  if (!PW) store_keys(dk, p.dk, p.sm_scale);
  store_keys(dv, p.dv, rp);
}

// ----------------------------------------------------------------------------------- dQ ----
template <class T, int D, bool PW>
struct QCfg {
  static constexpr int BM = 128;  // queries per workgroup (32 per wavefront)
  static constexpr int BN = 64;   // keys per pipeline step
  static constexpr int DV = D < 32 ? 32 : D;
  static constexpr int KSTEPS = D / 16;
  static constexpr int LD = DV + (DV == 128 ? 24 : 40);  // 16-byte row reads and transposing reads both conflict-free
  static constexpr int TILE = BN * LD;
  static constexpr int WAVES_PER_SIMD = 2;
  static constexpr size_t STAGE_BYTES = 2 * TILE * sizeof(T);  // K, V
  static constexpr size_t LDS_BYTES = 2 * STAGE_BYTES;
};

// PW: two passes over the key tiles, as in the forward kernel -- the far keys with (q2, k2)
// accumulating dQ2, then the near keys with (q1, k1) accumulating dQ1 in the same registers.
// DROP: dP is masked and scaled by 1 / (1 - dropout_p) before dS = P (dP - delta) (flash.py:877-890).
template <class T, int D, bool PW, bool DROP = false>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, (QCfg<T, D, PW>::WAVES_PER_SIMD)) fa_bwd_dq_kernel(BwdParams p) {
  static_assert(!(PW && DROP), "piecewise attention has no dropout");
  using C = QCfg<T, D, PW>;
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

  const T* gb = (const T*)p.dout.ptr + batch * p.dout.sb + head * p.dout.sh;
  const T* vb = (const T*)p.v.ptr + batch * p.v.sb + hk * p.v.sh;

  // Q (of the current regime) and dO rows of this lane as B operands
  V8 qreg[C::KSTEPS], greg[C::KSTEPS];
  auto load_rows = [&](V8* dst, const T* base, int64_t row_stride) {
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk) {
      u32x4 a = {0u, 0u, 0u, 0u};
      if (my_m < M) a = *(const u32x4*)(base + (int64_t)my_m * row_stride + 16 * kk + 8 * hh);
      dst[kk] = hw::as_v8<T>(a);
    }
  };
  load_rows(greg, gb, p.dout.st);
  // rows past M get L = +inf, hence P = 0
  const int64_t row_off = ((int64_t)batch * p.H + head) * M + my_m;
  const float l_row = my_m < M ? p.lse[row_off] * kLog2e : __builtin_inff();
  const float d_row = my_m < M ? p.delta[row_off] : 0.f;
  const float rp = DROP ? 1.f / (1.f - p.dropout_p) : 1.f;
  // dropout counter of (my_m, key 0)
  const uint64_t drop_row = DROP ? p.offset + (((uint64_t)batch * p.H + head) * M + (uint64_t)(my_m < M ? my_m : 0)) * N : 0;

  int hi = N;
  if (p.causal) hi = imin(N, pseq + m0 + C::BM);
  const int n_tiles = hi > 0 ? cdiv(hi, C::BN) : 0;

  if (C::DV != D) {
    for (int i = tid; i < (int)(C::LDS_BYTES / sizeof(T)); i += kThreads) lds[i] = (T)0.f;
    hw::block_sync();
  }

  f32x16 dq[C::DV / 32];
#pragma unroll
  for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[i][r] = 0.f;

  bool far_phase = false;
  const T* k_src = nullptr;
  int64_t k_stride = 0;
  TileMover<T, C::BN, D> kr, vr;
  vr.init(tid, p.v.st);
  auto fetch = [&](int n0) {
    const int rows = N - n0;
    kr.fetch(k_src + (int64_t)n0 * k_stride, rows);
    vr.fetch(vb + (int64_t)n0 * p.v.st, rows);
  };
  auto commit = [&](int stage) {
    T* s = (T*)(smem + stage * C::STAGE_BYTES);
    kr.template commit<C::LD>(s);
    vr.template commit<C::LD>(s + C::TILE);
  };

  const float c2 = p.sm_scale * kLog2e;

  // dQ^T blocks: lane owns one query row, registers run along D
  auto store_rows = [&](const View4& dst) {
    if (my_m < M) {
      T* o1 = (T*)dst.ptr + batch * dst.sb + head * dst.sh + (int64_t)my_m * dst.st;
#pragma unroll
      for (int db = 0; db < C::DV / 32; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          int d = db * 32 + 8 * g + 4 * hh;
          if (d < D) {
            hw::u32x2 w;
            w[0] = (uint32_t)hw::bits16<T>(dq[db][4 * g + 0] * p.sm_scale) | ((uint32_t)hw::bits16<T>(dq[db][4 * g + 1] * p.sm_scale) << 16);
            w[1] = (uint32_t)hw::bits16<T>(dq[db][4 * g + 2] * p.sm_scale) | ((uint32_t)hw::bits16<T>(dq[db][4 * g + 3] * p.sm_scale) << 16);
            *(hw::u32x2*)(o1 + d) = w;
          }
        }
    }
  };

  int stage = 0;
#pragma unroll 1
  for (int ph = 0; ph < (PW ? 2 : 1); ++ph) {
    far_phase = PW && ph == 0;
    int t_begin = 0, t_end = n_tiles;
    if (PW) {
      if (far_phase) {
        const int far_hi = imin(hi, m0 + C::BM + pseq - p.w);
        t_end = far_hi > 0 ? cdiv(far_hi, C::BN) : 0;
      } else {
        t_begin = imax(0, m0 + pseq - p.w + 1) / C::BN;
      }
    }
    if (t_begin < t_end) {
      k_src = (const T*)(far_phase ? p.k2.ptr : p.k.ptr) + batch * (far_phase ? p.k2.sb : p.k.sb) +
              hk * (far_phase ? p.k2.sh : p.k.sh);
      k_stride = far_phase ? p.k2.st : p.k.st;
      kr.init(tid, k_stride);
      if (far_phase) load_rows(qreg, (const T*)p.q2.ptr + batch * p.q2.sb + head * p.q2.sh, p.q2.st);
      else load_rows(qreg, (const T*)p.q.ptr + batch * p.q.sb + head * p.q.sh, p.q.st);
      fetch(t_begin * C::BN);
      commit(stage);
      hw::block_sync();
    }
    hw::wait_global_loads();  // Q and dO rows

    // One key tile.  `plain`: no mask touches the tile for any row of this wavefront (and there is no dropout or
    // second regime), so the body has no branch and the compiler may run the element-wise work of one 32-key block
    // under the matrix instructions of the other.  The two variants run in loops of their own.
    auto tile = [&](auto plain_tag, int it) {
      constexpr bool plain = decltype(plain_tag)::value;
      const int n0 = it * C::BN;
      const bool more = it + 1 < t_end;
      if (more) fetch(n0 + C::BN);

      const T* sK = (const T*)(smem + stage * C::STAGE_BYTES);
      const T* sV = sK + C::TILE;

#pragma unroll
      for (int nb = 0; nb < C::BN / 32; ++nb) {
        const int nlo = n0 + nb * 32;
        if constexpr (!plain) {
          if (p.causal && (mw + 31 + pseq < nlo)) continue;  // block fully masked for this wavefront
          if (PW && (far_phase ? (mw + 31 + pseq - nlo < p.w) : (mw + pseq - (nlo + 31) >= p.w))) continue;
        }
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < C::KSTEPS; ++kk)
          s = hw::mfma32(operand_rowmajor<T, C::LD>(sK, nb * 32, 16 * kk, lane), qreg[kk], s);
#pragma unroll
        for (int kk = 0; kk < C::KSTEPS; ++kk)
          dp = hw::mfma32(operand_rowmajor<T, C::LD>(sV, nb * 32, 16 * kk, lane), greg[kk], dp);
        hw::sched_prefetched_operands<2 * C::KSTEPS, (C::KSTEPS >= 4 ? 4 : 2)>();

        bool need_mask = !plain && ((nlo + 32 > N) || (p.causal && (nlo + 31 > pseq + mw)));
        if (PW) need_mask = need_mask || (far_phase ? (mw + pseq - (nlo + 31) < p.w) : (mw + 31 + pseq - nlo >= p.w));
        f32x16 ds;
        if (need_mask) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int n = nlo + block_row(r, hh);
            bool keep = (n < N) && (!p.causal || (my_m + pseq >= n));
            if (PW) keep = keep && ((my_m + pseq - n >= p.w) == far_phase);
            float pv = hw::exp2_fast(fmaf(s[r], c2, -l_row));
            pv = keep ? pv : 0.f;
            float dpv = dp[r];
            if (DROP) dpv = dropout_keeps(drop_row + (uint64_t)n, p.seed, p.dropout_p) ? dp[r] * rp : 0.f;
            ds[r] = pv * (dpv - d_row);
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float dpv = dp[r];
            if (DROP)
              dpv = dropout_keeps(drop_row + (uint64_t)(nlo + block_row(r, hh)), p.seed, p.dropout_p) ? dp[r] * rp : 0.f;
            ds[r] = hw::exp2_fast(fmaf(s[r], c2, -l_row)) * (dpv - d_row);
          }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          V8 db_ = pack_half_block<T>(ds, c);
#pragma unroll
          for (int db = 0; db < C::DV / 32; ++db)
            dq[db] = hw::mfma32(operand_transposed<T, C::LD>(sK, nb * 32 + 16 * c, db * 32, lane), db_, dq[db]);
        }
      }

      if (more) commit(stage ^ 1);
      hw::block_sync();
      stage ^= 1;
    };
    {
      int it = t_begin;
      if constexpr (!PW && !DROP) {
        // tiles whose 64 keys exist and are visible to the wavefront's first row
        int plain_end = imin(t_end, N / C::BN);
        if (p.causal) plain_end = imin(plain_end, imax(0, mw + pseq + 1) / C::BN);
        plain_end = hw::uniform(plain_end);
#pragma unroll 1
        for (; it < plain_end; ++it) tile(std::true_type{}, it);
      }
#pragma unroll 1
      for (; it < t_end; ++it) tile(std::false_type{}, it);
    }

    store_rows((PW && far_phase) ? p.dq2 : p.dq);
    if (PW && far_phase) {
#pragma unroll
      for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq[i][r] = 0.f;
    }
  }
}

// --------------------------------------------------------------------------- dQ from dS ----
// dQ = scale * dS K with dS read back from the workspace the dK/dV kernel left (see there for the
// chunk format) instead of being recomputed: one product instead of three and no exponentials,
// paid for with one write and one read of the B x H x M x N matrix in T -- a trade that HBM3E
// bandwidth makes worthwhile.  The kernel is bound by that read.
//
// A wavefront owns 32 queries and walks the keys in steps of 64.  Its own dS chunks (2 per step) go
// through a private LDS patch verbatim; the transposing read then hands lane (query, h) the keys
// t0 + 4h + 0..3 and t0 + 8 + 4h + 0..3 of a 16-key slice, the order in which the K^T operand
// (operand_transposed) lists them.  In the patch the two halves of a chunk vector (lanes 0..31 and
// 32..63 of the writer) are 64 bytes further apart than in memory, which keeps the 16 lanes of a
// transposing read in distinct banks.
template <class T, int D>
struct QdsCfg {
  static constexpr int BM = 128, BN = 64;
  static constexpr int DV = D < 32 ? 32 : D;
  // the K tile is only read through transposing reads: at head size 128, 64 B of padding keep the 4 rows x 2 halves
  // that 32 lanes touch in disjoint banks (with the 48 B of the other backward tiles the two halves collide)
  static constexpr int LD = DV + (DV == 128 ? 32 : 40);
  static constexpr int TILE = BN * LD;                 // K tile, elements
  static constexpr int VEC = 512 + 32 + 32;            // one chunk vector in the patch: 2 x (256 + 32 pad) elements
  static constexpr int PATCH = 2 * 2 * VEC;            // 2 chunks x 2 vectors per wavefront and stage
  static constexpr size_t STAGE_BYTES = (TILE + 4 * PATCH) * sizeof(T);
  static constexpr size_t LDS_BYTES = 2 * STAGE_BYTES;
};

template <class T, int D, bool PW = false>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, 2) fa_bwd_dq_from_ds_kernel(BwdParams p) {
  using C = QdsCfg<T, D>;
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
  const bool live = mw < M;  // wavefront has at least one query row

  const T* kb = (const T*)p.k.ptr + batch * p.k.sb + hk * p.k.sh;
  const int64_t nqb = 4 * (int64_t)cdiv(M, 128), nkb = 4 * (int64_t)cdiv(N, 128);
  // chunk (key block 0, this wavefront's query block); a key block further is nqb chunks further
  const bool far = PW && p.regime == 2;
  const T* ds_col = (const T*)p.ds + ((((int64_t)batch * p.H + head) * nkb) * nqb + mw / 32) * 1024 + lane * 8;
  if (far) ds_col += (int64_t)p.B * p.H * nkb * nqb * 1024;

  // key tiles that hold an entry of this launch's regime for some row of the block
  int lo = 0, hi = N;
  if (p.causal) hi = imin(N, pseq + m0 + C::BM);
  if (PW) {
    if (far) hi = imin(hi, m0 + C::BM - 1 + pseq - p.w + 1);  // far: n <= m + pseq - w
    else lo = imax(0, m0 + pseq - p.w + 1);                    // near: n > m + pseq - w
  }
  const int t_lo = lo / C::BN;
  const int n_tiles = hi > lo ? cdiv(hi, C::BN) : t_lo;

  if (C::DV != D) {
    for (int i = tid; i < (int)(C::LDS_BYTES / sizeof(T)); i += kThreads) lds[i] = (T)0.f;
    hw::block_sync();
  }

  f32x16 dq[C::DV / 32];
#pragma unroll
  for (int i = 0; i < C::DV / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[i][r] = 0.f;

  // a 32-key block contributes unless the mask hides all of it from this wavefront's rows
  // (the same conditions under which the dK/dV kernel computed, and stored, the block)
  auto block_used = [&](int nlo) {
    bool used = live && !(p.causal && (mw + 31 + pseq < nlo));
    if (PW) used = used && !(far ? (mw + 31 + pseq - nlo < p.w) : (mw + pseq - (nlo + 31) >= p.w));
    return used;
  };

  TileMover<T, C::BN, D> kr;
  kr.init(tid, p.k.st);
  u32x4 dsr[2][2];
  auto fetch = [&](int n0) {
    kr.fetch(kb + (int64_t)n0 * p.k.st, N - n0);
    // unconditional: chunks the mask hides were never written, are in bounds, and are not used below
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const T* chunk = ds_col + (int64_t)(n0 / 32 + nb) * nqb * 1024;
      dsr[nb][0] = hw::load_streaming(chunk);
      dsr[nb][1] = hw::load_streaming(chunk + 512);
    }
  };
  // patch position of what writer lane l (= this lane) stored: half l / 32 starts 288 elements on
  const int patch_off = l32 * 8 + hh * (256 + 32);
  auto commit = [&](int stage) {
    T* s = (T*)(smem + stage * C::STAGE_BYTES);
    kr.template commit<C::LD>(s);
    T* patch = s + C::TILE + wave * C::PATCH;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      *(u32x4*)(patch + (2 * nb + 0) * C::VEC + patch_off) = dsr[nb][0];
      *(u32x4*)(patch + (2 * nb + 1) * C::VEC + patch_off) = dsr[nb][1];
    }
  };
  // Supplier role of this lane in a transposing read (16-lane group G = lane / 16, row r = lane % 16 =
  // 4e + a): it points at key t0 + 4 (G / 2) + e of the queries 16 (G % 2) + 4a + 0..3, which the
  // writer kept in vector G % 2, half a % 2, elements 4 (a / 2) + 0..3.
  const int G = lane >> 4, r = lane & 15, e4 = r >> 2, a = r & 3;
  const int tr_off = (G & 1) * C::VEC + (a & 1) * (256 + 32) + (4 * (G >> 1) + e4) * 8 + 4 * (a >> 1);

  if (n_tiles > t_lo) { fetch(t_lo * C::BN); commit(0); }
  hw::block_sync();

  int stage = 0;
  for (int it = t_lo; it < n_tiles; ++it) {
    const int n0 = it * C::BN;
    const bool more = it + 1 < n_tiles;
    if (more) fetch(n0 + C::BN);

    const T* sK = (const T*)(smem + stage * C::STAGE_BYTES);
    const T* patch = sK + C::TILE + wave * C::PATCH;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      if (!block_used(n0 + 32 * nb)) continue;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const T* src = patch + 2 * nb * C::VEC + tr_off + 16 * c * 8;
        const V8 dsb = hw::join_v8<T>(hw::lds_read_tr16(src), hw::lds_read_tr16(src + 8 * 8));
#pragma unroll
        for (int db = 0; db < C::DV / 32; ++db)
          dq[db] = hw::mfma32(operand_transposed<T, C::LD>(sK, nb * 32 + 16 * c, db * 32, lane), dsb, dq[db]);
      }
    }

    if (more) commit(stage ^ 1);
    hw::block_sync();
    stage ^= 1;
  }

  if (my_m < M) {
    T* o1 = (T*)p.dq.ptr + batch * p.dq.sb + head * p.dq.sh + (int64_t)my_m * p.dq.st;
#pragma unroll
    for (int db = 0; db < C::DV / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        int d = db * 32 + 8 * g + 4 * hh;
        if (d < D) {
          hw::u32x2 w;
          w[0] = (uint32_t)hw::bits16<T>(dq[db][4 * g + 0] * p.sm_scale) | ((uint32_t)hw::bits16<T>(dq[db][4 * g + 1] * p.sm_scale) << 16);
          w[1] = (uint32_t)hw::bits16<T>(dq[db][4 * g + 2] * p.sm_scale) | ((uint32_t)hw::bits16<T>(dq[db][4 * g + 3] * p.sm_scale) << 16);
          *(hw::u32x2*)(o1 + d) = w;
        }
      }
  }
}

// ------------------------------------------------------------------------------ launchers ----
template <class T, bool PW, bool DS, bool DROP, bool GROUPED>
static int launch_dkdv(const BwdParams& p, hipStream_t stream) {
  const int chunk = GROUPED ? (p.chunk > 0 ? p.chunk : p.group) : 1;
  dim3 grid(((p.N + 127) / 128) * (p.H / chunk) * p.B, 1, 1);
  switch (p.D) {
    case 16: return launch(fa_bwd_dkdv_kernel<T, 16, PW, DS, DROP, GROUPED>, grid, KvCfg<T, 16, PW>::LDS_BYTES, stream, p);
    case 32: return launch(fa_bwd_dkdv_kernel<T, 32, PW, DS, DROP, GROUPED>, grid, KvCfg<T, 32, PW>::LDS_BYTES, stream, p);
    case 64: return launch(fa_bwd_dkdv_kernel<T, 64, PW, DS, DROP, GROUPED>, grid, KvCfg<T, 64, PW>::LDS_BYTES, stream, p);
    case 128: return launch(fa_bwd_dkdv_kernel<T, 128, PW, DS, DROP, GROUPED>, grid, KvCfg<T, 128, PW>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

template <class T, bool PW, bool DROP>
static int launch_dq(const BwdParams& p, hipStream_t stream) {
  dim3 grid(((p.M + 127) / 128) * p.H * p.B, 1, 1);
  switch (p.D) {
    case 16: return launch(fa_bwd_dq_kernel<T, 16, PW, DROP>, grid, QCfg<T, 16, PW>::LDS_BYTES, stream, p);
    case 32: return launch(fa_bwd_dq_kernel<T, 32, PW, DROP>, grid, QCfg<T, 32, PW>::LDS_BYTES, stream, p);
    case 64: return launch(fa_bwd_dq_kernel<T, 64, PW, DROP>, grid, QCfg<T, 64, PW>::LDS_BYTES, stream, p);
    case 128: return launch(fa_bwd_dq_kernel<T, 128, PW, DROP>, grid, QCfg<T, 128, PW>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

static bool bwd_args_ok(const BwdParams& p, bool piecewise) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0 || p.N <= 0 || p.group <= 0) return false;
  if (p.chunk < 0 || (p.chunk > 0 && p.group % p.chunk)) return false;
  if (!(p.dropout_p >= 0.f && p.dropout_p < 1.f) || (piecewise && p.dropout_p > 0.f)) return false;
  return true;
}

// summed dK/dV slices are built for plain attention without dropout
static bool dkdv_chunk_ok(const BwdParams& p, bool piecewise) {
  const int chunk = p.chunk > 0 ? p.chunk : p.group;
  return chunk == 1 || !(piecewise || p.dropout_p > 0.f);
}

template <class T>
static int dispatch_dkdv(const BwdParams& p, bool piecewise, bool keep_ds, hipStream_t stream) {
  if (piecewise) return keep_ds ? launch_dkdv<T, true, true, false, false>(p, stream) : launch_dkdv<T, true, false, false, false>(p, stream);
  const bool drop = p.dropout_p > 0.f;
  const bool grouped = (p.chunk > 0 ? p.chunk : p.group) > 1;
  if (keep_ds) {
    if (drop) return launch_dkdv<T, false, true, true, false>(p, stream);
    return grouped ? launch_dkdv<T, false, true, false, true>(p, stream) : launch_dkdv<T, false, true, false, false>(p, stream);
  }
  if (drop) return launch_dkdv<T, false, false, true, false>(p, stream);
  return grouped ? launch_dkdv<T, false, false, false, true>(p, stream) : launch_dkdv<T, false, false, false, false>(p, stream);
}

template <class T>
static int dispatch_dq(const BwdParams& p, bool piecewise, hipStream_t stream) {
  if (piecewise) return launch_dq<T, true, false>(p, stream);
  return p.dropout_p > 0.f ? launch_dq<T, false, true>(p, stream) : launch_dq<T, false, false>(p, stream);
}

int run_bwd_dkdv(const BwdParams& p, bool piecewise, hipStream_t stream) {
  if (!bwd_args_ok(p, piecewise) || !dkdv_chunk_ok(p, piecewise)) return kBadArgument;
  if (p.dtype == kDtypeF16) return dispatch_dkdv<hw::half_t>(p, piecewise, false, stream);
  if (p.dtype == kDtypeBF16) return dispatch_dkdv<hw::bf16_t>(p, piecewise, false, stream);
  return kUnsupported;
}

int run_bwd_dq(const BwdParams& p, bool piecewise, hipStream_t stream) {
  if (!bwd_args_ok(p, piecewise)) return kBadArgument;
  if (p.dtype == kDtypeF16) return dispatch_dq<hw::half_t>(p, piecewise, stream);
  if (p.dtype == kDtypeBF16) return dispatch_dq<hw::bf16_t>(p, piecewise, stream);
  return kUnsupported;
}

template <class T, bool PW>
static int launch_dq_from_ds(const BwdParams& p, hipStream_t stream) {
  dim3 grid(((p.M + 127) / 128) * p.H * p.B, 1, 1);
  switch (p.D) {
    case 16: return launch(fa_bwd_dq_from_ds_kernel<T, 16, PW>, grid, QdsCfg<T, 16>::LDS_BYTES, stream, p);
    case 32: return launch(fa_bwd_dq_from_ds_kernel<T, 32, PW>, grid, QdsCfg<T, 32>::LDS_BYTES, stream, p);
    case 64: return launch(fa_bwd_dq_from_ds_kernel<T, 64, PW>, grid, QdsCfg<T, 64>::LDS_BYTES, stream, p);
    case 128: return launch(fa_bwd_dq_from_ds_kernel<T, 128, PW>, grid, QdsCfg<T, 128>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

int64_t bwd_ds_workspace_bytes(int B, int H, int M, int N) {
  return (int64_t)B * H * (4 * (int64_t)((M + 127) / 128)) * (4 * (int64_t)((N + 127) / 128)) * 2048;
}

int run_bwd_dkdv_ds(const BwdParams& p, bool piecewise, hipStream_t stream) {
  if (!bwd_args_ok(p, piecewise) || !dkdv_chunk_ok(p, piecewise) || !p.ds) return kBadArgument;
  if (p.dtype == kDtypeF16) return dispatch_dkdv<hw::half_t>(p, piecewise, true, stream);
  if (p.dtype == kDtypeBF16) return dispatch_dkdv<hw::bf16_t>(p, piecewise, true, stream);
  return kUnsupported;
}

// piecewise: one launch per regime (p.regime, with p.k and p.dq set to that regime's tensors)
int run_bwd_dq_from_ds(const BwdParams& p, bool piecewise, hipStream_t stream) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0 || p.N <= 0 || p.group <= 0 || !p.ds) return kBadArgument;
  if (piecewise && !(p.regime == 1 || p.regime == 2)) return kBadArgument;
  if (p.dtype == kDtypeF16)
    return piecewise ? launch_dq_from_ds<hw::half_t, true>(p, stream) : launch_dq_from_ds<hw::half_t, false>(p, stream);
  if (p.dtype == kDtypeBF16)
    return piecewise ? launch_dq_from_ds<hw::bf16_t, true>(p, stream) : launch_dq_from_ds<hw::bf16_t, false>(p, stream);
  return kUnsupported;
}

}  // namespace fa
