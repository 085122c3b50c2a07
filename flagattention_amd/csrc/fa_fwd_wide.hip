// FlashAttention-2 forward for head size 128 with 64 query rows per wavefront, written as a
// hand-placed instruction stream ("slots").
//
// Replaces the reference's Triton kernel `_fwd_kernel` (src/flag_attn/flash.py:325-489) for the
// launches whose tile config is BLOCK_M = 256 (flash.py:64-87); fa_fwd.hip holds the 128-row kernel.
//
// Why a second forward kernel.  With 32 query rows per wavefront every matrix instruction needs a
// fresh 1 KB operand from LDS (1.8 LDS instructions per matrix instruction, counting the transposing
// reads).  Here a wavefront owns two 32-row blocks (A and B), so one K (or V^T) operand read from LDS
// feeds two matrix instructions (0.75 per matrix instruction; the cycles spent waiting for LDS fall
// to a sixth).  That takes most of the register file (O^T: 128, Q: 64, S: 64, P: 32), i.e. ONE
// wavefront per SIMD, so nothing but the wavefront itself can fill the matrix pipe while it does the
// softmax.  The overlap therefore comes from the instruction order, which is fixed by hand:
//
//   * An iteration i issues 64 matrix instructions in four runs of 16:
//         S(i+1) keys 0-31 | O += V(i)^T P(i) keys 0-31 | S(i+1) keys 32-63 | O += V(i)^T P(i) keys 32-63
//     and a scheduling fence after every slot keeps the compiler from regrouping them.  All matrix
//     instructions go through inline assembly so that S accumulates in VGPRs (where the vector ALU reads
//     it without copies) and O in AGPRs.
//   * The softmax works on 32-key halves.  A half's scores are complete 16 slots into its run; its row
//     maximum takes the next 13 slots, and its 32 exponential steps (one multiply-add and one
//     exponential per slot, a pack and a row-sum update every other slot) follow at one step per slot --
//     so the exponential steps of consecutive halves form one unbroken sequence, one per slot, and every
//     register of S and of P is free again just before the matrix instructions overwrite it: neither is
//     double buffered.
//   * The reference maximum of the exponentials is only raised when a half exceeds it by more than 2^8
//     (in the base-2 domain of the exponentials).  It is then almost always the old one, so the rescale
//     of O is a rare, wavefront-uniform branch between two runs instead of 128 multiplications per tile.
//     Softmax is invariant to the reference; probabilities up to 2^8 are exact in fp32 and in range for
//     fp16 and bf16.
//   * K and V tiles go from global memory straight into LDS (no registers, no ds_write), 1 KB per
//     instruction, into unpadded 256-byte rows whose 16-byte chunks are XOR-swizzled so that both the
//     16-byte row reads of K and the transposing reads of V are free of bank conflicts.  Two K stages
//     and three V stages; one workgroup barrier per iteration (slot 48).
#include "common.hpp"
#include "params.hpp"

namespace fa {

struct WideCfg {
  static constexpr int D = 128;
  static constexpr int BM = 256, BN = 64;  // query rows per workgroup (64 per wavefront), keys per tile
  static constexpr int KSTEPS = D / 16;
  static constexpr int ROW_BYTES = 2 * D;
  static constexpr int TILE_BYTES = BN * ROW_BYTES;   // 16 KB, no padding
  static constexpr int K_STAGES = 2, V_STAGES = 3;
  static constexpr int K_BASE = 0, V_BASE = K_STAGES * TILE_BYTES;
  static constexpr size_t LDS_BYTES = (K_STAGES + V_STAGES) * TILE_BYTES;  // 80 KB
  // slot positions inside an iteration (the second half run repeats the pattern 32 slots later)
  static constexpr int kSlots = 64;
  static constexpr int kBarrierSlot = 48;     // K(i+1) is read out; V(i+1) and K(i+2) have landed
  static constexpr int kLoadSlot = 49;        // 8 tile loads, one per slot
  static constexpr int kLead = 6;             // an operand is requested this many slots before its first use
  static constexpr int kMax = 17;             // 8 slots of row-maximum work per half (its S run ended in slot 15)
  static constexpr int kSwap = 25, kFinal = 28, kExp0 = 30;
  static constexpr float kTau = 8.f;          // the reference maximum is raised when exceeded by 2^kTau
};

// Hazard distances that the compiler cannot see (the matrix instructions are inline assembly): the last
// product of a half's S run sits in slot 15 (+ 32); a slot issues its matrix instruction first and its
// vector work after it, so vector work in slot 17 follows two further matrix instructions, the first of
// which cannot issue before the S product has left the front of the pipe and the second not before it
// has written back.  (Iteration -1 has no matrix instructions behind its S run and waits explicitly
// there; tests/test_emitted_hazard_distances.py checks the distances in the emitted code.)
static_assert(WideCfg::kMax >= 15 + 2, "the row maximum reads S before its last product has written back");
static_assert(WideCfg::kMax + 8 <= WideCfg::kSwap && WideCfg::kSwap + 3 <= WideCfg::kFinal &&
              WideCfg::kFinal + 2 <= WideCfg::kExp0, "maximum, exchange, decision and first exponential in this order");
// Step t of a tile's exponential pass runs in slot kExp0 + t (modulo 64, spilling into the next iteration).
// S of keys 0-31 is read by steps 0..31 and overwritten from slot 64; S of keys 32-63 by steps 32..63 and
// overwritten from slot 96.  P group g is complete after step 16 g + 18 and read from slot 80 + 8 g (g < 2)
// or 96 + 8 g (g >= 2); it is rewritten from step 16 g + 4, after its readers in slots 16 + 8 g ... (g < 2)
// or 32 + 8 g ... + 7 (g >= 2).
static_assert(WideCfg::kExp0 + 31 < 64 && WideCfg::kExp0 + 63 < 96, "S is exponentiated before the next tile's products overwrite it");
static_assert(WideCfg::kExp0 + 18 < 80 && WideCfg::kExp0 + 34 < 88 && WideCfg::kExp0 + 50 < 112 && WideCfg::kExp0 + 66 < 120,
              "every P group is packed before the second product reads it");
static_assert(WideCfg::kExp0 + 4 > 23 && WideCfg::kExp0 + 20 > 31 && WideCfg::kExp0 + 36 > 55 && WideCfg::kExp0 + 52 > 63,
              "a P group is rewritten only after the second product has read it");

// Element order of the exponential pass of a tile: step e = 16 g + s handles group g = 2 kb + c (keys
// 32 kb + 16 c ... + 15, the contraction slice of one second-product operand), and within the group
// alternates pairs of block A and block B: pair q = s / 2, block q % 2, registers 8 c + 2 (q / 2) + s % 2.
struct ExpStep {
  int g, kb, c, x, r, word;
  constexpr explicit ExpStep(int e)
      : g(e / 16), kb(e / 32), c((e / 16) % 2), x(((e % 16) / 2) % 2),
        r(8 * ((e / 16) % 2) + 2 * ((e % 16) / 4) + e % 2), word((e % 16) / 4) {}
};

template <class T>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, 1) fa_fwd_wide_kernel(FwdParams p) {
  using C = WideCfg;
  using V8 = typename hw::Elem<T>::v8;
  FA_LDS_DECL(smem);

  const int tid = hw::thread_id(), lane = tid & 63, wave = hw::uniform(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;
  // With the key axis in pieces a workgroup owns (row block, head, piece); the piece index runs fastest, so the
  // pieces of a head share an XCD's L2 with its other row blocks.
  const int pieces = p.num_splits > 0 ? p.num_splits : 1;
  const TileId wg = tile_of_workgroup(p.H * pieces, p.B);
  const int mb = (p.M + C::BM - 1) / C::BM - 1 - wg.rank;  // long rows first under the causal mask
  const int head = wg.head / pieces, piece = wg.head - head * pieces, batch = wg.batch;
  const int hk = head / p.group;
  // keys first_key .. first_key + N - 1 of the p.N keys; everything below works on the piece as if it were the
  // whole key axis: key index relative to first_key, pseq the offset of the causal diagonal in those terms
  const int first_key = piece * (p.num_splits > 0 ? p.split_size : 0);
  const int M = p.M, N = imin(p.N - first_key, p.num_splits > 0 ? p.split_size : p.N), pseq = p.N - M - first_key;
  const int m0 = mb * C::BM, mw = m0 + wave * 64;
  const int my_m[2] = {mw + l32, mw + 32 + l32};

  const T* qb = (const T*)p.q.ptr + batch * p.q.sb + head * p.q.sh;
  const T* kb = (const T*)p.k.ptr + batch * p.k.sb + hk * p.k.sh + (int64_t)first_key * p.k.st;
  const T* vb = (const T*)p.v.ptr + batch * p.v.sb + hk * p.v.sh + (int64_t)first_key * p.v.st;

  // ---- Q rows of this lane (one per block) as B operands: k = 16 kk + 8 hh + 0..7 ----
  V8 qreg[2][C::KSTEPS];
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk) {
      u32x4 z = {0u, 0u, 0u, 0u};
      if (my_m[x] < M) z = *(const u32x4*)(qb + (int64_t)my_m[x] * p.q.st + 16 * kk + 8 * hh);
      qreg[x][kk] = hw::as_v8<T>(z);
    }

  int hi = N;
  if (p.causal) hi = imin(N, pseq + m0 + C::BM);
  const int n_tiles = hi > 0 ? cdiv(hi, C::BN) : 0;

  // ---- LDS layout: row r of a tile at r * 256 bytes; its 16-byte chunk c sits at position
  //      c ^ (r & 15) in a K tile and c ^ (4 (r & 3)) in a V tile ----
  const uint32_t lds0 = hw::lds_address(smem);
  // K operand (kb, kk): row 32 kb + l32, chunk 2 kk + hh.  One address per kk, stage included (the two K
  // stages differ in one address bit, toggled once per iteration); kb is an immediate offset.
  uint32_t kaddr[C::KSTEPS];
#pragma unroll
  for (int kk = 0; kk < C::KSTEPS; ++kk) kaddr[kk] = lds0 + (uint32_t)(l32 * C::ROW_BYTES + (((2 * kk + hh) ^ (l32 & 15)) << 4));
  // V^T operand (g, db): two transposing reads; supplier lane (i = lane % 16, dhalf, hh) points at row
  // 32 kb + 16 c + 4 hh + i / 4 (+ 8), elements 32 db + 16 dhalf + 4 (i % 4) .. + 3.  One address per db,
  // stage included (advanced once per iteration); group and second read are immediate offsets.
  uint32_t vaddr[4];
  {
    const int i = lane & 15, dhalf = (lane >> 4) & 1, rowl = 4 * hh + (i >> 2), rho = (i >> 2) & 3;
#pragma unroll
    for (int db = 0; db < 4; ++db)
      vaddr[db] = lds0 + (uint32_t)(rowl * C::ROW_BYTES + ((4 * (db ^ rho) + 2 * dhalf + ((i & 3) >> 1)) << 4) + (i & 1) * 8);
  }

  // ---- tile loads: wavefront w, instruction j (0..3) fills LDS bytes j * 4096 + w * 1024 .. + 1023 of a
  //      tile = rows 16 j + 4 w + lane / 16, positions lane % 16.  A lane's row modulo 16 (what the swizzles
  //      look at) is the same in all four instructions, so one lane offset serves them and j only moves the
  //      wave-uniform base ----
  const int ld_rowl = 4 * wave + (lane >> 4), ld_pos = lane & 15;   // row of instruction j: 16 j + ld_rowl
  const uint32_t kchunk_bytes = (uint32_t)((ld_pos ^ ld_rowl) << 4);
  const uint32_t vchunk_bytes = (uint32_t)((ld_pos ^ (4 * (ld_rowl & 3))) << 4);
  const uint32_t kstride_b = (uint32_t)(p.k.st * (int64_t)sizeof(T)), vstride_b = (uint32_t)(p.v.st * (int64_t)sizeof(T));
  const uint32_t ld_lds = lds0 + (uint32_t)wave * 1024u;
  // `tile` names the stage; past the last tile the last one is fetched again (into a stage nobody reads
  // any more) so that the loads stay unconditional.  Rows past N re-read row N - 1: their scores are masked.
  auto load_k = [&](int tile, int j) {
    const int n0 = imin(tile, n_tiles - 1) * C::BN;
    const uint32_t row = (uint32_t)imin(16 * j + ld_rowl, N - 1 - n0);
    hw::dma_load16(kb + (int64_t)n0 * p.k.st, row * kstride_b + kchunk_bytes,
                   ld_lds + (uint32_t)(C::K_BASE + (tile & 1) * C::TILE_BYTES + j * 4096));
  };
  auto load_v = [&](int tile, int j) {
    const int n0 = imin(tile, n_tiles - 1) * C::BN;
    const uint32_t row = (uint32_t)imin(16 * j + ld_rowl, N - 1 - n0);
    hw::dma_load16(vb + (int64_t)n0 * p.v.st, row * vstride_b + vchunk_bytes,
                   ld_lds + (uint32_t)(C::V_BASE + (tile % 3) * C::TILE_BYTES + j * 4096));
  };
  // The same loads for iterations whose tiles (K: i + 3, V: i + 2) exist and are complete, so that nothing needs
  // clamping: the lane offsets are loop invariants, the wave-uniform source pointers walk on by 16 rows per
  // instruction (four instructions = one tile = the step to the next iteration) and the LDS stages rotate in
  // scalar registers.  fast_begin() sets them for iteration i.
  const uint32_t koff_fast = (uint32_t)ld_rowl * kstride_b + kchunk_bytes, voff_fast = (uint32_t)ld_rowl * vstride_b + vchunk_bytes;
  const char* ksrc_fast = nullptr;
  const char* vsrc_fast = nullptr;
  uint32_t kdst_fast = 0, vdst_fast = 0;
  auto fast_begin = [&](int i) {
    ksrc_fast = (const char*)(kb + (int64_t)(i + 3) * C::BN * p.k.st);
    vsrc_fast = (const char*)(vb + (int64_t)(i + 2) * C::BN * p.v.st);
    kdst_fast = ld_lds + (uint32_t)(C::K_BASE + ((i + 3) & 1) * C::TILE_BYTES);
    vdst_fast = ld_lds + (uint32_t)(C::V_BASE + ((i + 2) % 3) * C::TILE_BYTES);
  };
  auto load_k_fast = [&](auto j_tag) {
    constexpr int j = decltype(j_tag)::value;
    hw::dma_load16_at<j * 4096>(ksrc_fast, koff_fast, kdst_fast);
    ksrc_fast += 16 * (int64_t)kstride_b;
    if constexpr (j == 3) kdst_fast ^= (uint32_t)C::TILE_BYTES;   // the two K stages differ in this address bit alone (the LDS allocation starts at a multiple of 2 TILE_BYTES)
  };
  auto load_v_fast = [&](auto j_tag) {
    constexpr int j = decltype(j_tag)::value;
    hw::dma_load16_at<j * 4096>(vsrc_fast, voff_fast, vdst_fast);
    vsrc_fast += 16 * (int64_t)vstride_b;
    if constexpr (j == 3) {
      const uint32_t last = ld_lds + (uint32_t)(C::V_BASE + 2 * C::TILE_BYTES);
      vdst_fast = vdst_fast == last ? vdst_fast - 2 * (uint32_t)C::TILE_BYTES : vdst_fast + (uint32_t)C::TILE_BYTES;
    }
  };

  // ---- state ----
  f32x16 S[2][2];      // [block][32-key half]: scores, in VGPRs
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 16; ++r) S[x][h][r] = 0.f;
  u32x4 P[2][4];       // [block][group]: probabilities rounded to T, the B operand of the second product
  // [block][32-wide slice of D]: O^T.  On the GPU it lives in a[0:127], which only the pinned_o_* statements
  // name (they hide those registers from the compiler, see pinned_regs.hpp); this array carries the values in the
  // host simulator build and is never touched on the GPU.
  hw::o_tuples O;
  const float c2 = p.sm_scale * kLog2e;
  const float tau = C::kTau / c2;           // in units of raw scores (sm_scale > 0)
  // Reference maximum of the exponentials (raw score units).  A row that has seen no key yet holds a large
  // finite stand-in instead of -inf, so that -m_ref * c2 and differences of references need no special cases:
  // exp2(c2 (-inf - m_ref)) is 0 for a masked score and exp2(c2 (m_ref - m_new)) is 0 when the first key arrives.
  constexpr float kNoKeyYet = -1e30f;
  float m_ref[2] = {kNoKeyYet, kNoKeyYet};
  float shift[2] = {0.f, 0.f};              // -m_ref * c2 (set by a half's decision before its first multiply-add)
  float lsum[2][2] = {{0.f, 0.f}, {0.f, 0.f}};   // [block][partial]: this lane's part of the row sum (fp32, before rounding)
  // decisions of the two halves of a tile: factor by which O and the row sums move to the new reference
  // decisions of the two halves of a tile: by how much the reference moved (old - new, 0 where it stays); O and
  // the row sums are multiplied by exp2(c2 * moved) in the rare wavefront-uniform branch between two runs
  float moved[2][2] = {{0.f, 0.f}, {0.f, 0.f}};   // [half][block]
  bool changed[2] = {false, false};               // [half]
  float m_new[2] = {kNoKeyYet, kNoKeyYet}, shift_new[2] = {0.f, 0.f};
  float mx[2] = {neg_inf(), neg_inf()};
  float xpend = 0.f;    // multiply-add result waiting for its exponential
  float ering[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};   // exponentials waiting to be summed and packed
  V8 ring[4];           // matrix operands read from LDS, kLead slots ahead
  int rel[2] = {0, 0};  // masked tiles: key index (relative to the tile, minus 4 hh) up to which this lane's row sees keys

  // operand q of an iteration (used by slots 2 q and 2 q + 1):
  //   q in [0, 8):   K(keys 0-31, kk = q)          q in [8, 16):  V^T(group (q - 8) / 4, db = q % 4)
  //   q in [16, 24): K(keys 32-63, kk = q - 16)    q in [24, 32): V^T(group 2 + (q - 24) / 4, db = q % 4)
  auto request = [&](auto q_tag) {
    constexpr int q = decltype(q_tag)::value;
    if constexpr (q % 16 < 8) {
      ring[q % 4] = hw::as_v8<T>(hw::lds_load16(kaddr[q % 8] + (uint32_t)(C::K_BASE + (q / 16) * 32 * C::ROW_BYTES)));
    } else {
      constexpr int g = 2 * (q / 16) + (q % 8) / 4, db = q % 4;
      const uint32_t a = vaddr[db] + (uint32_t)(C::V_BASE + g * 16 * C::ROW_BYTES);
      ring[q % 4] = hw::join_v8<T>(hw::lds_read_tr16_at(a), hw::lds_read_tr16_at(a + 8 * C::ROW_BYTES));
    }
  };

  // Half an iteration: slots 32 HALF .. 32 HALF + 31.  The first 16 accumulate S of keys 32 HALF .. + 31
  // of tile i + 1 (if DO_S), the last 16 add the same keys of tile i to O (if DO_PV).  The vector work
  // belongs to tile i (steps 34.. of its exponential pass, if DO_PV) and to tile i + 1 (row maxima and
  // steps ..33, if DO_S).  MASKED: tile i + 1 needs the key tail / causal select.
  auto half_iteration = [&](auto half_tag, auto masked_tag, auto do_s_tag, auto do_pv_tag, auto fast_tag, int i) {
    constexpr int HALF = decltype(half_tag)::value;
    constexpr bool MASKED = decltype(masked_tag)::value, DO_S = decltype(do_s_tag)::value, DO_PV = decltype(do_pv_tag)::value;
    constexpr bool FAST = decltype(fast_tag)::value;   // the tiles this iteration fetches need no clamping (load_k_fast)
    if constexpr (MASKED && DO_S && HALF == 0) {
      const int n0 = (i + 1) * C::BN;
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const int lim = p.causal ? imin(my_m[x] + pseq, N - 1) : N - 1;
        rel[x] = lim - n0 - 4 * hh;
      }
    }
    hw::sched_fence();
    static_for<32>([&](auto slot) {
      constexpr int k = 32 * HALF + decltype(slot)::value, kl = k % 32;
      // ---------------------------------------------------------------- matrix instruction
      if constexpr (kl < 16) {
        if constexpr (DO_S) {
          constexpr int q = k / 2, x = k % 2, kk = q % 8;
          if constexpr (kk == 0) hw::pinned_s_mfma_first<2 * x + HALF>(ring[q % 4], qreg[x][kk], S[x][HALF], O);
          else hw::pinned_s_mfma<2 * x + HALF>(ring[q % 4], qreg[x][kk], S[x][HALF], O);
        }
      } else {
        if constexpr (DO_PV) {
          constexpr int q = k / 2, x = k % 2, g = 2 * HALF + (q % 8) / 4, db = q % 4;
          hw::pinned_o_mfma<4 * x + db>(ring[q % 4], hw::as_v8<T>(P[x][g]), O);
        }
      }
      // Iteration -1 has no second product: the slots behind its S run hold no matrix instruction, and the
      // vector work of slot kMax would follow the run's last products too closely (hazard distances above)
      if constexpr (DO_S && !DO_PV && kl == 16) hw::mfma_drain();
      // ---------------------------------------------------------------- stages, barrier, tile loads
      // all K operands of this iteration have been requested by slot 40 (operand 23): toggle the K stage
      if constexpr (k >= 41 && k < 41 + C::KSTEPS / 2) {
        kaddr[2 * (k - 41)] ^= (uint32_t)C::TILE_BYTES;
        kaddr[2 * (k - 41) + 1] ^= (uint32_t)C::TILE_BYTES;
      }
      // all V operands have been requested by slot 56 (operand 31): advance the V stage
      if constexpr (k >= 57 && k < 61) {
        // from the stage of tile i to that of tile i + 1, read in the next iteration (tile 0 sits in stage 0,
        // where the addresses start)
        const int step = i < 0 ? 0 : ((i + 1) % 3 == 0 ? -2 * C::TILE_BYTES : C::TILE_BYTES);
        vaddr[k - 57] += (uint32_t)step;
      }
      if constexpr (k == C::kBarrierSlot - 1) hw::wait_global_loads();
      if constexpr (k == C::kBarrierSlot) hw::barrier_only();
      if constexpr (k >= C::kLoadSlot && k < C::kLoadSlot + 4) {
        if constexpr (FAST) load_k_fast(std::integral_constant<int, k - C::kLoadSlot>{});
        else load_k(i + 3, k - C::kLoadSlot);
      }
      if constexpr (k >= C::kLoadSlot + 4 && k < C::kLoadSlot + 8) {
        if constexpr (FAST) load_v_fast(std::integral_constant<int, k - C::kLoadSlot - 4>{});
        else load_v(i + 2, k - C::kLoadSlot - 4);
      }
      // ---------------------------------------------------------------- row maximum of this half of tile i + 1
      if constexpr (DO_S) {
        if constexpr (kl >= C::kMax && kl < C::kMax + 8) {
          static_for<2>([&](auto u) {   // one step of each block per slot: consecutive instructions are independent
            constexpr int x = decltype(u)::value, r0 = 2 * (kl - C::kMax);
            f32x16& s = S[x][HALF];
            if constexpr (MASKED) {   // key 32 HALF + 8 (r / 4) + r % 4 + 4 hh of the tile is visible iff <= lim
              s[r0] = (HALF * 32 + 8 * (r0 / 4) + r0 % 4 <= rel[x]) ? s[r0] : neg_inf();
              s[r0 + 1] = (HALF * 32 + 8 * ((r0 + 1) / 4) + (r0 + 1) % 4 <= rel[x]) ? s[r0 + 1] : neg_inf();
            }
            if constexpr (r0 == 0) mx[x] = hw::slot_max2(s[0], s[1]);
            else mx[x] = hw::slot_max3(mx[x], s[r0], s[r0 + 1]);
          });
        }
        // a row lives in lanes l and l ^ 32: [A.lo, B.lo] vs [A.hi, B.hi], then both halves get both
        // (with a second product in the slots, the exchange sits at the end of its slot, below: the slot's own
        // vector work then supplies the wait states the exchange needs before it, the next slot's matrix
        // instruction those behind it)
        if constexpr (!DO_PV && (kl == C::kSwap || kl == C::kSwap + 2)) hw::swap_halves(mx[0], mx[1]);
        if constexpr (kl == C::kSwap + 1) { mx[0] = hw::max2(mx[0], mx[1]); mx[1] = mx[0]; }
        if constexpr (kl == C::kFinal || kl == C::kFinal + 1) {
          constexpr int x = kl - C::kFinal;
          const bool grow = mx[x] > m_ref[x] + tau;   // always on the first half with a visible key
          m_new[x] = grow ? mx[x] : m_ref[x];
          moved[HALF][x] = m_ref[x] - m_new[x];
          shift_new[x] = -m_new[x] * c2;
          if constexpr (x == 0) changed[HALF] = grow;
          else changed[HALF] = changed[HALF] || grow;
        }
        if constexpr (kl == C::kExp0) {   // from this slot on the multiply-adds belong to this half
#pragma unroll
          for (int x = 0; x < 2; ++x) { m_ref[x] = m_new[x]; shift[x] = shift_new[x]; }
        }
      }
      // the last iteration decides nothing: what its predecessor decided for this half has been applied to O
      // before this run, and must not reach the row sums a second time at the next boundary
      if constexpr (!DO_S && kl == C::kFinal) { moved[HALF][0] = 0.f; moved[HALF][1] = 0.f; changed[HALF] = false; }
      // ---------------------------------------------------------------- exponential passes
      // Step t of a tile's exponential pass: the multiply-add of element t, the exponential of element
      // t - 1, the row-sum update with element t - 2 and, every other step, the pack of elements t - 4 and
      // t - 3 -- no instruction consumes a result of the same or the preceding slot.
      auto exp_step = [&](auto t_tag) {
        constexpr int t = decltype(t_tag)::value;
        if constexpr (t >= 4 && t <= 66 && t % 2 == 0) {
          constexpr ExpStep e(t - 3);
          P[e.x][e.g][e.word] = hw::slot_pack2(T{}, ering[(t - 4) % 6], ering[(t - 3) % 6]);
        }
        if constexpr (t >= 2 && t <= 65) {   // two partial sums per block, so that consecutive updates are independent
          constexpr ExpStep e(t - 2);
          hw::slot_add(lsum[e.x][(e.r / 2) % 2], ering[(t - 2) % 6]);
        }
        if constexpr (t >= 1 && t <= 64) ering[(t - 1) % 6] = hw::slot_exp2(xpend);
        if constexpr (t <= 63) {
          constexpr ExpStep e(t);
          xpend = hw::slot_fma(S[e.x][e.kb][e.r], c2, shift[e.x]);
        }
      };
      // (the row sums move to a half's reference between the last update of the half before it -- steps 33 / 65,
      // slots 63 / 31 -- and its own first update -- steps 34 / 2, slots 0 / 32: at the boundary between two runs,
      // in rescale() below)
      // tile i: steps 34 + k (slots 30 to 32 only finish its last elements); placed before tile i + 1's step
      // of the same slot, because step 64 reads the pending multiply-add that step 0 overwrites
      if constexpr (DO_PV && k < C::kExp0 + 3) exp_step(std::integral_constant<int, k + 64 - C::kExp0>{});
      if constexpr (DO_S && k >= C::kExp0) exp_step(std::integral_constant<int, k - C::kExp0>{});
      if constexpr (DO_S && DO_PV && (kl == C::kSwap || kl == C::kSwap + 2)) hw::swap_halves_in_slot(mx[0], mx[1]);
      // ------------------------------------------------- operand of the slot pair kLead ahead
      // (last in its slot: the compiler pads two assembly statements that touch the same register and have no
      // instruction it knows between them with an s_nop; the LDS read of an even slot and the wait for an
      // operand before an odd slot's successor put one at every slot boundary)
      if constexpr (k % 2 == 0) {
        constexpr int q = (k + C::kLead) / 2;
        if constexpr (q < 32) {
          if constexpr ((q % 16 < 8 && DO_S) || (q % 16 >= 8 && DO_PV)) request(std::integral_constant<int, q>{});
        } else {   // operands 0..2 of the next iteration: kaddr already points at the other K stage
          request(std::integral_constant<int, q - 32>{});
        }
      }
      hw::sched_fence();
    });
  };

  if (n_tiles > 0) {
    // ---- prologue: K(0), K(1), V(0) ----
#pragma unroll
    for (int j = 0; j < 4; ++j) load_k(0, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) load_k(1, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) load_v(0, j);
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
      for (int kk = 0; kk < C::KSTEPS; ++kk) hw::keep_in_agprs(qreg[x][kk]);
    hw::wait_global_loads();
    hw::block_sync();
    request(std::integral_constant<int, 0>{});
    request(std::integral_constant<int, 1>{});
    request(std::integral_constant<int, 2>{});

    auto tile_masked = [&](int t) { return (t * C::BN + C::BN > N) || (p.causal && (t * C::BN + C::BN - 1 > mw + pseq)); };
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    using Yes = std::true_type;
    using No = std::false_type;
    // Between two runs: O moves to the reference of the half whose probabilities the coming run multiplies
    // (decided one iteration ago), and the row sums to the reference of the half whose exponentials the coming
    // run starts to add (decided in the run just finished: it is the other half).  Either happens only when some
    // row's reference moved, which is rare: one wavefront-uniform branch covers both.
    auto rescale = [&](auto half_tag) {
      constexpr int h = decltype(half_tag)::value;
      if (hw::wave_any(changed[0] || changed[1])) {
        hw::keep_branch();
        hw::mfma_drain();
        float to_o[2], to_sum[2];
#pragma unroll
        for (int x = 0; x < 2; ++x) {
          to_o[x] = hw::exp2_fast(moved[h][x] * c2);
          to_sum[x] = hw::exp2_fast(moved[1 - h][x] * c2);
          lsum[x][0] *= to_sum[x];
          lsum[x][1] *= to_sum[x];
        }
        static_for<8>([&](auto i) {
          constexpr int x = decltype(i)::value / 4, db = decltype(i)::value % 4;
          hw::pinned_o_scale<4 * x + db>(O, to_o[x]);
        });
        hw::mfma_drain();   // the rewritten accumulators are read by matrix instructions next
      }
    };

    // The variants of the iteration follow one another, each in a loop of its own: with alternatives inside
    // one loop the register allocator gives up on keeping S, O and Q in place.  Masked tiles come last (the
    // key tail, and under the causal mask the tiles on and above the wavefront's diagonal).
    // iteration -1: S(0) only.  Its V stage advance (to tile 0's stage) is the identity.
    // (cleared here, next to the first statements that hide a[0:127] from the compiler: earlier, the prologue's
    // own code could still use those registers)
    static_for<8>([&](auto t) { hw::pinned_o_clear<decltype(t)::value>(O); });
    if (tile_masked(0)) { half_iteration(H0{}, Yes{}, Yes{}, No{}, No{}, -1); half_iteration(H1{}, Yes{}, Yes{}, No{}, No{}, -1); }
    else { half_iteration(H0{}, No{}, Yes{}, No{}, No{}, -1); half_iteration(H1{}, No{}, Yes{}, No{}, No{}, -1); }
    int i = 0;
    // tiles [0, n_plain) are crossed by no mask for this wavefront: complete, and under the causal mask wholly
    // visible to its first row (tile t: 64 t + 63 <= mw + pseq)
    int n_plain = N / C::BN;
    if (p.causal) n_plain = imin(n_plain, imax(0, mw + pseq + 1) / C::BN);
    const int end_plain = imin(n_tiles, n_plain) - 1;                   // iterations i < end_plain form S of a plain tile i + 1
    // of these, the ones whose fetched tiles (up to tile i + 3) exist and are complete
    const int end_fast = imin(end_plain, imin(n_tiles, N / C::BN) - 3);
    fast_begin(0);
#pragma unroll 1
    for (; i < end_fast; ++i) {
      rescale(H0{});
      half_iteration(H0{}, No{}, Yes{}, Yes{}, Yes{}, i);
      rescale(H1{});
      half_iteration(H1{}, No{}, Yes{}, Yes{}, Yes{}, i);
    }
#pragma unroll 1
    for (; i < end_plain; ++i) {
      rescale(H0{});
      half_iteration(H0{}, No{}, Yes{}, Yes{}, No{}, i);
      rescale(H1{});
      half_iteration(H1{}, No{}, Yes{}, Yes{}, No{}, i);
    }
#pragma unroll 1
    for (; i + 1 < n_tiles; ++i) {
      rescale(H0{});
      half_iteration(H0{}, Yes{}, Yes{}, Yes{}, No{}, i);
      rescale(H1{});
      half_iteration(H1{}, Yes{}, Yes{}, Yes{}, No{}, i);
    }
    rescale(H0{});
    half_iteration(H0{}, No{}, No{}, Yes{}, No{}, i);
    rescale(H1{});
    half_iteration(H1{}, No{}, No{}, Yes{}, No{}, i);
    hw::wait_global_loads();   // the unconditional loads of the last iterations must not outlive the LDS allocation
    hw::mfma_drain();
  } else {   // no key is visible to any row of the workgroup: the epilogue writes zeros
    static_for<8>([&](auto t) { hw::pinned_o_clear<decltype(t)::value>(O); });
  }

  // ---- epilogue: O = acc / l, L = m * scale + ln(l); rows that saw no key give O = 0, L = -inf ----
  static_for<2>([&](auto x_tag) {
    constexpr int x = decltype(x_tag)::value;
    const float l_lane = lsum[x][0] + lsum[x][1];
    const float l_tot = l_lane + hw::xor32(l_lane);
    const bool empty = !(l_tot > 0.f);
    const float inv = empty ? 0.f : 1.f / l_tot;
    if (my_m[x] < M) {
      const bool whole = p.num_splits <= 0;
      const int64_t part_row = (((int64_t)batch * p.H + head) * pieces + piece) * M + my_m[x];
      T* ob = whole ? (T*)p.o.ptr + batch * p.o.sb + head * p.o.sh + (int64_t)my_m[x] * p.o.st
                    : (T*)((hw::half_t*)p.part_o + part_row * C::D);   // fp16 whatever T is; same element size
      static_for<16>([&](auto j_tag) {
        constexpr int db = decltype(j_tag)::value / 4, g = decltype(j_tag)::value % 4, I = 4 * x + db;
        const int d = db * 32 + 8 * g + 4 * hh;
        const float o0 = hw::pinned_o_read<I, 4 * g + 0>(O) * inv, o1 = hw::pinned_o_read<I, 4 * g + 1>(O) * inv;
        const float o2 = hw::pinned_o_read<I, 4 * g + 2>(O) * inv, o3 = hw::pinned_o_read<I, 4 * g + 3>(O) * inv;
        hw::u32x2 w;
        w[0] = whole ? hw::pack2(T{}, o0, o1) : hw::pack2(hw::half_t{}, o0, o1);
        w[1] = whole ? hw::pack2(T{}, o2, o3) : hw::pack2(hw::half_t{}, o2, o3);
        *(hw::u32x2*)(ob + d) = w;
      });
      if (hh == 0) {
        float* lse_out = whole ? p.lse + ((int64_t)batch * p.H + head) * M + my_m[x] : p.part_lse + part_row;
        *lse_out = empty ? neg_inf() : m_ref[x] * p.sm_scale + hw::log_nat(l_tot);
      }
    }
  });
}

// The wide kernel serves plain attention (no dropout, no second score regime) at head size 128 with row
// strides whose byte offsets inside a 64-row tile fit a 32-bit product.
bool fwd_wide_supported(const FwdParams& p) {
  if (p.D != 128 || p.dropout_p > 0.f || !(p.sm_scale > 0.f)) return false;
  const int64_t limit = (int64_t)1 << 24;   // bytes per row
  return p.k.st >= 0 && p.v.st >= 0 && p.k.st * 2 < limit && p.v.st * 2 < limit;
}

int run_fwd_wide(const FwdParams& p, hipStream_t stream) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0 || p.N < 0 || p.group <= 0 || !fwd_wide_supported(p)) return kBadArgument;
  if (p.num_splits < 0 || (p.num_splits > 0 && (p.split_size <= 0 || !p.part_o || !p.part_lse))) return kBadArgument;
  const int pieces = p.num_splits > 0 ? p.num_splits : 1;
  dim3 grid(((p.M + WideCfg::BM - 1) / WideCfg::BM) * p.H * p.B * pieces, 1, 1);
  if (p.dtype == kDtypeF16) return launch(fa_fwd_wide_kernel<hw::half_t>, grid, WideCfg::LDS_BYTES, stream, p);
  if (p.dtype == kDtypeBF16) return launch(fa_fwd_wide_kernel<hw::bf16_t>, grid, WideCfg::LDS_BYTES, stream, p);
  return kUnsupported;
}

// Split-KV launches with enough query rows to fill 256-row tiles run this kernel over pieces of the key axis
// (the decode kernel behind run_splitkv serves 16 rows per workgroup).
static FwdParams as_forward(const SplitParams& s) {
  FwdParams p = {};
  p.q = s.q; p.k = s.k; p.v = s.v;
  p.B = s.B; p.H = s.H; p.M = s.M; p.N = s.N; p.D = s.D;
  p.group = s.group; p.causal = s.causal; p.sm_scale = s.sm_scale; p.dtype = s.dtype;
  p.num_splits = s.num_splits; p.split_size = s.split_size;
  p.part_o = s.part_o; p.part_lse = s.part_lse;
  return p;
}

bool splitkv_wide_applies(const SplitParams& s) {
  return s.M >= WideCfg::BM && s.num_splits > 0 && s.split_size % WideCfg::BN == 0 && fwd_wide_supported(as_forward(s));
}

int run_splitkv_wide(const SplitParams& s, hipStream_t stream) { return run_fwd_wide(as_forward(s), stream); }

}  // namespace fa
