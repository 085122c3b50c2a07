// dK/dV backward kernel of plain (non-piecewise) attention, software pipelined for one wavefront
// per SIMD.  Replaces `_bwd_kv_kernel` (src/flag_attn/flash.py:571-745).  The piecewise variant keeps
// the simpler kernel in fa_bwd.hip.
//
// Same decomposition as fa_bwd.hip: a wavefront owns 32 keys whose K and V rows are register-resident
// B operands of S = Q K^T and dP = dO V^T; P and dS are the A operands of dV += P^T dO and
// dK += dS^T Q, whose B operands are read transposed from the Q/dO tiles in LDS.
//
// With D = 128 the accumulators leave room for only one wavefront per SIMD, so nothing but this
// wavefront's own instruction stream can hide LDS latency.  The loop is therefore laid out so that
// every LDS operand is requested one phase before the MFMAs that consume it:
//
//   step t (32 query rows, tile t in LDS stage t % 3):
//     commit tile t+1 (registers -> stage (t+1) % 3), request tile t+2 from HBM
//     request the transposed operands of tile t (for dV, dK) and its L / delta rows
//     S, dP MFMAs        <- row-major operands requested during step t-1
//     exp / dS arithmetic
//     workgroup barrier  (tile t+1 is now visible to every wavefront)
//     request the row-major operands of tile t+1
//     dV, dK MFMAs       <- transposed operands requested at the top of the step
//
// Three LDS stages make the single barrier per step sufficient: stage (t+1) % 3 was last read in
// step t-2, and every wavefront has left step t-2 before any passes the barrier of step t-1.
#include "common.hpp"
#include "params.hpp"

namespace fa {

template <class T, int D>
struct KvPipeCfg {
  static constexpr int BN = 128;  // keys per workgroup (32 per wavefront)
  static constexpr int BM = 32;   // queries per step
  static constexpr int NS = 3;    // LDS stages
  static constexpr int DV = D < 32 ? 32 : D;
  static constexpr int KSTEPS = D / 16;
  static constexpr int NDB = DV / 32;
  static constexpr int LD = DV + 40;  // rows 20 banks apart: good for both row-major and transposing reads
  static constexpr int TILE = BM * LD;
  static constexpr size_t STAGE_BYTES = 2 * TILE * sizeof(T) + 2 * BM * sizeof(float);
  static constexpr size_t LDS_BYTES = NS * STAGE_BYTES;
  static constexpr int WAVES_PER_SIMD = D <= 64 ? 2 : 1;
};

template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, (KvPipeCfg<T, D>::WAVES_PER_SIMD)) fa_bwd_dkdv_pipe_kernel(BwdParams p) {
  using C = KvPipeCfg<T, D>;
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
  const T* gb = (const T*)p.dout.ptr + batch * p.dout.sb + head * p.dout.sh;
  const T* kb = (const T*)p.k.ptr + batch * p.k.sb + hk * p.k.sh;
  const T* vb = (const T*)p.v.ptr + batch * p.v.sb + hk * p.v.sh;
  const float* lse = p.lse + ((int64_t)batch * p.H + head) * M;
  const float* dlt = p.delta + ((int64_t)batch * p.H + head) * M;

  V8 kreg[C::KSTEPS], vreg[C::KSTEPS];
#pragma unroll
  for (int kk = 0; kk < C::KSTEPS; ++kk) {
    u32x4 a = {0u, 0u, 0u, 0u}, b = a;
    if (my_n < N) {
      a = *(const u32x4*)(kb + (int64_t)my_n * p.k.st + 16 * kk + 8 * hh);
      b = *(const u32x4*)(vb + (int64_t)my_n * p.v.st + 16 * kk + 8 * hh);
    }
    kreg[kk] = hw::as_v8<T>(a);
    vreg[kk] = hw::as_v8<T>(b);
  }

  int m_lo = 0;
  if (p.causal) m_lo = (imax(0, n0 - pseq) / C::BM) * C::BM;
  const int n_tiles = m_lo < M ? cdiv(M - m_lo, C::BM) : 0;

  if (C::DV != D) {  // columns D..DV-1 of the tiles are read by the transposing loads, never written
    T* z = (T*)smem;
    for (int i = tid; i < (int)(C::LDS_BYTES / sizeof(T)); i += kThreads) z[i] = (T)0.f;
    hw::block_sync();
  }

  f32x16 dk[C::NDB], dv[C::NDB];
#pragma unroll
  for (int i = 0; i < C::NDB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dk[i][r] = 0.f; dv[i][r] = 0.f; }

  TileRegs<C::BM, D> qr, gr;
  float l_reg = 0.f, d_reg = 0.f;
  auto fetch = [&](int m0) {
    tile_fetch<T, C::BM, D>(qr, qb, p.q.st, m0, M, tid);
    tile_fetch<T, C::BM, D>(gr, gb, p.dout.st, m0, M, tid);
    if (tid < C::BM) {
      const int m = m0 + tid;
      l_reg = m < M ? lse[m] * kLog2e : __builtin_inff();  // rows past M: P = 0
      d_reg = m < M ? dlt[m] : 0.f;
    }
  };
  auto stage_base = [&](int t) { return smem + (t % C::NS) * C::STAGE_BYTES; };
  auto commit = [&](int t) {
    unsigned char* base = stage_base(t);
    tile_commit<T, C::BM, D, C::LD>(qr, (T*)base, tid);
    tile_commit<T, C::BM, D, C::LD>(gr, (T*)base + C::TILE, tid);
    float* f = (float*)(base + 2 * C::TILE * sizeof(T));
    if (tid < C::BM) { f[tid] = l_reg; f[C::BM + tid] = d_reg; }
  };

  // operands in flight
  V8 a_q[C::KSTEPS], a_g[C::KSTEPS];        // row-major Q / dO rows of the next S, dP products
  V8 b_g[2][C::NDB], b_q[2][C::NDB];        // transposed dO / Q operands of the current dV, dK products
  hw::f32x4 lrow[4], drow[4];               // L * log2e and delta of this lane's 16 query rows
  auto load_rowmajor = [&](int t) {
    const T* sQ = (const T*)stage_base(t);
    const T* sG = sQ + C::TILE;
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk) {
      a_q[kk] = operand_rowmajor<T, C::LD>(sQ, 0, 16 * kk, lane);
      a_g[kk] = operand_rowmajor<T, C::LD>(sG, 0, 16 * kk, lane);
    }
  };
  auto load_transposed = [&](int t) {
    const T* sQ = (const T*)stage_base(t);
    const T* sG = sQ + C::TILE;
    const float* sL = (const float*)(stage_base(t) + 2 * C::TILE * sizeof(T));
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      lrow[g] = *(const hw::f32x4*)(sL + 8 * g + 4 * hh);
      drow[g] = *(const hw::f32x4*)(sL + C::BM + 8 * g + 4 * hh);
    }
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int db = 0; db < C::NDB; ++db) {
        b_g[c][db] = operand_transposed<T, C::LD>(sG, 16 * c, db * 32, lane);
        b_q[c][db] = operand_transposed<T, C::LD>(sQ, 16 * c, db * 32, lane);
      }
  };

  if (n_tiles > 0) {
    fetch(m_lo);
    commit(0);
    if (n_tiles > 1) fetch(m_lo + C::BM);
  }
  hw::block_sync();
  if (n_tiles > 0) load_rowmajor(0);

  const float c2 = p.sm_scale * kLog2e;

  for (int it = 0; it < n_tiles; ++it) {
    const int m0 = m_lo + it * C::BM;
    if (it + 1 < n_tiles) commit(it + 1);
    if (it + 2 < n_tiles) fetch(m0 + 2 * C::BM);
    load_transposed(it);

    f32x16 s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
    for (int kk = 0; kk < C::KSTEPS; ++kk) {
      s = hw::mfma32(a_q[kk], kreg[kk], s);
      dp = hw::mfma32(a_g[kk], vreg[kk], dp);
    }
    // interleave: the transposed operands of this step trickle in behind the S / dP products
#pragma unroll
    for (int i = 0; i < 2 * C::KSTEPS; ++i) hw::sched_mfma_then_lds<1, 3>();
    hw::sched_fence();

    f32x16 pr, ds;
    const bool need_mask = p.causal && (m0 + pseq < nw + 31);
    if (need_mask) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + block_row(r, hh);
        float pv = hw::exp2_fast(fmaf(s[r], c2, -lrow[r >> 2][r & 3]));
        pv = (m + pseq >= my_n) ? pv : 0.f;
        pr[r] = pv;
        ds[r] = pv * (dp[r] - drow[r >> 2][r & 3]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = hw::exp2_fast(fmaf(s[r], c2, -lrow[r >> 2][r & 3]));
        pr[r] = pv;
        ds[r] = pv * (dp[r] - drow[r >> 2][r & 3]);
      }
    }
    V8 pa[2], da[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      pa[c] = pack_half_block<T>(pr, c);
      da[c] = pack_half_block<T>(ds, c);
    }

    hw::block_sync();
    const bool more = it + 1 < n_tiles;
    if (more) load_rowmajor(it + 1);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int db = 0; db < C::NDB; ++db) {
        dv[db] = hw::mfma32(pa[c], b_g[c][db], dv[db]);
        dk[db] = hw::mfma32(da[c], b_q[c][db], dk[db]);
      }
    // interleave: next step's row-major operands behind the dV / dK products
#pragma unroll
    for (int i = 0; i < 4 * C::NDB; ++i) hw::sched_mfma_then_lds<1, 1>();
    hw::sched_fence();
  }

  // ---- store: result block (keys x D) has D along lanes, keys along registers ----
  T* dkb = (T*)p.dk.ptr + batch * p.dk.sb + head * p.dk.sh;
  T* dvb = (T*)p.dv.ptr + batch * p.dv.sb + head * p.dv.sh;
#pragma unroll
  for (int db = 0; db < C::NDB; ++db) {
    const int d = db * 32 + l32;
    if (d < D) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int n = nw + block_row(r, hh);
        if (n < N) {
          dkb[(int64_t)n * p.dk.st + d] = (T)(dk[db][r] * p.sm_scale);
          dvb[(int64_t)n * p.dv.st + d] = (T)dv[db][r];
        }
      }
    }
  }
}

template <class T>
static int launch_dkdv_pipe(const BwdParams& p, hipStream_t stream) {
  dim3 grid(((p.N + 127) / 128) * p.H * p.B, 1, 1);
  switch (p.D) {
    case 16: return launch(fa_bwd_dkdv_pipe_kernel<T, 16>, grid, KvPipeCfg<T, 16>::LDS_BYTES, stream, p);
    case 32: return launch(fa_bwd_dkdv_pipe_kernel<T, 32>, grid, KvPipeCfg<T, 32>::LDS_BYTES, stream, p);
    case 64: return launch(fa_bwd_dkdv_pipe_kernel<T, 64>, grid, KvPipeCfg<T, 64>::LDS_BYTES, stream, p);
    case 128: return launch(fa_bwd_dkdv_pipe_kernel<T, 128>, grid, KvPipeCfg<T, 128>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

int run_bwd_dkdv_plain(const BwdParams& p, hipStream_t stream) {
  if (p.dtype == kDtypeF16) return launch_dkdv_pipe<hw::half_t>(p, stream);
  if (p.dtype == kDtypeBF16) return launch_dkdv_pipe<hw::bf16_t>(p, stream);
  return kUnsupported;
}

}  // namespace fa
