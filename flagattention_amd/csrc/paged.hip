// Paged attention decode (one query token per sequence, keys/values gathered through a block table)
// and the merge of its partitions.
//
// Replaces `_paged_attn_kernel` (src/flag_attn/paged.py:204-349) and
// `_paged_attn_v2_reduce_kernel` (paged.py:352-435).  The kernel is the decode core of decode.hpp
// with a gathering key/value source: every 16-byte load resolves its token's cache block through
// the sequence's row of the block table, and the table entries of the step after next are requested
// before the current step's arithmetic so that the two dependent loads never sit on the critical
// path.  All query heads of a kv head are served by one workgroup, so a cache block is read from
// HBM once per kv head.
#include "decode.hpp"
#include "params.hpp"

namespace fa {

template <class T, int D>
struct PagedSrc {
  using C = DecCfg<T, D>;
  const T* kc;
  const T* vc;
  const void* table;  // this sequence's row of the block table
  int bt64;
  int64_t s_blk, s_tok;
  int bs, bs_shift;  // bs_shift >= 0 when the block size is a power of two
  struct Ids { int blk[C::CH]; };
  FA_DEVICE int block_of(int n) const { return bs_shift >= 0 ? (n >> bs_shift) : (n / bs); }
  FA_DEVICE int slot_of(int n) const { return bs_shift >= 0 ? (n & (bs - 1)) : (n % bs); }
  FA_DEVICE void lookup(Ids& ids, int n0, int n_end, int lane) const {
#pragma unroll
    for (int i = 0; i < C::CH; ++i) {
      const int row = (lane + 64 * i) / C::CPR;
      const int n = imin(n0 + row, n_end - 1);  // branch-free: rows past the end resolve the last valid token
      ids.blk[i] = bt64 ? (int)((const int64_t*)table)[block_of(n)] : ((const int32_t*)table)[block_of(n)];
    }
  }
  FA_DEVICE const T* k_row(const Ids& ids, int i, int n) const {
    return kc + (int64_t)ids.blk[i] * s_blk + (int64_t)slot_of(n) * s_tok;
  }
  FA_DEVICE const T* v_row(const Ids& ids, int i, int n) const {
    return vc + (int64_t)ids.blk[i] * s_blk + (int64_t)slot_of(n) * s_tok;
  }
};

template <class T, int D>
FA_DEVICE PagedSrc<T, D> paged_source(const PagedParams& p, int seq, int hk) {
  PagedSrc<T, D> src;
  src.kc = (const T*)p.kc + (int64_t)hk * p.kv_sh;
  src.vc = (const T*)p.vc + (int64_t)hk * p.kv_sh;
  src.table = p.bt64 ? (const void*)((const int64_t*)p.block_tables + (int64_t)seq * p.bt_stride)
                     : (const void*)((const int32_t*)p.block_tables + (int64_t)seq * p.bt_stride);
  src.bt64 = p.bt64;
  src.s_blk = p.kv_sblk;
  src.s_tok = p.kv_stok;
  src.bs = p.block_size;
  src.bs_shift = (p.block_size & (p.block_size - 1)) == 0 ? __builtin_ctz(p.block_size) : -1;
  return src;
}

template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, (D <= 128 ? 2 : 1)) paged_attn_kernel(PagedParams p) {
  using C = DecCfg<T, D>;
  FA_LDS_DECL(smem);
  const int tid = hw::thread_id(), lane = tid & 63, li = lane & 15;
  const int seq = hw::block_x(), hk = hw::block_y();
  const int G = p.Hq / p.Hkv;
  const int row_blocks = (G + 15) / 16;
  // Partitions are issued last-first: high partitions exist only for the longest sequences, so
  // dispatching them at the end would leave a tail in which few workgroups run; partition 0, which
  // every sequence has, closes the launch instead.
  const int zz = (int)hw::grid_z() - 1 - hw::block_z();
  const int part = zz / row_blocks, rb = zz % row_blocks;
  const int ctx = p.context_lens[seq];

  int n_begin = 0, n_end = ctx;
  if (p.partition_size > 0) {
    n_begin = part * p.partition_size;
    if (n_begin >= ctx) return;  // whole workgroup: this partition lies past the context
    n_end = imin(ctx, n_begin + p.partition_size);
  }

  const PagedSrc<T, D> src = paged_source<T, D>(p, seq, hk);

  const int g_lane = rb * 16 + li;
  const T* q_row = nullptr;
  if (g_lane < G) q_row = (const T*)p.q + (int64_t)seq * p.q_ss + (int64_t)(hk * G + g_lane) * p.q_sh;

  DecodeOut<D> res;
  decode_block<T, D>(src, q_row, n_begin, n_end, n_end, p.scale * kLog2e, smem, res);

#pragma unroll
  for (int e = 0; e < DecodeOut<D>::kPerThread; ++e) {
    const int idx = tid + e * kThreads;
    const int row = idx / D, d = idx % D;
    const int g = rb * 16 + row;
    if (g < G) {
      const float val = res.row_sum[e] > 0.f ? res.o[e] / res.row_sum[e] : 0.f;
      if (p.partition_size > 0) {
        const int64_t slot = (((int64_t)seq * p.Hkv + hk) * p.num_parts + part) * G + g;
        ((T*)p.tmp_out)[slot * D + d] = (T)val;
        if (d == 0) {
          p.max_logits[slot] = res.row_max[e] * p.scale;
          p.exp_sums[slot] = res.row_sum[e];
        }
      } else {
        ((T*)p.out)[(int64_t)seq * p.o_ss + (int64_t)(hk * G + g) * p.o_sh + d] = (T)val;
      }
    }
  }
}

// out = sum_j w_j o_j / sum_j w_j with w_j = l_j exp(m_j - max_j m_j) over n partial results of one
// output element.  The loads of eight partials are issued together: a loop that loads, waits and
// accumulates one partial at a time costs a full memory latency per partial.
template <class FM, class FL, class FO>
FA_DEVICE float merge_partials(int n, FM m_of, FL l_of, FO o_of) {
  constexpr int kBatch = 8;
  float top = neg_inf();
  for (int j0 = 0; j0 < n; j0 += kBatch) {
    float t[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) t[u] = m_of(imin(j0 + u, n - 1));
#pragma unroll
    for (int u = 0; u < kBatch; ++u) top = fmaxf(top, t[u]);
  }
  float acc = 0.f, z = 0.f;
  for (int j0 = 0; j0 < n; j0 += kBatch) {
    float mv[kBatch], lv[kBatch], ov[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int j = imin(j0 + u, n - 1);
      mv[u] = m_of(j);
      lv[u] = l_of(j);
      ov[u] = o_of(j);
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      if (j0 + u < n && lv[u] > 0.f) {
        const float wgt = lv[u] * hw::exp2_fast((mv[u] - top) * kLog2e);
        z += wgt;
        acc += wgt * ov[u];
      }
    }
  }
  return z > 0.f ? acc / z : 0.f;
}

// One workgroup per (sequence, kv head): out = sum_p tmp_out_p * w_p / sum_p w_p with
// w_p = exp_sum_p * exp(max_p - max).  Partitions past the context were never written and are skipped.
template <class T>
FA_KERNEL void FA_LAUNCH_BOUNDS(kThreads) paged_reduce_kernel(PagedParams p) {
  const int tid = hw::thread_id();
  const int seq = hw::block_x(), hk = hw::block_y();
  const int G = p.Hq / p.Hkv, D = p.D;
  const int ctx = p.context_lens[seq];
  const int parts = imin(p.num_parts, cdiv(ctx, p.partition_size));
  const int64_t base = ((int64_t)seq * p.Hkv + hk) * p.num_parts * G;
  for (int idx = tid; idx < G * D; idx += kThreads) {
    const int g = idx / D, d = idx % D;
    const float val = merge_partials(
        parts, [&](int j) { return p.max_logits[base + (int64_t)j * G + g]; },
        [&](int j) { return p.exp_sums[base + (int64_t)j * G + g]; },
        [&](int j) { return (float)((const T*)p.tmp_out)[(base + (int64_t)j * G + g) * D + d]; });
    ((T*)p.out)[(int64_t)seq * p.o_ss + (int64_t)(hk * G + g) * p.o_sh + d] = (T)val;
  }
}


// ---------------------------------------------------------------------------------------------
// Balanced launch: the keys of all (sequence, kv head) pairs, counted in units of 128, are laid end
// to end and cut into num_wgs equal ranges, one per workgroup, so that every workgroup streams the
// same number of bytes whatever the spread of context lengths and the launch is exactly one
// resident wave of workgroups.  A pair that lies inside one range is finished by that workgroup
// and written to `out`; a pair cut by range boundaries leaves one partial result per workgroup it
// touches (at most two per workgroup: the pair it starts in the middle of, slot 2w, and the pair it
// leaves unfinished, slot 2w + 1), which paged_balanced_reduce_kernel merges.
//
// Workspace (floats): 2 * num_wgs slots of [16][D] normalised outputs, [16] max logits, [16] sums of
// exponentials; then num_wgs records of 4 ints {sequence, kv head, row block, number of following
// workgroups that continue the pair left unfinished} (the last is 0 when there is no such pair).
// ---------------------------------------------------------------------------------------------
constexpr int kUnitKeys = 128;
constexpr int kMinUnitsPerWg = 2;

template <int D> FA_DEVICE int balanced_slot_floats() { return 16 * D + 32; }

template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, (D <= 128 ? 2 : 1)) paged_balanced_kernel(PagedParams p) {
  using C = DecCfg<T, D>;
  FA_LDS_DECL(smem);
  const int tid = hw::thread_id(), lane = tid & 63, li = lane & 15;
  const int w = hw::block_x();
  const int G = p.Hq / p.Hkv;
  const int row_blocks = (G + 15) / 16;
  const int pairs_per_seq = p.Hkv * row_blocks;
  auto units_of = [&](int seq) { const int c = p.context_lens[seq]; return c > 0 ? (c + kUnitKeys - 1) / kUnitKeys : 0; };

  // ---- every wavefront scans the context lengths for itself, 64 at a time: no LDS, no barrier ----
  auto prefix_in_wave = [&](int u) {   // inclusive prefix sum over the lanes
    int incl = u;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int t = hw::shfl_up(incl, d);
      if (lane >= d) incl += t;
    }
    return incl;
  };
  int total_units = 0;
  for (int base = 0; base < p.num_seqs; base += 64) {
    const int s = base + lane;
    const int u = s < p.num_seqs ? units_of(s) : 0;
    // An empty sequence has no keys to stream: its output rows are zero.  Every wavefront sees the same
    // empty sequences here; they are dealt round-robin to the workgroups, and the threads of the one
    // that takes a sequence clear its rows together.
    for (uint64_t todo = hw::ballot(s < p.num_seqs && u == 0 && s % p.num_wgs == w); todo; todo &= todo - 1) {
      const int e = base + __builtin_ctzll(todo);
      for (int i = tid; i < p.Hq * D; i += kThreads) ((T*)p.out)[(int64_t)e * p.o_ss + (int64_t)(i / D) * p.o_sh + i % D] = (T)0.f;
    }
    total_units += hw::uniform(hw::lane_value(prefix_in_wave(u), 63));
  }
  // everything derived from the total (the key ranges, the step counts of the wavefronts) stays in scalar registers
  const int64_t total = (int64_t)total_units * pairs_per_seq;
  const int64_t per = (int64_t)imax(kMinUnitsPerWg, (int)((total + p.num_wgs - 1) / p.num_wgs));
  const int64_t u_begin = (int64_t)w * per;
  const int64_t u_end = u_begin + per < total ? u_begin + per : total;
  int* meta = (int*)(p.ws + (int64_t)2 * p.num_wgs * balanced_slot_floats<D>()) + 4 * w;
  if (u_begin >= total) {  // whole workgroup
    if (tid == 0) meta[3] = 0;
    return;
  }
  // the sequence whose pairs hold unit u_begin, and the units of the sequences before it
  int seq = 0, before = 0;
  {
    int running = 0;
    for (int base = 0; base < p.num_seqs; base += 64) {
      const int s = base + lane;
      const int u = s < p.num_seqs ? units_of(s) : 0;
      const int incl = prefix_in_wave(u), excl = incl - u;
      const bool here = u > 0 && (int64_t)(running + excl) * pairs_per_seq <= u_begin &&
                        u_begin < (int64_t)(running + incl) * pairs_per_seq;
      const uint64_t hit = hw::ballot(here);
      const int first = hit ? __builtin_ctzll(hit) : 0;
      const int excl_first = hw::lane_value(excl, first), all = hw::lane_value(incl, 63);
      if (hit) { seq = base + first; before = running + excl_first; }
      running += all;
    }
    seq = hw::uniform(seq);
    before = hw::uniform(before);
  }
  int64_t u = u_begin;
  int unfinished = 0;

  while (u < u_end) {
    const int ctx = hw::uniform(p.context_lens[seq]);
    const int us = ctx > 0 ? (ctx + kUnitKeys - 1) / kUnitKeys : 0;
    const int local = (int)(u - (int64_t)before * pairs_per_seq);  // unit index inside this sequence's pairs
    if (us == 0 || local >= us * pairs_per_seq) { before += us; ++seq; continue; }
    const int pr = local / us, lo = local % us;
    const int hk = pr / row_blocks, rb = pr % row_blocks;
    const int hi = (int)(u_end - u < (int64_t)(us - lo) ? lo + (u_end - u) : us);
    const int n_begin = lo * kUnitKeys, n_end = imin(ctx, hi * kUnitKeys);

    const PagedSrc<T, D> src = paged_source<T, D>(p, seq, hk);
    const int g_lane = rb * 16 + li;
    const T* q_row = nullptr;
    if (g_lane < G) q_row = (const T*)p.q + (int64_t)seq * p.q_ss + (int64_t)(hk * G + g_lane) * p.q_sh;

    hw::block_sync();  // the previous pair's merge area is read out before staging reuses it
    DecodeOut<D> res;
    decode_block<T, D>(src, q_row, n_begin, n_end, n_end, p.scale * kLog2e, smem, res);

    const bool whole = lo == 0 && hi == us;
    float* slot = p.ws + (int64_t)(2 * w + (lo == 0 ? 1 : 0)) * balanced_slot_floats<D>();
#pragma unroll
    for (int e = 0; e < DecodeOut<D>::kPerThread; ++e) {
      const int idx = tid + e * kThreads;
      const int row = idx / D, d = idx % D;
      const int g = rb * 16 + row;
      if (idx < 16 * D && g < G) {
        const float val = res.row_sum[e] > 0.f ? res.o[e] / res.row_sum[e] : 0.f;
        if (whole) {
          ((T*)p.out)[(int64_t)seq * p.o_ss + (int64_t)(hk * G + g) * p.o_sh + d] = (T)val;
        } else {
          slot[row * D + d] = val;
          if (d == 0) {
            slot[16 * D + row] = res.row_max[e] * p.scale;
            slot[16 * D + 16 + row] = res.row_sum[e];
          }
        }
      }
    }
    if (lo == 0 && hi < us) {  // this pair continues in the following workgroups, `per` units each
      unfinished = (int)(((int64_t)(us - hi) + per - 1) / per);
      if (tid == 0) { meta[0] = seq; meta[1] = hk; meta[2] = rb; }
    }
    u += hi - lo;
  }
  if (tid == 0) meta[3] = unfinished;
}

// Workgroup w merges the pair that attention workgroup w started and left unfinished: slot 2w + 1
// and slot 2(w + j) of each of the following workgroups that continued it.
template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS(kThreads) paged_balanced_reduce_kernel(PagedParams p) {
  const int tid = hw::thread_id();
  const int w = hw::block_x();
  const int SF = balanced_slot_floats<D>();
  const int* meta = (const int*)(p.ws + (int64_t)2 * p.num_wgs * SF) + 4 * w;
  const int follow = meta[3];
  if (follow <= 0) return;
  const int seq = meta[0], hk = meta[1], rb = meta[2];
  const int G = p.Hq / p.Hkv;
  for (int idx = tid; idx < 16 * D; idx += kThreads) {
    const int row = idx / D, d = idx % D;
    const int g = rb * 16 + row;
    if (g >= G) continue;
    auto slot_of = [&](int j) { return p.ws + (int64_t)(j == 0 ? 2 * w + 1 : 2 * (w + j)) * SF; };
    const float val = merge_partials(
        follow + 1, [&](int j) { return slot_of(j)[16 * D + row]; },
        [&](int j) { return slot_of(j)[16 * D + 16 + row]; }, [&](int j) { return slot_of(j)[row * D + d]; });
    ((T*)p.out)[(int64_t)seq * p.o_ss + (int64_t)(hk * G + g) * p.o_sh + d] = (T)val;
  }
}

template <class T, int D>
static int launch_balanced_d(const PagedParams& p, hipStream_t stream) {
  dim3 grid(p.num_wgs, 1, 1);
  const size_t lds = DecCfg<T, D>::LDS_BYTES > 4096 ? DecCfg<T, D>::LDS_BYTES : 4096;
  int rc = launch(paged_balanced_kernel<T, D>, grid, lds, stream, p);
  if (rc) return rc;
  return launch(paged_balanced_reduce_kernel<T, D>, grid, 0, stream, p);
}

template <class T>
static int launch_balanced(const PagedParams& p, hipStream_t stream) {
  switch (p.D) {
    case 16: return launch_balanced_d<T, 16>(p, stream);
    case 32: return launch_balanced_d<T, 32>(p, stream);
    case 64: return launch_balanced_d<T, 64>(p, stream);
    case 128: return launch_balanced_d<T, 128>(p, stream);
    case 256: return launch_balanced_d<T, 256>(p, stream);
    case 512: return launch_balanced_d<T, 512>(p, stream);
  }
  return kUnsupported;
}

template <class T>
static int launch_paged(const PagedParams& p, hipStream_t stream) {
  const int G = p.Hq / p.Hkv;
  const int parts = p.partition_size > 0 ? p.num_parts : 1;
  dim3 grid(p.num_seqs, p.Hkv, parts * ((G + 15) / 16));
  switch (p.D) {
    case 16: return launch(paged_attn_kernel<T, 16>, grid, DecCfg<T, 16>::LDS_BYTES, stream, p);
    case 32: return launch(paged_attn_kernel<T, 32>, grid, DecCfg<T, 32>::LDS_BYTES, stream, p);
    case 64: return launch(paged_attn_kernel<T, 64>, grid, DecCfg<T, 64>::LDS_BYTES, stream, p);
    case 128: return launch(paged_attn_kernel<T, 128>, grid, DecCfg<T, 128>::LDS_BYTES, stream, p);
    case 256: return launch(paged_attn_kernel<T, 256>, grid, DecCfg<T, 256>::LDS_BYTES, stream, p);
    case 512: return launch(paged_attn_kernel<T, 512>, grid, DecCfg<T, 512>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

static bool paged_args_ok(const PagedParams& p) {
  if (p.num_seqs <= 0 || p.Hq <= 0 || p.Hkv <= 0 || p.Hq % p.Hkv || p.block_size <= 0) return false;
  if (p.partition_size < 0) return false;
  if (p.partition_size > 0 && (p.partition_size % p.block_size || p.num_parts <= 0)) return false;
  return true;
}

int run_paged(const PagedParams& p, hipStream_t stream) {
  if (!paged_args_ok(p)) return kBadArgument;
  if (p.dtype == kDtypeF16) return launch_paged<hw::half_t>(p, stream);
  if (p.dtype == kDtypeBF16) return launch_paged<hw::bf16_t>(p, stream);
  return kUnsupported;
}

int64_t paged_balanced_workspace_bytes(int num_wgs, int D) {
  return (int64_t)num_wgs * (2 * (16 * (int64_t)D + 32) * (int64_t)sizeof(float) + 4 * (int64_t)sizeof(int));
}

int run_paged_balanced(const PagedParams& p, hipStream_t stream) {
  if (!paged_args_ok(p) || p.partition_size != 0 || p.num_wgs <= 0 || !p.ws) return kBadArgument;
  if (p.dtype == kDtypeF16) return launch_balanced<hw::half_t>(p, stream);
  if (p.dtype == kDtypeBF16) return launch_balanced<hw::bf16_t>(p, stream);
  return kUnsupported;
}

int run_paged_reduce(const PagedParams& p, hipStream_t stream) {
  if (!paged_args_ok(p) || p.partition_size <= 0) return kBadArgument;
  dim3 grid(p.num_seqs, p.Hkv, 1);
  if (p.dtype == kDtypeF16) return launch(paged_reduce_kernel<hw::half_t>, grid, 0, stream, p);
  if (p.dtype == kDtypeBF16) return launch(paged_reduce_kernel<hw::bf16_t>, grid, 0, stream, p);
  return kUnsupported;
}

}  // namespace fa
