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
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, (D <= 128 ? 2 : 1)) paged_attn_kernel(PagedParams p) {
  using C = DecCfg<T, D>;
  FA_LDS_DECL(smem);
  const int tid = hw::thread_id(), lane = tid & 63, li = lane & 15;
  const int seq = hw::block_x(), hk = hw::block_y();
  const int G = p.Hq / p.Hkv;
  const int row_blocks = (G + 15) / 16;
  const int part = hw::block_z() / row_blocks, rb = hw::block_z() % row_blocks;
  const int ctx = p.context_lens[seq];

  int n_begin = 0, n_end = ctx;
  if (p.partition_size > 0) {
    n_begin = part * p.partition_size;
    if (n_begin >= ctx) return;  // whole workgroup: this partition lies past the context
    n_end = imin(ctx, n_begin + p.partition_size);
  }

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
    float top = neg_inf();
    for (int s = 0; s < parts; ++s) top = fmaxf(top, p.max_logits[base + (int64_t)s * G + g]);
    float acc = 0.f, z = 0.f;
    for (int s = 0; s < parts; ++s) {
      const int64_t slot = base + (int64_t)s * G + g;
      const float l = p.exp_sums[slot];
      if (!(l > 0.f)) continue;
      const float wgt = l * hw::exp2_fast((p.max_logits[slot] - top) * kLog2e);
      z += wgt;
      acc += wgt * (float)((const T*)p.tmp_out)[slot * D + d];
    }
    ((T*)p.out)[(int64_t)seq * p.o_ss + (int64_t)(hk * G + g) * p.o_sh + d] = (T)(z > 0.f ? acc / z : 0.f);
  }
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

int run_paged_reduce(const PagedParams& p, hipStream_t stream) {
  if (!paged_args_ok(p) || p.partition_size <= 0) return kBadArgument;
  dim3 grid(p.num_seqs, p.Hkv, 1);
  if (p.dtype == kDtypeF16) return launch(paged_reduce_kernel<hw::half_t>, grid, 0, stream, p);
  if (p.dtype == kDtypeBF16) return launch(paged_reduce_kernel<hw::bf16_t>, grid, 0, stream, p);
  return kUnsupported;
}

}  // namespace fa
