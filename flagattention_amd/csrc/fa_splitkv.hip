// Split-KV forward (flash decoding) and the merge of its partial results.
//
// Replaces `_fwd_split_kv_kernel` (src/flag_attn/split_kv.py:14-160) and `_fwd_combine_kv_splits`
// (split_kv.py:162-227).  The split kernel is the decode core of decode.hpp over a dense K/V
// stream: a workgroup takes one (batch, kv head, split) and up to 16 of the G * M query rows that
// share that kv head, so the keys and values of a split are read once for the whole GQA group.
// Partial outputs are fp16 whatever the input dtype, as in the reference (flash.py:96); a split
// that holds no visible key for a row stores 0 and a log-normalizer of -inf, and the merge weights
// by select so that such splits drop out instead of producing NaN.
#include "decode.hpp"
#include "params.hpp"

namespace fa {

template <class T, int D>
struct DenseSrc {
  const T* kb;
  const T* vb;
  int64_t k_st, v_st;
  struct Ids {};
  FA_DEVICE void lookup(Ids&, int, int, int) const {}
  FA_DEVICE const T* k_row(const Ids&, int, int n) const { return kb + (int64_t)n * k_st; }
  FA_DEVICE const T* v_row(const Ids&, int, int n) const { return vb + (int64_t)n * v_st; }
};

template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, 2) fa_splitkv_kernel(SplitParams p) {
  using C = DecCfg<T, D>;
  FA_LDS_DECL(smem);
  const int tid = hw::thread_id(), lane = tid & 63, li = lane & 15;
  const int rb = hw::block_x(), split = hw::block_y();
  const int batch = hw::block_z() / (p.H / p.group), hk = hw::block_z() % (p.H / p.group);
  const int M = p.M, N = p.N, pseq = N - M;
  const int rows = p.group * M;

  DenseSrc<T, D> src;
  src.kb = (const T*)p.k.ptr + batch * p.k.sb + hk * p.k.sh;
  src.vb = (const T*)p.v.ptr + batch * p.v.sb + hk * p.v.sh;
  src.k_st = p.k.st;
  src.v_st = p.v.st;

  // this lane's query row: rho = g * M + m
  const int rho = rb * 16 + li;
  const T* q_row = nullptr;
  int lane_limit = 0;
  if (rho < rows) {
    const int g = rho / M, m = rho % M;
    q_row = (const T*)p.q.ptr + batch * p.q.sb + (hk * p.group + g) * p.q.sh + (int64_t)m * p.q.st;
    lane_limit = p.causal ? imin(N, m + pseq + 1) : N;
  }
  const int n_begin = split * p.split_size;
  const int n_end = imin(N, n_begin + p.split_size);

  DecodeOut<D> res;
  decode_block<T, D>(src, q_row, n_begin, n_end, lane_limit, p.sm_scale * kLog2e, smem, res);

#pragma unroll
  for (int e = 0; e < DecodeOut<D>::kPerThread; ++e) {
    const int idx = tid + e * kThreads;
    const int row = idx / D, d = idx % D;
    const int r = rb * 16 + row;
    if (r < rows) {
      const int g = r / M, m = r % M;
      const int64_t slot = (((int64_t)batch * p.H + hk * p.group + g) * p.num_splits + split) * M + m;
      const bool empty = !(res.row_sum[e] > 0.f);
      ((hw::half_t*)p.part_o)[slot * D + d] = (hw::half_t)(empty ? 0.f : res.o[e] / res.row_sum[e]);
      if (d == 0)
        p.part_lse[slot] = empty ? neg_inf() : res.row_max[e] * p.sm_scale + hw::log_nat(res.row_sum[e]);
    }
  }
}

template <class T, int D>
FA_KERNEL void FA_LAUNCH_BOUNDS(kThreads) fa_combine_kernel(CombineParams p) {
  constexpr int kLanesPerRow = D / 8;
  constexpr int kRows = kThreads / kLanesPerRow;
  const int tid = hw::thread_id();
  const int64_t row = (int64_t)hw::block_x() * kRows + tid / kLanesPerRow;  // over B * H * M
  const int col = (tid % kLanesPerRow) * 8;
  const int64_t total_rows = (int64_t)p.B * p.H * p.M;
  if (row >= total_rows) return;
  const int m = (int)(row % p.M);
  const int64_t bh = row / p.M;
  const int S = p.num_splits;
  const float* ls = p.part_lse + bh * S * p.M + m;  // stride M between splits
  // loads of four splits are issued together: one split at a time would cost a memory latency each
  constexpr int kBatch = 4;
  float top = neg_inf();
  for (int s0 = 0; s0 < S; s0 += kBatch) {
    float t[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) t[u] = ls[(int64_t)imin(s0 + u, S - 1) * p.M];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) top = fmaxf(top, t[u]);
  }
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float z = 0.f;
  if (top > neg_inf()) {
    for (int s0 = 0; s0 < S; s0 += kBatch) {
      float l[kBatch];
      u32x4 raw[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int s = imin(s0 + u, S - 1);
        l[u] = ls[(int64_t)s * p.M];
        raw[u] = *(const u32x4*)((const hw::half_t*)p.part_o + ((bh * S + s) * p.M + m) * D + col);
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        if (s0 + u >= S || l[u] == neg_inf()) continue;  // past the end, or a split without a visible key
        const float wgt = hw::exp2_fast((l[u] - top) * kLog2e);
        z += wgt;
        auto v = hw::as_v8<hw::half_t>(raw[u]);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += wgt * (float)v[e];
      }
    }
  }
  const float inv = z > 0.f ? 1.f / z : 0.f;
  const int b = (int)(bh / p.H), h = (int)(bh % p.H);
  T* o = (T*)p.o.ptr + b * p.o.sb + h * p.o.sh + (int64_t)m * p.o.st + col;
  u32x4 w;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    w[e] = (uint32_t)hw::bits16<T>(acc[2 * e] * inv) | ((uint32_t)hw::bits16<T>(acc[2 * e + 1] * inv) << 16);
  *(u32x4*)o = w;
  if (col == 0) p.lse[row] = z > 0.f ? top + hw::log_nat(z) : neg_inf();
}

template <class T>
static int launch_split(const SplitParams& p, hipStream_t stream) {
  const int rows = p.group * p.M;
  dim3 grid((rows + 15) / 16, p.num_splits, p.B * (p.H / p.group));
  switch (p.D) {
    case 16: return launch(fa_splitkv_kernel<T, 16>, grid, DecCfg<T, 16>::LDS_BYTES, stream, p);
    case 32: return launch(fa_splitkv_kernel<T, 32>, grid, DecCfg<T, 32>::LDS_BYTES, stream, p);
    case 64: return launch(fa_splitkv_kernel<T, 64>, grid, DecCfg<T, 64>::LDS_BYTES, stream, p);
    case 128: return launch(fa_splitkv_kernel<T, 128>, grid, DecCfg<T, 128>::LDS_BYTES, stream, p);
  }
  return kUnsupported;
}

int run_splitkv(const SplitParams& p, hipStream_t stream) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0 || p.N <= 0 || p.group <= 0 || p.num_splits <= 0 || p.split_size <= 0)
    return kBadArgument;
  if ((int64_t)p.num_splits * p.split_size < p.N) return kBadArgument;
  if (splitkv_wide_applies(p)) return run_splitkv_wide(p, stream);   // many query rows: 256-row tiles
  if (p.dtype == kDtypeF16) return launch_split<hw::half_t>(p, stream);
  if (p.dtype == kDtypeBF16) return launch_split<hw::bf16_t>(p, stream);
  return kUnsupported;
}

template <class T>
static int launch_combine(const CombineParams& p, hipStream_t stream) {
  auto rows = [](int D) { return kThreads / (D / 8); };
  const int64_t total = (int64_t)p.B * p.H * p.M;
  auto blocks = [&](int D) { return dim3((unsigned)((total + rows(D) - 1) / rows(D))); };
  switch (p.D) {
    case 16: return launch(fa_combine_kernel<T, 16>, blocks(16), 0, stream, p);
    case 32: return launch(fa_combine_kernel<T, 32>, blocks(32), 0, stream, p);
    case 64: return launch(fa_combine_kernel<T, 64>, blocks(64), 0, stream, p);
    case 128: return launch(fa_combine_kernel<T, 128>, blocks(128), 0, stream, p);
  }
  return kUnsupported;
}

int run_combine(const CombineParams& p, hipStream_t stream) {
  if (p.B <= 0 || p.H <= 0 || p.M <= 0 || p.num_splits <= 0) return kBadArgument;
  if (p.dtype == kDtypeF16) return launch_combine<hw::half_t>(p, stream);
  if (p.dtype == kDtypeBF16) return launch_combine<hw::bf16_t>(p, stream);
  return kUnsupported;
}

}  // namespace fa
