// extern "C" surface of the library: validates arguments, fills the kernels' parameter blocks and
// forwards to the launchers.  Declarations and the reference interfaces they replace are in
// include/flagattn.h.
#include "../../include/flagattn.h"
#include "params.hpp"

#include <atomic>

namespace {

constexpr int kVersion = FA_ABI_VERSION;

bool head_dim_ok(int D) { return D == 16 || D == 32 || D == 64 || D == 128; }

bool view_ok(const fa_view4* v) {
  if (!v || !v->ptr) return false;
  if (((uintptr_t)v->ptr) & 15) return false;
  return (v->stride_b % 8 == 0) && (v->stride_h % 8 == 0) && (v->stride_t % 8 == 0);
}

fa::View4 to_view(const fa_view4* v) {
  fa::View4 r;
  r.ptr = v ? v->ptr : nullptr;
  r.sb = v ? v->stride_b : 0;
  r.sh = v ? v->stride_h : 0;
  r.st = v ? v->stride_t : 0;
  return r;
}

}  // namespace

namespace fa {
int num_cus_of_current_device() {
  constexpr int kDevices = 64;
  static std::atomic<int> known[kDevices];
  int dev = -1, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return 0;
  if (dev < kDevices) {
    n = known[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
  }
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
  if (dev < kDevices) known[dev].store(n, std::memory_order_relaxed);
  return n;
}
}  // namespace fa

extern "C" {

int fa_version(void) { return kVersion; }

int fa_num_cus(void) {
  const int n = fa::num_cus_of_current_device();
  return n > 0 ? n : -1;
}

int fa_fwd(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v, const fa_view4* o,
           float* lse, int B, int H, int Hk, int M, int N, int D, int causal, float sm_scale,
           float dropout_p, uint64_t seed, uint64_t offset, int block_m, void* stream) {
  if (!view_ok(q) || !view_ok(k) || !view_ok(v) || !view_ok(o) || !lse) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  if (Hk <= 0 || H % Hk) return FA_ERR_BAD_ARGUMENT;
  fa::FwdParams p = {};
  p.q = to_view(q); p.k = to_view(k); p.v = to_view(v); p.o = to_view(o);
  p.lse = lse;
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D;
  p.group = H / Hk;
  p.causal = causal; p.w = 0; p.sm_scale = sm_scale; p.dtype = dtype;
  p.dropout_p = dropout_p; p.seed = seed; p.offset = offset;
  p.block_m = block_m;
  return fa::run_fwd(p, false, (hipStream_t)stream);
}

int pw_fwd(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2, const fa_view4* k2,
           const fa_view4* v, const fa_view4* o, float* lse, int B, int H, int M, int N, int D,
           int dist_threshold, int causal, float sm_scale, void* stream) {
  if (!view_ok(q1) || !view_ok(k1) || !view_ok(q2) || !view_ok(k2) || !view_ok(v) || !view_ok(o) || !lse)
    return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  fa::FwdParams p = {};
  p.q = to_view(q1); p.k = to_view(k1); p.q2 = to_view(q2); p.k2 = to_view(k2);
  p.v = to_view(v); p.o = to_view(o);
  p.lse = lse;
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D;
  p.group = 1;
  p.causal = causal; p.w = dist_threshold; p.sm_scale = sm_scale; p.dtype = dtype;
  return fa::run_fwd(p, true, (hipStream_t)stream);
}

int fa_bwd_delta(int dtype, const fa_view4* o, const fa_view4* dout, float* delta, int B, int H,
                 int M, int D, void* stream) {
  if (!view_ok(o) || !view_ok(dout) || !delta) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  fa::BwdParams p = {};
  p.o = to_view(o); p.dout = to_view(dout); p.delta = delta;
  p.B = B; p.H = H; p.M = M; p.D = D; p.dtype = dtype;
  return fa::run_bwd_delta(p, (hipStream_t)stream);
}

static int fill_bwd(fa::BwdParams& p, int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v,
                    const fa_view4* dout, const float* lse, const float* delta, int B, int H, int Hk,
                    int M, int N, int D, int causal, float sm_scale) {
  if (!view_ok(q) || !view_ok(k) || !view_ok(v) || !view_ok(dout) || !lse || !delta)
    return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  if (Hk <= 0 || H % Hk) return FA_ERR_BAD_ARGUMENT;
  p.q = to_view(q); p.k = to_view(k); p.v = to_view(v); p.dout = to_view(dout);
  p.lse = lse; p.delta = const_cast<float*>(delta);
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D;
  p.group = H / Hk; p.causal = causal; p.sm_scale = sm_scale; p.dtype = dtype;
  return 0;
}

int fa_bwd_dkdv(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v,
                const fa_view4* dout, const float* lse, const float* delta, const fa_view4* dk,
                const fa_view4* dv, int heads_per_slice, int B, int H, int Hk, int M, int N, int D,
                int causal, float sm_scale, float dropout_p, uint64_t seed, uint64_t offset, void* stream) {
  fa::BwdParams p = {};
  int rc = fill_bwd(p, dtype, q, k, v, dout, lse, delta, B, H, Hk, M, N, D, causal, sm_scale);
  if (rc) return rc;
  if (!view_ok(dk) || !view_ok(dv)) return FA_ERR_BAD_ARGUMENT;
  p.dk = to_view(dk); p.dv = to_view(dv);
  p.chunk = heads_per_slice;
  p.dropout_p = dropout_p; p.seed = seed; p.offset = offset;
  return fa::run_bwd_dkdv(p, false, (hipStream_t)stream);
}

int fa_bwd_dq(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v,
              const fa_view4* dout, const float* lse, const float* delta, const fa_view4* dq, int B,
              int H, int Hk, int M, int N, int D, int causal, float sm_scale, float dropout_p,
              uint64_t seed, uint64_t offset, void* stream) {
  fa::BwdParams p = {};
  int rc = fill_bwd(p, dtype, q, k, v, dout, lse, delta, B, H, Hk, M, N, D, causal, sm_scale);
  if (rc) return rc;
  if (!view_ok(dq)) return FA_ERR_BAD_ARGUMENT;
  p.dq = to_view(dq);
  p.dropout_p = dropout_p; p.seed = seed; p.offset = offset;
  return fa::run_bwd_dq(p, false, (hipStream_t)stream);
}

int fa_bwd_ds_workspace_mib(int B, int H, int M, int N) {
  if (B <= 0 || H <= 0 || M <= 0 || N <= 0) return FA_ERR_BAD_ARGUMENT;
  const int64_t mib = (fa::bwd_ds_workspace_bytes(B, H, M, N) + (1 << 20) - 1) >> 20;
  return mib > 0x7fffffff ? FA_ERR_BAD_ARGUMENT : (int)mib;
}

int fa_bwd_dkdv_ds(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v,
                   const fa_view4* dout, const float* lse, const float* delta, const fa_view4* dk,
                   const fa_view4* dv, int heads_per_slice, void* ds_workspace, int64_t ds_workspace_bytes,
                   int B, int H, int Hk, int M, int N, int D, int causal, float sm_scale, float dropout_p,
                   uint64_t seed, uint64_t offset, void* stream) {
  fa::BwdParams p = {};
  int rc = fill_bwd(p, dtype, q, k, v, dout, lse, delta, B, H, Hk, M, N, D, causal, sm_scale);
  if (rc) return rc;
  if (!view_ok(dk) || !view_ok(dv)) return FA_ERR_BAD_ARGUMENT;
  if (!ds_workspace || (((uintptr_t)ds_workspace) & 15) ||
      ds_workspace_bytes < fa::bwd_ds_workspace_bytes(B, H, M, N))
    return FA_ERR_BAD_ARGUMENT;
  p.dk = to_view(dk); p.dv = to_view(dv);
  p.chunk = heads_per_slice;
  p.dropout_p = dropout_p; p.seed = seed; p.offset = offset;
  p.ds = ds_workspace;
  return fa::run_bwd_dkdv_ds(p, false, (hipStream_t)stream);
}

int fa_bwd_dq_from_ds(int dtype, const fa_view4* k, const void* ds_workspace, int64_t ds_workspace_bytes,
                      const fa_view4* dq, int B, int H, int Hk, int M, int N, int D, int causal,
                      float sm_scale, void* stream) {
  if (!view_ok(k) || !view_ok(dq)) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  if (B <= 0 || H <= 0 || Hk <= 0 || H % Hk || M <= 0 || N <= 0) return FA_ERR_BAD_ARGUMENT;
  if (!ds_workspace || (((uintptr_t)ds_workspace) & 15) ||
      ds_workspace_bytes < fa::bwd_ds_workspace_bytes(B, H, M, N))
    return FA_ERR_BAD_ARGUMENT;
  fa::BwdParams p = {};
  p.k = to_view(k); p.dq = to_view(dq);
  p.ds = const_cast<void*>(ds_workspace);
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D; p.group = H / Hk;
  p.causal = causal; p.sm_scale = sm_scale; p.dtype = dtype;
  return fa::run_bwd_dq_from_ds(p, false, (hipStream_t)stream);
}

int pw_bwd_dkdv(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2,
                const fa_view4* k2, const fa_view4* v, const fa_view4* dout, const float* lse,
                const float* delta, const fa_view4* dk1, const fa_view4* dk2, const fa_view4* dv,
                int B, int H, int M, int N, int D, int dist_threshold, int causal, float sm_scale,
                void* stream) {
  fa::BwdParams p = {};
  int rc = fill_bwd(p, dtype, q1, k1, v, dout, lse, delta, B, H, H, M, N, D, causal, sm_scale);
  if (rc) return rc;
  if (!view_ok(q2) || !view_ok(k2) || !view_ok(dk1) || !view_ok(dk2) || !view_ok(dv))
    return FA_ERR_BAD_ARGUMENT;
  p.q2 = to_view(q2); p.k2 = to_view(k2);
  p.dk = to_view(dk1); p.dk2 = to_view(dk2); p.dv = to_view(dv);
  p.w = dist_threshold;
  return fa::run_bwd_dkdv(p, true, (hipStream_t)stream);
}

int pw_bwd_dq(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2,
              const fa_view4* k2, const fa_view4* v, const fa_view4* dout, const float* lse,
              const float* delta, const fa_view4* dq1, const fa_view4* dq2, int B, int H, int M,
              int N, int D, int dist_threshold, int causal, float sm_scale, void* stream) {
  fa::BwdParams p = {};
  int rc = fill_bwd(p, dtype, q1, k1, v, dout, lse, delta, B, H, H, M, N, D, causal, sm_scale);
  if (rc) return rc;
  if (!view_ok(q2) || !view_ok(k2) || !view_ok(dq1) || !view_ok(dq2)) return FA_ERR_BAD_ARGUMENT;
  p.q2 = to_view(q2); p.k2 = to_view(k2);
  p.dq = to_view(dq1); p.dq2 = to_view(dq2);
  p.w = dist_threshold;
  return fa::run_bwd_dq(p, true, (hipStream_t)stream);
}

int pw_bwd_dkdv_ds(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2,
                   const fa_view4* k2, const fa_view4* v, const fa_view4* dout, const float* lse,
                   const float* delta, const fa_view4* dk1, const fa_view4* dk2, const fa_view4* dv,
                   void* ds_workspace, int64_t ds_workspace_bytes, int B, int H, int M, int N, int D,
                   int dist_threshold, int causal, float sm_scale, void* stream) {
  fa::BwdParams p = {};
  int rc = fill_bwd(p, dtype, q1, k1, v, dout, lse, delta, B, H, H, M, N, D, causal, sm_scale);
  if (rc) return rc;
  if (!view_ok(q2) || !view_ok(k2) || !view_ok(dk1) || !view_ok(dk2) || !view_ok(dv))
    return FA_ERR_BAD_ARGUMENT;
  if (!ds_workspace || (((uintptr_t)ds_workspace) & 15) ||
      ds_workspace_bytes < 2 * fa::bwd_ds_workspace_bytes(B, H, M, N))
    return FA_ERR_BAD_ARGUMENT;
  p.q2 = to_view(q2); p.k2 = to_view(k2);
  p.dk = to_view(dk1); p.dk2 = to_view(dk2); p.dv = to_view(dv);
  p.w = dist_threshold;
  p.ds = ds_workspace;
  return fa::run_bwd_dkdv_ds(p, true, (hipStream_t)stream);
}

int pw_bwd_dq_from_ds(int dtype, const fa_view4* k1, const fa_view4* k2, const void* ds_workspace,
                      int64_t ds_workspace_bytes, const fa_view4* dq1, const fa_view4* dq2, int B, int H,
                      int M, int N, int D, int dist_threshold, int causal, float sm_scale, void* stream) {
  if (!view_ok(k1) || !view_ok(k2) || !view_ok(dq1) || !view_ok(dq2)) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  if (B <= 0 || H <= 0 || M <= 0 || N <= 0) return FA_ERR_BAD_ARGUMENT;
  if (!ds_workspace || (((uintptr_t)ds_workspace) & 15) ||
      ds_workspace_bytes < 2 * fa::bwd_ds_workspace_bytes(B, H, M, N))
    return FA_ERR_BAD_ARGUMENT;
  fa::BwdParams p = {};
  p.ds = const_cast<void*>(ds_workspace);
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D; p.group = 1;
  p.causal = causal; p.w = dist_threshold; p.sm_scale = sm_scale; p.dtype = dtype;
  p.k = to_view(k1); p.dq = to_view(dq1); p.regime = 1;
  int rc = fa::run_bwd_dq_from_ds(p, true, (hipStream_t)stream);
  if (rc) return rc;
  p.k = to_view(k2); p.dq = to_view(dq2); p.regime = 2;
  return fa::run_bwd_dq_from_ds(p, true, (hipStream_t)stream);
}

int fa_dropout_mask(uint8_t* mask, int B, int H, int M, int N, float dropout_p, uint64_t seed,
                    uint64_t offset, void* stream) {
  if (B <= 0 || H <= 0 || M <= 0 || N <= 0) return FA_ERR_BAD_ARGUMENT;
  fa::MaskParams p = {};
  p.mask = mask;
  p.total = (int64_t)B * H * M * N;
  p.dropout_p = dropout_p; p.seed = seed; p.offset = offset;
  return fa::run_dropout_mask(p, (hipStream_t)stream);
}

int fa_total_attn(int dtype, const fa_view4* q, const fa_view4* k, const float* lse, float* total,
                  int B, int H, int Hk, int M, int N, int D, int causal, float sm_scale,
                  void* stream) {
  if (!view_ok(q) || !view_ok(k) || !lse || !total) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  if (Hk <= 0 || H % Hk) return FA_ERR_BAD_ARGUMENT;
  fa::TotalParams p = {};
  p.q = to_view(q); p.k = to_view(k); p.lse = lse; p.total = total;
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D;
  p.group = H / Hk; p.causal = causal; p.sm_scale = sm_scale; p.dtype = dtype;
  return fa::run_total(p, (hipStream_t)stream);
}

int fa_splitkv_fwd(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v, void* part_o,
                   float* part_lse, int B, int H, int Hk, int M, int N, int D, int causal,
                   float sm_scale, int num_splits, int split_size, void* stream) {
  if (!view_ok(q) || !view_ok(k) || !view_ok(v) || !part_o || !part_lse) return FA_ERR_BAD_ARGUMENT;
  if (((uintptr_t)part_o) & 15) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  if (Hk <= 0 || H % Hk) return FA_ERR_BAD_ARGUMENT;
  fa::SplitParams p = {};
  p.q = to_view(q); p.k = to_view(k); p.v = to_view(v);
  p.part_o = part_o; p.part_lse = part_lse;
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D;
  p.group = H / Hk; p.causal = causal;
  p.num_splits = num_splits; p.split_size = split_size;
  p.sm_scale = sm_scale; p.dtype = dtype;
  return fa::run_splitkv(p, (hipStream_t)stream);
}

int fa_splitkv_combine(int dtype, const void* part_o, const float* part_lse, const fa_view4* o,
                       float* lse, int B, int H, int M, int D, int num_splits, void* stream) {
  if (!part_o || !part_lse || !view_ok(o) || !lse) return FA_ERR_BAD_ARGUMENT;
  if (((uintptr_t)part_o) & 15) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  fa::CombineParams p = {};
  p.part_o = part_o; p.part_lse = part_lse; p.o = to_view(o); p.lse = lse;
  p.B = B; p.H = H; p.M = M; p.D = D; p.num_splits = num_splits; p.dtype = dtype;
  return fa::run_combine(p, (hipStream_t)stream);
}

static int fill_paged(fa::PagedParams& p, int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h,
                      const int32_t* context_lens, int num_seqs, int num_q_heads, int num_kv_heads,
                      int head_size, int partition_size, int num_parts, void* tmp_out, float* max_logits,
                      float* exp_sums) {
  if (!out || !context_lens) return FA_ERR_BAD_ARGUMENT;
  if (partition_size > 0 && (!tmp_out || !max_logits || !exp_sums)) return FA_ERR_BAD_ARGUMENT;
  p.out = out; p.o_ss = o_stride_s; p.o_sh = o_stride_h;
  p.context_lens = context_lens;
  p.num_seqs = num_seqs; p.Hq = num_q_heads; p.Hkv = num_kv_heads; p.D = head_size;
  p.partition_size = partition_size; p.num_parts = num_parts;
  p.tmp_out = tmp_out; p.max_logits = max_logits; p.exp_sums = exp_sums;
  p.dtype = dtype;
  return 0;
}

int paged_attn(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* query,
               int64_t q_stride_s, int64_t q_stride_h, const void* key_cache, const void* value_cache,
               int64_t kv_stride_blk, int64_t kv_stride_h, int64_t kv_stride_tok,
               const int32_t* context_lens, const void* block_tables, int bt_is_int64,
               int64_t bt_stride, float attn_scale, int num_seqs, int num_q_heads, int num_kv_heads,
               int head_size, int block_size, int partition_size, int num_parts, void* tmp_out,
               float* max_logits, float* exp_sums, void* stream) {
  fa::PagedParams p = {};
  int rc = fill_paged(p, dtype, out, o_stride_s, o_stride_h, context_lens, num_seqs, num_q_heads,
                      num_kv_heads, head_size, partition_size, num_parts, tmp_out, max_logits, exp_sums);
  if (rc) return rc;
  if (!query || !key_cache || !value_cache || !block_tables) return FA_ERR_BAD_ARGUMENT;
  if ((((uintptr_t)query) | ((uintptr_t)key_cache) | ((uintptr_t)value_cache)) & 15) return FA_ERR_BAD_ARGUMENT;
  if ((q_stride_s | q_stride_h | kv_stride_blk | kv_stride_h | kv_stride_tok) % 8) return FA_ERR_BAD_ARGUMENT;
  if (!(head_size == 16 || head_size == 32 || head_size == 64 || head_size == 128 || head_size == 256 || head_size == 512))
    return FA_ERR_UNSUPPORTED;
  p.q = query; p.q_ss = q_stride_s; p.q_sh = q_stride_h;
  p.kc = key_cache; p.vc = value_cache;
  p.kv_sblk = kv_stride_blk; p.kv_sh = kv_stride_h; p.kv_stok = kv_stride_tok;
  p.block_tables = block_tables; p.bt64 = bt_is_int64; p.bt_stride = bt_stride;
  p.scale = attn_scale; p.block_size = block_size;
  return fa::run_paged(p, (hipStream_t)stream);
}

int paged_attn_balanced_workspace(int num_workgroups, int head_size) {
  if (num_workgroups <= 0 || head_size <= 0) return FA_ERR_BAD_ARGUMENT;
  const int64_t bytes = fa::paged_balanced_workspace_bytes(num_workgroups, head_size);
  return bytes > 0x7fffffff ? FA_ERR_BAD_ARGUMENT : (int)bytes;
}

int paged_attn_balanced(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* query,
                        int64_t q_stride_s, int64_t q_stride_h, const void* key_cache,
                        const void* value_cache, int64_t kv_stride_blk, int64_t kv_stride_h,
                        int64_t kv_stride_tok, const int32_t* context_lens, const void* block_tables,
                        int bt_is_int64, int64_t bt_stride, float attn_scale, int num_seqs,
                        int num_q_heads, int num_kv_heads, int head_size, int block_size,
                        void* workspace, int64_t workspace_bytes, int num_workgroups, void* stream) {
  fa::PagedParams p = {};
  int rc = fill_paged(p, dtype, out, o_stride_s, o_stride_h, context_lens, num_seqs, num_q_heads,
                      num_kv_heads, head_size, 0, 1, nullptr, nullptr, nullptr);
  if (rc) return rc;
  if (!query || !key_cache || !value_cache || !block_tables || !workspace) return FA_ERR_BAD_ARGUMENT;
  if ((((uintptr_t)query) | ((uintptr_t)key_cache) | ((uintptr_t)value_cache) | ((uintptr_t)workspace)) & 15)
    return FA_ERR_BAD_ARGUMENT;
  if ((q_stride_s | q_stride_h | kv_stride_blk | kv_stride_h | kv_stride_tok) % 8) return FA_ERR_BAD_ARGUMENT;
  if (!(head_size == 16 || head_size == 32 || head_size == 64 || head_size == 128 || head_size == 256 || head_size == 512))
    return FA_ERR_UNSUPPORTED;
  if (num_workgroups <= 0 || workspace_bytes < fa::paged_balanced_workspace_bytes(num_workgroups, head_size))
    return FA_ERR_BAD_ARGUMENT;
  p.q = query; p.q_ss = q_stride_s; p.q_sh = q_stride_h;
  p.kc = key_cache; p.vc = value_cache;
  p.kv_sblk = kv_stride_blk; p.kv_sh = kv_stride_h; p.kv_stok = kv_stride_tok;
  p.block_tables = block_tables; p.bt64 = bt_is_int64; p.bt_stride = bt_stride;
  p.scale = attn_scale; p.block_size = block_size;
  p.ws = (float*)workspace; p.num_wgs = num_workgroups;
  return fa::run_paged_balanced(p, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------
// paged_attn_balanced without a caller-provided workspace: the partial-result slots and the
// per-workgroup records live in a device array that is part of the library's code object.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[FA_STATIC_SCRATCH_BYTES];

namespace {
// The array's name is only a host-side handle; each device that loads the library holds its own copy
// at its own address, looked up once per device (with that device current) and kept here.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_of_device[kMaxDevices];

int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return FA_ERR_UNSUPPORTED;
  void* ptr = g_scratch_of_device[dev].load(std::memory_order_acquire);
  if (!ptr) {  // first call on this device; a concurrent first call looks up the same address
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return FA_ERR_UNSUPPORTED;
    g_scratch_of_device[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return 0;
}
}  // namespace

int paged_attn_balanced_static_prepare(void) {
  void* ws = nullptr;
  return scratch_of_current_device(&ws);
}

int paged_attn_balanced_static(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* query,
                               int64_t q_stride_s, int64_t q_stride_h, const void* key_cache,
                               const void* value_cache, int64_t kv_stride_blk, int64_t kv_stride_h,
                               int64_t kv_stride_tok, const int32_t* context_lens, const void* block_tables,
                               int bt_is_int64, int64_t bt_stride, float attn_scale, int num_seqs,
                               int num_q_heads, int num_kv_heads, int head_size, int block_size,
                               int num_workgroups, void* stream) {
  if (num_workgroups <= 0 || head_size <= 0) return FA_ERR_BAD_ARGUMENT;
  const int64_t need = fa::paged_balanced_workspace_bytes(num_workgroups, head_size);
  if (need > (int64_t)FA_STATIC_SCRATCH_BYTES) return FA_ERR_SCRATCH_TOO_SMALL;
  void* ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc) return rc;
  // nothing in the scratch has to start at zero: every slot and record that the merge kernel reads was
  // written by the attention kernel of the same call
  return paged_attn_balanced(dtype, out, o_stride_s, o_stride_h, query, q_stride_s, q_stride_h, key_cache,
                             value_cache, kv_stride_blk, kv_stride_h, kv_stride_tok, context_lens,
                             block_tables, bt_is_int64, bt_stride, attn_scale, num_seqs, num_q_heads,
                             num_kv_heads, head_size, block_size, ws, need, num_workgroups, stream);
}

int fa_probe_mfma(int dtype, int random_operands, int iters, float* sink, int64_t sink_floats, void* stream) {
  const int cus = fa::num_cus_of_current_device();
  if (cus <= 0) return FA_ERR_UNSUPPORTED;
  if (iters <= 0 || !sink || sink_floats < (int64_t)cus * 256) return FA_ERR_BAD_ARGUMENT;
  fa::ProbeParams p = {};
  p.sink = sink; p.workgroups = cus; p.iters = iters; p.random_operands = random_operands; p.dtype = dtype;
  return fa::run_probe_mfma(p, (hipStream_t)stream);
}

int paged_reduce(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* tmp_out,
                 const float* max_logits, const float* exp_sums, const int32_t* context_lens,
                 int num_seqs, int num_q_heads, int num_kv_heads, int head_size, int partition_size,
                 int num_parts, void* stream) {
  fa::PagedParams p = {};
  int rc = fill_paged(p, dtype, out, o_stride_s, o_stride_h, context_lens, num_seqs, num_q_heads,
                      num_kv_heads, head_size, partition_size, num_parts, const_cast<void*>(tmp_out),
                      const_cast<float*>(max_logits), const_cast<float*>(exp_sums));
  if (rc) return rc;
  p.block_size = 1;
  return fa::run_paged_reduce(p, (hipStream_t)stream);
}

}  // extern "C"
