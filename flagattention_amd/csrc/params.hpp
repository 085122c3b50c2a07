// Plain-data argument blocks passed by value to the kernels, and the internal entry points that the
// C interface (capi.cpp, include/flagattn.h) forwards to.
#pragma once
#include <stdint.h>

namespace fa {

// (batch, head, token, D) view: element strides, unit stride on D.
struct View4 {
  const void* ptr;
  int64_t sb, sh, st;
};

struct FwdParams {
  View4 q, k, v, q2, k2;  // q2/k2 only for the piecewise variant
  View4 o;                // written
  float* lse;             // (B, H, M) contiguous, natural-log normalizer
  int B, H, M, N, D;
  int group;              // query heads per key/value head
  int causal;
  int w;                  // piecewise distance threshold
  float sm_scale;
  int dtype;
  float dropout_p;        // 0 = no dropout; otherwise the mask is drawn from (seed, offset)
  uint64_t seed, offset;
  int block_m;            // query rows per workgroup: 128, 256, or 0 = the library's choice
  // 256-row kernel over pieces of the key axis (0 = the whole axis, results to o / lse): piece s covers keys
  // s * split_size .. + split_size - 1 and leaves its normalised output as fp16 in part_o (B, H, num_splits, M, D)
  // and its log-normalizer in part_lse (B, H, num_splits, M), the layout fa_combine_kernel merges
  int num_splits, split_size;
  void* part_o;
  float* part_lse;
};

struct BwdParams {
  View4 q, k, v, q2, k2, o, dout;
  View4 dq, dk, dv, dq2, dk2;  // written; dk/dv have one slice per `chunk` query heads
  const float* lse;            // (B, H, M)
  float* delta;                // (B, H, M) rowsum(O * dO): written by the preprocess, read by the rest
  void* ds;                    // optional dS workspace: written by the dK/dV kernel, read by dQ-from-dS
                               // (piecewise: the near regime's grid, then the far regime's)
  int regime;                  // piecewise dQ-from-dS only: 1 = near entries (k = k1), 2 = far entries (k = k2)
  int B, H, M, N, D;
  int group;
  int chunk;  // query heads whose dK/dV one workgroup accumulates (divides group; 0 = group)
  int causal;
  int w;
  float sm_scale;
  int dtype;
  float dropout_p;
  uint64_t seed, offset;
};

struct TotalParams {
  View4 q, k;
  const float* lse;  // (B, H, M)
  float* total;      // (B, H, N)
  int B, H, M, N, D;
  int group;
  int causal;
  float sm_scale;
  int dtype;
};

}  // namespace fa

#include "hw.hpp"  // hipStream_t

namespace fa {
// Compute units of the current device (0 if the runtime cannot tell); asked once per device, then remembered.
int num_cus_of_current_device();
int run_fwd(const FwdParams& p, bool piecewise, hipStream_t stream);
bool fwd_wide_supported(const FwdParams& p);   // the 256-row kernel (fa_fwd_wide.hip) can serve this launch
int run_fwd_wide(const FwdParams& p, hipStream_t stream);
struct SplitParams;
bool splitkv_wide_applies(const SplitParams& p);   // the split-KV launch is served by the 256-row kernel
int run_splitkv_wide(const SplitParams& p, hipStream_t stream);
int run_bwd_delta(const BwdParams& p, hipStream_t stream);
int run_bwd_dkdv(const BwdParams& p, bool piecewise, hipStream_t stream);
int run_bwd_dq(const BwdParams& p, bool piecewise, hipStream_t stream);
int run_total(const TotalParams& p, hipStream_t stream);
}  // namespace fa

namespace fa {

struct SplitParams {
  View4 q, k, v;
  void* part_o;      // (B, H, S, M, D) fp16, contiguous
  float* part_lse;   // (B, H, S, M)
  int B, H, M, N, D;
  int group;
  int causal;
  int num_splits, split_size;
  float sm_scale;
  int dtype;
};

struct CombineParams {
  const void* part_o;
  const float* part_lse;
  View4 o;
  float* lse;  // (B, H, M)
  int B, H, M, D, num_splits;
  int dtype;
};

struct PagedParams {
  void* out; int64_t o_ss, o_sh;          // final output (num_seqs, Hq, D) when partition_size == 0
  const void* q; int64_t q_ss, q_sh;
  const void* kc; const void* vc;
  int64_t kv_sblk, kv_sh, kv_stok;
  const int32_t* context_lens;
  const void* block_tables; int bt64; int64_t bt_stride;
  float scale;
  int num_seqs, Hq, Hkv, D, block_size;
  int partition_size, num_parts;
  void* tmp_out; float* max_logits; float* exp_sums;
  int dtype;
  // balanced launch only: partial results of workgroups that share a (sequence, kv head) pair
  float* ws; int num_wgs;
};

struct MaskParams {
  uint8_t* mask;   // (B, H, M, N) contiguous, one byte per element: 1 = kept
  int64_t total;   // B * H * M * N
  float dropout_p;
  uint64_t seed, offset;
};
int run_dropout_mask(const MaskParams& p, hipStream_t stream);

// Matrix-pipe rate probe (probe.hip): `workgroups` workgroups of four wavefronts, each wavefront issuing
// iters * kProbeMfmaPerIteration 32x32x16 matrix instructions from registers; sink takes one float per thread.
constexpr int kProbeMfmaPerIteration = 16;
struct ProbeParams {
  float* sink;
  int workgroups, iters, random_operands;
  int dtype;
};
int run_probe_mfma(const ProbeParams& p, hipStream_t stream);

int64_t bwd_ds_workspace_bytes(int B, int H, int M, int N);
int run_bwd_dkdv_ds(const BwdParams& p, bool piecewise, hipStream_t stream);
int run_bwd_dq_from_ds(const BwdParams& p, bool piecewise, hipStream_t stream);
int run_splitkv(const SplitParams& p, hipStream_t stream);
int run_combine(const CombineParams& p, hipStream_t stream);
int run_paged(const PagedParams& p, hipStream_t stream);
int run_paged_reduce(const PagedParams& p, hipStream_t stream);
int64_t paged_balanced_workspace_bytes(int num_wgs, int D);
int run_paged_balanced(const PagedParams& p, hipStream_t stream);

}  // namespace fa
