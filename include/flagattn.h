/*
 * C interface of libflagattn_hip.so: hand-written gfx950 (MI355X) attention kernels behind the
 * flag_attn operator API.
 *
 * Every entry point enqueues its kernels on `stream` (a hipStream_t, passed as void*) of the
 * current device and returns without synchronizing.  The library never allocates or frees device
 * memory: outputs and workspaces are caller-owned.  Return value: 0 on success, a negative
 * FA_ERR_* code for a rejected argument, a positive hipError_t if a launch failed.
 *
 * Tensors are described by fa_view4: a device pointer and element strides of a
 * (batch, head, token, D) view whose D stride is 1.  Pointers must be 16-byte aligned and the three
 * strides multiples of 8 elements.  `dtype` is FA_F16 or FA_BF16 and applies to every 16-bit tensor
 * of the call; log-normalizer, delta, total-attention and partial-softmax buffers are fp32.
 * Batch, head and query extents must be positive and pointers non-null (FA_ERR_BAD_ARGUMENT
 * otherwise): a caller with an empty problem launches nothing.  A paged sequence of context length 0
 * is valid and gets a zero output row.
 *
 * Each declaration cites the interface of the reference (FlagOpen/FlagAttention, Triton) that it
 * replaces.
 */
#ifndef FLAGATTN_H
#define FLAGATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_F16 0
#define FA_BF16 1

#define FA_ERR_BAD_ARGUMENT (-1)
#define FA_ERR_UNSUPPORTED (-2)
#define FA_ERR_SCRATCH_TOO_SMALL (-3) /* paged_attn_balanced_static: the launch needs more than FA_STATIC_SCRATCH_BYTES */

typedef struct fa_view4 {
  void* ptr;
  int64_t stride_b, stride_h, stride_t; /* in elements */
} fa_view4;

/* Library facts.  fa_version() returns the FA_ABI_VERSION the library was built from; it changes whenever an
 * entry point changes its argument list (2: fa_fwd gained block_m), and a caller built against another
 * revision must not call the library. */
#define FA_ABI_VERSION 2
int fa_version(void);
/* Number of compute units of the current device (the reference reads
 * torch.cuda.get_device_properties(...).multi_processor_count, src/flag_attn/flash.py:47-48). */
int fa_num_cus(void);

/* ------------------------------------------------------------------ flash attention, forward --
 * Replaces the launch of `_fwd_kernel` in FlashAttention.forward, src/flag_attn/flash.py:64-87
 * (kernel: flash.py:325-489).
 * q (B, H, M, D); k, v (B, Hk, N, D); o (B, H, M, D) written; lse (B, H, M) contiguous fp32 written
 * (natural-log normalizer of sm_scale * scores).  H % Hk == 0.  D in {16, 32, 64, 128}.
 * Causal masking is aligned bottom-right: row m sees key n iff m + N - M >= n; rows that see no key
 * get o = 0 and lse = -inf.
 * dropout_p in [0, 1), seed, offset: the reference's kernel arguments of the same names
 * (flash.py:328-330); with dropout_p > 0 the probability of (b, h, m, n) enters the second product
 * only if the uniform number Triton's tl.rand(seed, offset + ((b H + h) M + m) N + n, n_rounds=6) would
 * give exceeds dropout_p, and o is scaled by 1 / (1 - dropout_p); lse is unaffected.  The backward
 * entry points below take the same three values and must be given the forward's.
 * block_m: the BLOCK_M of the reference's launch (flash.py:64-66, 84: query rows per workgroup, chosen
 * by the overridable get_fwd_config).  Two kernels are compiled: 128 (every head size, dropout) and 256
 * (head size 128 without dropout: 64 rows per wavefront, one wavefront per SIMD); 0 lets the library
 * choose (256 where it applies and the launch has at least one workgroup per compute unit).  Any other
 * value, or 256 where it does not apply, returns FA_ERR_UNSUPPORTED.  The results of the two kernels
 * differ only in rounding. */
int fa_fwd(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v, const fa_view4* o,
           float* lse, int B, int H, int Hk, int M, int N, int D, int causal, float sm_scale,
           float dropout_p, uint64_t seed, uint64_t offset, int block_m, void* stream);

/* ----------------------------------------------------------------- flash attention, backward --
 * The reference's three launches in FlashAttention.backward, src/flag_attn/flash.py:191-249:
 *
 * fa_bwd_delta  <- `_bwd_preprocess` (flash.py:522-568): delta[b,h,m] = sum_d o * dout, fp32.
 * fa_bwd_dkdv   <- `_bwd_kv_kernel`  (flash.py:571-745) and, in part or in full, the group reduction
 *                  that follows it (flash.py:205-206, 250-251): dk, dv of shape
 *                  (B, H / heads_per_slice, N, D); slice s is the sum over query heads
 *                  s * heads_per_slice ... + heads_per_slice - 1 (fp32 accumulation inside the kernel).
 *                  heads_per_slice must divide H / Hk; 0 means H / Hk (one slice per kv head);
 *                  1 reproduces the reference's one slice per query head and is the only value
 *                  accepted together with dropout_p > 0.
 * fa_bwd_dq     <- `_bwd_q_kernel`   (flash.py:748-909): dq (B, H, M, D), every element written.
 * No atomics; each workgroup owns its output tile. */
int fa_bwd_delta(int dtype, const fa_view4* o, const fa_view4* dout, float* delta, int B, int H,
                 int M, int D, void* stream);
int fa_bwd_dkdv(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v,
                const fa_view4* dout, const float* lse, const float* delta, const fa_view4* dk,
                const fa_view4* dv, int heads_per_slice, int B, int H, int Hk, int M, int N, int D,
                int causal, float sm_scale, float dropout_p, uint64_t seed, uint64_t offset, void* stream);
int fa_bwd_dq(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v,
              const fa_view4* dout, const float* lse, const float* delta, const fa_view4* dq, int B,
              int H, int Hk, int M, int N, int D, int causal, float sm_scale, float dropout_p,
              uint64_t seed, uint64_t offset, void* stream);

/* The same backward with dS kept instead of recomputed (no counterpart in the reference, whose
 * `_bwd_q_kernel`, flash.py:748-909, recomputes the scores, the probabilities and dP): fa_bwd_dkdv_ds
 * is fa_bwd_dkdv that also leaves dS, rounded to the input dtype, in `ds_workspace`, and
 * fa_bwd_dq_from_ds computes dq = sm_scale * dS k from it -- one matrix product instead of three,
 * for one write and one read of a (B, H, M, N) matrix.  The workspace is device memory of at least
 * fa_bwd_ds_workspace_mib(B, H, M, N) MiB, 16-byte aligned, in a private blocked order; its contents
 * on entry do not matter.  Its size grows with the score matrix, O(M * N) per (batch, head) slice:
 * B * H * ceil(M / 128) * ceil(N / 128) * 32 KiB, i.e. 2 bytes per score with M and N rounded up to
 * 128 (128 MiB per slice at M = N = 8192, 4 GiB for 32 such slices), whether or not the mask is
 * causal.  Both calls must use the same B, H, M, N and causal flag; to bound the workspace, callers
 * may process slices of the batch or of the heads one after the other, with launches of at least
 * about 32 heads x 8192 keys if the device is to stay full. */
int fa_bwd_ds_workspace_mib(int B, int H, int M, int N);
int fa_bwd_dkdv_ds(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v,
                   const fa_view4* dout, const float* lse, const float* delta, const fa_view4* dk,
                   const fa_view4* dv, int heads_per_slice, void* ds_workspace, int64_t ds_workspace_bytes,
                   int B, int H, int Hk, int M, int N, int D, int causal, float sm_scale, float dropout_p,
                   uint64_t seed, uint64_t offset, void* stream);
int fa_bwd_dq_from_ds(int dtype, const fa_view4* k, const void* ds_workspace, int64_t ds_workspace_bytes,
                      const fa_view4* dq, int B, int H, int Hk, int M, int N, int D, int causal,
                      float sm_scale, void* stream);

/* ------------------------------------------------------------------------- total attention --
 * Replaces `_total_attention_kernel` (src/flag_attn/total.py:50-142; launches flash.py:128-140 and
 * total.py:35-46): total[b,h,n] = sum_m softmax(scores)[m,n], recomputed from q, k and lse. */
int fa_total_attn(int dtype, const fa_view4* q, const fa_view4* k, const float* lse, float* total,
                  int B, int H, int Hk, int M, int N, int D, int causal, float sm_scale,
                  void* stream);

/* ----------------------------------------------------------- split-KV forward (flash decoding) --
 * fa_splitkv_fwd     <- `_fwd_split_kv_kernel` (src/flag_attn/split_kv.py:14-160; launches
 *                       flash.py:97-111, split_kv.py:298-312).
 * fa_splitkv_combine <- `_fwd_combine_kv_splits` (split_kv.py:162-227; launches flash.py:113-125,
 *                       split_kv.py:317-329).
 * Split s covers keys [s * split_size, min(N, (s + 1) * split_size)).  part_o (B, H, S, M, D)
 * contiguous, always fp16 as in the reference (flash.py:96); part_lse (B, H, S, M) fp32.  A split
 * that holds no visible key for a row writes part_o = 0, part_lse = -inf. */
int fa_splitkv_fwd(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v, void* part_o,
                   float* part_lse, int B, int H, int Hk, int M, int N, int D, int causal,
                   float sm_scale, int num_splits, int split_size, void* stream);
int fa_splitkv_combine(int dtype, const void* part_o, const float* part_lse, const fa_view4* o,
                       float* lse, int B, int H, int M, int D, int num_splits, void* stream);

/* fa_dropout_mask <- `recompute_mask_kernel` (src/flag_attn/testing/dropout.py:5-25, launched by
 * `recompute_mask`, :19-25): writes the (B, H, M, N) contiguous mask, one byte per element (1 = kept),
 * that fa_fwd / fa_bwd_* apply for the same (dropout_p, seed, offset).  `mask` 16-byte aligned. */
int fa_dropout_mask(uint8_t* mask, int B, int H, int M, int N, float dropout_p, uint64_t seed,
                    uint64_t offset, void* stream);

/* ------------------------------------------------------------------------ piecewise attention --
 * pw_fwd      <- piecewise `_fwd_kernel`    (src/flag_attn/piecewise.py:223-370, launch :50-69)
 * pw_bwd_dkdv <- piecewise `_bwd_kv_kernel` (piecewise.py:450-627, launch :114-139)
 * pw_bwd_dq   <- piecewise `_bwd_q_kernel`  (piecewise.py:630-792, launch :141-164)
 * The score of (m, n) is q2.k2 when m + N - M - n >= dist_threshold, else q1.k1.  No grouped heads.
 * The preprocess is fa_bwd_delta (piecewise.py:407-447 is the same computation). */
int pw_fwd(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2, const fa_view4* k2,
           const fa_view4* v, const fa_view4* o, float* lse, int B, int H, int M, int N, int D,
           int dist_threshold, int causal, float sm_scale, void* stream);
int pw_bwd_dkdv(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2,
                const fa_view4* k2, const fa_view4* v, const fa_view4* dout, const float* lse,
                const float* delta, const fa_view4* dk1, const fa_view4* dk2, const fa_view4* dv,
                int B, int H, int M, int N, int D, int dist_threshold, int causal, float sm_scale,
                void* stream);
int pw_bwd_dq(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2,
              const fa_view4* k2, const fa_view4* v, const fa_view4* dout, const float* lse,
              const float* delta, const fa_view4* dq1, const fa_view4* dq2, int B, int H, int M,
              int N, int D, int dist_threshold, int causal, float sm_scale, void* stream);

/* pw_bwd_dkdv_ds + pw_bwd_dq_from_ds <- the same two reference kernels (piecewise.py:450-627 and
 * :630-792) with dS handed over instead of recomputed, as fa_bwd_dkdv_ds / fa_bwd_dq_from_ds do for
 * flash attention.  An entry of dS belongs to exactly one regime, so the workspace holds two chunk
 * grids, the near regime's (q1.k1 entries, read for dq1 = dS k1) followed by the far regime's (read
 * for dq2 = dS k2): at least 2 * fa_bwd_ds_workspace_mib(B, H, M, N) MiB, 16-byte aligned, contents
 * on entry irrelevant.  pw_bwd_dq_from_ds launches one kernel per regime and must follow, on the same
 * stream, the pw_bwd_dkdv_ds call with the same shape, dist_threshold and causal flag. */
int pw_bwd_dkdv_ds(int dtype, const fa_view4* q1, const fa_view4* k1, const fa_view4* q2,
                   const fa_view4* k2, const fa_view4* v, const fa_view4* dout, const float* lse,
                   const float* delta, const fa_view4* dk1, const fa_view4* dk2, const fa_view4* dv,
                   void* ds_workspace, int64_t ds_workspace_bytes, int B, int H, int M, int N, int D,
                   int dist_threshold, int causal, float sm_scale, void* stream);
int pw_bwd_dq_from_ds(int dtype, const fa_view4* k1, const fa_view4* k2, const void* ds_workspace,
                      int64_t ds_workspace_bytes, const fa_view4* dq1, const fa_view4* dq2, int B, int H,
                      int M, int N, int D, int dist_threshold, int causal, float sm_scale, void* stream);

/* ---------------------------------------------------------------------------- paged attention --
 * paged_attn   <- `_paged_attn_kernel` (src/flag_attn/paged.py:204-349; launches :57-88, :112-142)
 * paged_reduce <- `_paged_attn_v2_reduce_kernel` (paged.py:352-435; launch :144-162)
 *
 * query (num_seqs, Hq, D) with element strides q_stride_s, q_stride_h; key_cache / value_cache
 * (num_blocks, Hkv, block_size, D) sharing the element strides kv_stride_{blk,h,tok};
 * context_lens int32; block_tables int32 or int64 (bt_is_int64) with row stride bt_stride.
 * head_size in {16, 32, 64, 128, 256, 512} (paged.py:31).
 * partition_size == 0: one pass, `out` (num_seqs, Hq, D) with strides o_stride_s, o_stride_h.
 * partition_size > 0 (a multiple of block_size): grid over num_parts partitions; writes
 * tmp_out (num_seqs, Hkv, num_parts, G, D) in the cache dtype and max_logits / exp_sums
 * (num_seqs, Hkv, num_parts, G) fp32, to be merged by paged_reduce. */
int paged_attn(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* query,
               int64_t q_stride_s, int64_t q_stride_h, const void* key_cache, const void* value_cache,
               int64_t kv_stride_blk, int64_t kv_stride_h, int64_t kv_stride_tok,
               const int32_t* context_lens, const void* block_tables, int bt_is_int64,
               int64_t bt_stride, float attn_scale, int num_seqs, int num_q_heads, int num_kv_heads,
               int head_size, int block_size, int partition_size, int num_parts, void* tmp_out,
               float* max_logits, float* exp_sums, void* stream);
int paged_reduce(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* tmp_out,
                 const float* max_logits, const float* exp_sums, const int32_t* context_lens,
                 int num_seqs, int num_q_heads, int num_kv_heads, int head_size, int partition_size,
                 int num_parts, void* stream);


/* paged_attn_balanced <- the automatic choice of partitions in `attention` (paged.py:44-56, the
 * `num_splits == 0` branch) together with the two launches it leads to (:57-162).  Instead of
 * cutting every sequence into partitions of one size, the keys of all (sequence, kv head) pairs are
 * laid end to end and divided evenly over num_workgroups workgroups (use twice the number of compute
 * units for head_size <= 128, once above); pairs cut by a boundary are merged by a second kernel
 * launched by the same call.  `workspace` is device memory of at least
 * paged_attn_balanced_workspace(num_workgroups, head_size) bytes, 16-byte aligned; its contents on
 * entry do not matter and it may be reused by the next call on the same stream. */
int paged_attn_balanced_workspace(int num_workgroups, int head_size);
int paged_attn_balanced(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* query,
                        int64_t q_stride_s, int64_t q_stride_h, const void* key_cache,
                        const void* value_cache, int64_t kv_stride_blk, int64_t kv_stride_h,
                        int64_t kv_stride_tok, const int32_t* context_lens, const void* block_tables,
                        int bt_is_int64, int64_t bt_stride, float attn_scale, int num_seqs,
                        int num_q_heads, int num_kv_heads, int head_size, int block_size,
                        void* workspace, int64_t workspace_bytes, int num_workgroups, void* stream);

/* paged_attn_balanced_static: paged_attn_balanced for callers that cannot allocate device memory --
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose wrapper allocates its partition buffers with torch,
 * paged.py:92-108).  Same arguments and same result as paged_attn_balanced minus the workspace: the
 * partial-result slots live in a device array of FA_STATIC_SCRATCH_BYTES inside the library, which
 * every device that runs the library holds until the process ends.  The call allocates and frees
 * nothing.  The array's device address is looked up on the first call on each device, which makes the
 * runtime load the library's code object there: that first call (or paged_attn_balanced_static_prepare(),
 * which does the lookup and launches nothing) has to happen before a stream capture begins.  A launch whose
 * paged_attn_balanced_workspace(num_workgroups, head_size) exceeds FA_STATIC_SCRATCH_BYTES is rejected
 * with FA_ERR_SCRATCH_TOO_SMALL and nothing is launched (the array holds 1024 workgroups at head_size
 * <= 128 and 256 workgroups at head_size 512: more than one resident wave of a 256-CU device).  All calls on
 * one device share the one array: calls that may overlap on a device (different streams, or threads
 * that do not order their launches) race on it and must use paged_attn_balanced with separate
 * workspaces instead. */
#define FA_STATIC_SCRATCH_BYTES (17 * 1024 * 1024)
/* Looks up (and remembers) the scratch array's address on the current device; launches nothing.  Returns 0,
 * or the runtime's error.  Like paged_attn_balanced_static it has no counterpart in the reference. */
int paged_attn_balanced_static_prepare(void);
int paged_attn_balanced_static(int dtype, void* out, int64_t o_stride_s, int64_t o_stride_h, const void* query,
                               int64_t q_stride_s, int64_t q_stride_h, const void* key_cache,
                               const void* value_cache, int64_t kv_stride_blk, int64_t kv_stride_h,
                               int64_t kv_stride_tok, const int32_t* context_lens, const void* block_tables,
                               int bt_is_int64, int64_t bt_stride, float attn_scale, int num_seqs,
                               int num_q_heads, int num_kv_heads, int head_size, int block_size,
                               int num_workgroups, void* stream);

/* fa_probe_mfma: a measurement aid, no counterpart in the reference.  Enqueues one workgroup per compute unit
 * (fa_num_cus() of them, 256 threads each, one wavefront per SIMD) whose wavefronts issue nothing but
 * iters * 16 32x32x16 matrix instructions of the given dtype from registers: 2 * 32 * 32 * 16 FLOP each, so the
 * launch executes fa_num_cus() * 4 * iters * 16 * 32768 FLOP.  With random_operands != 0 the operands are uniform
 * in [-1, 1) and differ from lane to lane, otherwise they are a few small integers.  The caller times the launch
 * (events on `stream`); the clock that the device grants a busy matrix pipe, and with it the rate, depends on the
 * operand values.  sink (at least fa_num_cus() * 256 floats, sink_floats = its size) receives one float per
 * thread and only keeps the arithmetic alive. */
int fa_probe_mfma(int dtype, int random_operands, int iters, float* sink, int64_t sink_floats, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLAGATTN_H */
