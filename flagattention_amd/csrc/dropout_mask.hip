// The dropout mask as a tensor: which score elements flash attention keeps for a given
// (dropout_p, seed, offset).  Replaces `recompute_mask_kernel` (src/flag_attn/testing/dropout.py:5-25),
// with which callers and tests rebuild the mask that the forward and backward kernels drew on the fly.
// Element i of the contiguous (B, H, M, N) mask uses the Philox counter offset + i (common.hpp).
// Bound: the Philox rounds (about 60 integer instructions per byte written).
#include "common.hpp"
#include "params.hpp"

namespace fa {

constexpr int kMaskPerThread = 16;  // one 16-byte store

FA_KERNEL void FA_LAUNCH_BOUNDS(kThreads) fa_dropout_mask_kernel(MaskParams p) {
  const int64_t first = ((int64_t)hw::block_x() * kThreads + hw::thread_id()) * kMaskPerThread;
  if (first >= p.total) return;
  uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < kMaskPerThread; ++e) {
    const bool keep = dropout_keeps(p.offset + (uint64_t)(first + e), p.seed, p.dropout_p);
    w[e >> 2] |= (keep ? 1u : 0u) << (8 * (e & 3));
  }
  if (first + kMaskPerThread <= p.total) {
    *(u32x4*)(p.mask + first) = u32x4{w[0], w[1], w[2], w[3]};
  } else {
    for (int e = 0; first + e < p.total; ++e) p.mask[first + e] = (uint8_t)((w[e >> 2] >> (8 * (e & 3))) & 1u);
  }
}

int run_dropout_mask(const MaskParams& p, hipStream_t stream) {
  if (!p.mask || p.total <= 0 || !(p.dropout_p >= 0.f && p.dropout_p < 1.f)) return kBadArgument;
  if (((uintptr_t)p.mask) & 15) return kBadArgument;
  const int64_t per_wg = (int64_t)kThreads * kMaskPerThread;
  const int64_t wgs = (p.total + per_wg - 1) / per_wg;
  if (wgs > 0x7fffffff) return kUnsupported;
  return launch(fa_dropout_mask_kernel, dim3((unsigned)wgs, 1, 1), 0, stream, p);
}

}  // namespace fa
