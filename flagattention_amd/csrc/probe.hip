// Rate of the matrix pipe by itself: every compute unit runs one workgroup whose four wavefronts (one per
// SIMD) issue nothing but 32x32x16 matrix instructions from registers.  A measurement aid with no counterpart
// in the reference: the benchmark reports what this loop reaches next to the kernels' own rates, because the
// clock the device grants a busy matrix pipe depends on the operand VALUES -- with random operands the loop
// settles well below the rate it reaches with constant ones, and far below the published peak, which no
// kernel working on real data can then reach either.
#include "common.hpp"
#include "params.hpp"

namespace fa {

FA_DEVICE uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

template <class T>
FA_KERNEL void FA_LAUNCH_BOUNDS2(kThreads, 1) fa_probe_mfma_kernel(ProbeParams p) {
  using V8 = typename hw::Elem<T>::v8;
  const int tid = hw::thread_id();
  V8 a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (p.random_operands) {   // uniform in [-1, 1), different in every lane and operand
        a[j][e] = (T)(((int)(probe_hash((uint32_t)(tid * 64 + j * 8 + e)) & 0xffff) - 32768) * (1.f / 32768.f));
        b[j][e] = (T)(((int)(probe_hash((uint32_t)(tid * 64 + j * 8 + e) + 77777u) & 0xffff) - 32768) * (1.f / 32768.f));
      } else {                   // a few small integers: the products toggle next to nothing
        a[j][e] = (T)(float)((tid + e) & 3);
        b[j][e] = (T)((e & 1) ? 0.5f : -0.5f);
      }
    }
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  for (int it = 0; it < p.iters; ++it) {
#pragma unroll
    for (int m = 0; m < kProbeMfmaPerIteration; ++m)   // four independent chains, the operand pairs in turn
      acc[m & 3] = hw::mfma32(a[(m + m / 4) & 3], b[m & 3], acc[m & 3]);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[j][r];
  p.sink[(int64_t)hw::block_x() * kThreads + tid] = s;
}

int run_probe_mfma(const ProbeParams& p, hipStream_t stream) {
  if (p.iters <= 0 || p.workgroups <= 0 || !p.sink) return kBadArgument;
  // 96 KB of LDS (unused) per workgroup: no two of them share a compute unit
  const size_t lds = 96 * 1024;
  if (p.dtype == kDtypeF16) return launch(fa_probe_mfma_kernel<hw::half_t>, dim3(p.workgroups), lds, stream, p);
  if (p.dtype == kDtypeBF16) return launch(fa_probe_mfma_kernel<hw::bf16_t>, dim3(p.workgroups), lds, stream, p);
  return kUnsupported;
}

}  // namespace fa
