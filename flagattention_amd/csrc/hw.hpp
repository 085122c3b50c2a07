// Thin layer over the gfx950 (CDNA4) instructions the attention kernels are built from.
//
// Every kernel in this directory reaches the hardware only through the functions declared here:
// 64-lane wavefronts, v_mfma_f32_32x32x16_{f16,bf16}, ds_read_b64_tr_b16, a lane^32 exchange and
// v_exp_f32.  The operand layouts documented below were checked on an MI355X with one-off probes.
//
// A second implementation of the same functions (tests/sim/hw_sim.hpp, selected by
// FLAGATTN_HOST_SIM) runs the unchanged kernel sources lane by lane on the host, with bounds-checked
// memory, so that index arithmetic can be debugged without a GPU.  It is test infrastructure; the
// shipped library is always built from the gfx950 half of this file.
#pragma once
#include <stdint.h>

#ifdef FLAGATTN_HOST_SIM
#include "hw_sim.hpp"
#else
#include <hip/hip_runtime.h>

namespace hw {

using half_t = _Float16;
using bf16_t = __bf16;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define FA_DEVICE __device__ __forceinline__
#define FA_KERNEL __global__
#define FA_LAUNCH_BOUNDS(n) __launch_bounds__(n)
#define FA_LAUNCH_BOUNDS2(n, w) __launch_bounds__(n, w)
#define FA_LDS_DECL(name) extern __shared__ __attribute__((aligned(16))) unsigned char name[]

FA_DEVICE int thread_id() { return (int)threadIdx.x; }
FA_DEVICE int block_x() { return (int)blockIdx.x; }
FA_DEVICE int block_y() { return (int)blockIdx.y; }
FA_DEVICE int block_z() { return (int)blockIdx.z; }
FA_DEVICE int grid_z() { return (int)gridDim.z; }
FA_DEVICE void block_sync() { __syncthreads(); }
// The workgroup barrier alone, without the memory fence of block_sync(): for code that has already
// waited for the accesses it needs ordered.
FA_DEVICE void barrier_only() { __builtin_amdgcn_s_barrier(); }
// Orders the LDS traffic of one wavefront: writes issued by any lane before the call are visible
// to reads issued by any lane after it (LDS serves a wavefront's requests in order; this only stops
// the compiler from moving accesses across).
FA_DEVICE void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// D(32x32) += A(32x16) * B(16x32).  Lane l holds, for h = l / 32:
//   A[i = l % 32][k = 8h + e], e = 0..7          B[k = 8h + e][j = l % 32]
//   D[i = 8 * (r / 4) + 4h + r % 4][j = l % 32], r = 0..15
FA_DEVICE f32x16 mfma32(half8 a, half8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
FA_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
// The same product with the accumulator pinned to VGPRs and the B operand to AGPRs.  Left to itself
// the compiler keeps every accumulator of a kernel that may use all 512 registers in AGPRs, from where
// each element costs a v_accvgpr_read before the vector ALU can touch it; here the accumulator is what
// the vector ALU works on and the B operand (a register-resident K or V row) is what can live in AGPRs.
// The compiler does not see into the assembly, so the CALLER keeps the distance the hardware needs
// between this instruction and a vector-ALU read of its result: another matrix instruction in between.
FA_DEVICE f32x16 mfma32_vacc(half8 a, half8 b, f32x16 c) {
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  return c;
}
FA_DEVICE f32x16 mfma32_vacc(bf16x8 a, bf16x8 b, f32x16 c) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  return c;
}
// max(a, b, c) and max(a, b) as single instructions (no canonicalisation of the inputs: callers pass
// matrix-instruction results and values derived from them)
FA_DEVICE float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
FA_DEVICE float max2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
// More wait states than any matrix instruction needs before its result may be read by other units.
FA_DEVICE void mfma_drain() { asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7" ::: "memory"); }
// Moves a register-resident operand to AGPRs for good (what mfma32_vacc takes as B).
template <class V>
FA_DEVICE void keep_in_agprs(V& v) { asm volatile("" : "+a"(v)); }
// D(16x16) += A(16x32) * B(32x16).  Lane l holds, for q = l / 16:
//   A[i = l % 16][k = 8q + e]     B[k = 8q + e][j = l % 16]     D[i = 4q + r][j = l % 16], r = 0..3
FA_DEVICE f32x4 mfma16(half8 a, half8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
FA_DEVICE f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Transposing 64-bit LDS read over 16-bit elements.  Within each group of 16 lanes, lane i passes
// the address of 4 consecutive elements in[i][0..3] and receives
//   out[i][e] = in[4e + i / 4][i % 4],  e = 0..3
// i.e. if lane c points at row c / 4, columns 4 * (c % 4).. of a row-major 4 x 16 patch, lane i gets
// column i of that patch.
FA_DEVICE short4v lds_read_tr16(const void* lds_ptr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) short4v*)(uintptr_t)lds_ptr);
}

// LDS accesses by byte address (as returned by lds_address()): the address arithmetic stays in
// 32-bit registers and constant parts fold into the instruction's offset field.
FA_DEVICE u32x4 lds_load16(uint32_t addr) {
  return *(const __attribute__((address_space(3))) u32x4*)(uintptr_t)addr;
}
FA_DEVICE short4v lds_read_tr16_at(uint32_t addr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(uintptr_t)addr);
}

// True in every lane if the predicate holds in any lane of the wavefront.
FA_DEVICE bool wave_any(bool pred) { return __builtin_amdgcn_ballot_w64(pred) != 0; }

// Lanes of the wavefront in which the predicate holds, as a bit mask.
FA_DEVICE uint64_t ballot(bool pred) { return __builtin_amdgcn_ballot_w64(pred); }
// Value held by lane l - delta (lanes below delta keep their own), and by a given lane.
FA_DEVICE int shfl_up(int x, int delta) { return __shfl_up(x, delta, 64); }
FA_DEVICE int lane_value(int x, int lane) { return __shfl(x, lane, 64); }

// Value held by lane (l ^ 32).
FA_DEVICE float xor32(float x) { return __shfl_xor(x, 32, 64); }
// Value held by lane (l ^ mask) for mask < 64.
FA_DEVICE float shfl_xor(float x, int mask) { return __shfl_xor(x, mask, 64); }

// Exchanges the upper 32 lanes of a with the lower 32 lanes of b (one instruction):
//   a' = [a.lo, b.lo],  b' = [a.hi, b.hi]
FA_DEVICE void swap_halves(float& a, float& b) {
  // written as assembly: the compiler's lowering of the corresponding builtin returns the first result
  // for both halves of its result pair.  The wait states around it are the ones the compiler places
  // around the instruction itself (vector-ALU results feeding it, its results feeding the vector ALU).
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}

// The exchange alone, for hand-placed streams: the CALLER keeps two instructions that do not touch a or b on
// either side of it.
FA_DEVICE void swap_halves_in_slot(float& a, float& b) { asm volatile("v_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }

// Tells the compiler that x has the same value in every lane (kept in a scalar register).
FA_DEVICE int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// 16-byte global accesses for data that is written once and read once much later (or read once):
// marked non-temporal so that they do not displace the tiles the kernel re-reads from the L2.
FA_DEVICE void store_streaming(void* p, u32x4 v) { __builtin_nontemporal_store(v, (u32x4*)p); }
FA_DEVICE u32x4 load_streaming(const void* p) { return __builtin_nontemporal_load((const u32x4*)p); }

// 16 bytes per lane from global memory straight into LDS, no register in between: lane i's bytes land
// at LDS byte address lds_base + 16 i (lds_base wave-uniform, a multiple of 16); the source address is
// base (wave-uniform) + lane_offset bytes.  Completion is counted like any global load
// (wait_global_loads()); the compiler is not told that LDS changes, so the caller orders the LDS reads
// of that region behind the wait and a barrier itself.
FA_DEVICE void dma_load16(const void* base, uint32_t lane_offset, uint32_t lds_base) {
  // (one wait state between the scalar write of M0 and the instruction that reads it)
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_offset), "s"(base), "s"(lds_base) : "memory", "m0");
}
// The same with a compile-time addition to the LDS base (a fixed place inside a rotating stage): the sum goes
// straight into M0, one scalar instruction.
template <int LDS_OFFSET>
FA_DEVICE void dma_load16_at(const void* base, uint32_t lane_offset, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               : : "v"(lane_offset), "s"(base), "s"(lds_base), "n"(LDS_OFFSET) : "memory", "m0", "scc");
}
// LDS byte address of a pointer into the workgroup's LDS allocation.
FA_DEVICE uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// Waits until every global load issued so far has delivered its registers.  Placed between the
// loads of loop-invariant operands and a loop that also prefetches: otherwise the compiler puts the
// wait at the operands' first use INSIDE the loop, where it also covers the prefetch just issued.
FA_DEVICE void wait_global_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0), others unconstrained
// Waits until at most N of the LDS accesses issued so far are still outstanding (they complete in order).  The
// compiler places such waits itself, one in front of every first use of a read's result; an explicit one that
// covers the reads of two consumers lets it drop the second's.
template <int N>
FA_DEVICE void wait_lds_pending() {
  static_assert(N >= 0 && N <= 15, "the counter has four bits");
  __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));   // lgkmcnt(N), vmcnt and expcnt unconstrained
}

// Marks a branch body as not speculatable, so that a wavefront-uniform `if` stays a branch instead
// of being turned into unconditional arithmetic on selected operands.
FA_DEVICE void keep_branch() { asm volatile("" ::: "memory"); }

// Makes the compiler materialise x at this point of the instruction stream: the scheduling fence only
// binds the instruction scheduler, while earlier passes sink a side-effect-free computation towards its
// first use, across fences and branches.  Costs no instruction.
FA_DEVICE void pin(float& x) { asm volatile("" : "+v"(x)); }
FA_DEVICE void pin(uint32_t& x) { asm volatile("" : "+v"(x)); }

// Nothing is scheduled across this point by the compiler (software-pipelining fence).
FA_DEVICE void sched_fence() { __builtin_amdgcn_sched_barrier(0); }

// Scheduling hint for a region of N matrix instructions that each consume an operand fetched by RPM
// LDS reads: keep the operands of DEPTH matrix instructions in flight ahead of their consumer.
// EXTRA other LDS reads precede the first operand read.
template <int N, int DEPTH, int RPM = 1, int EXTRA = 0>
FA_DEVICE void sched_prefetched_operands() {
  __builtin_amdgcn_sched_group_barrier(0x100, DEPTH * RPM + EXTRA, 0);
#pragma unroll
  for (int i = 0; i < N - DEPTH; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, RPM, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, DEPTH, 0);
}

FA_DEVICE float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
FA_DEVICE float log_nat(float x) { return __logf(x); }

// Vector-ALU steps that stay exactly where the source puts them ("slotted" variants for the hand-placed
// instruction streams).  The scheduling fence binds the instruction scheduler only: earlier passes move
// side-effect-free arithmetic across it, towards its operands or its first use, and so fill one slot with the
// work of two and leave the next one empty.  A wavefront that is alone on its SIMD issues one instruction per
// 4 clocks whatever its kind (8 for an exponential), so what a slot holds beyond about five instructions is not
// hidden under its matrix instruction; these keep a slot's share in that slot.  The compiler does not see into
// them: the CALLER keeps one other instruction between an exponential and the first use of its result.
FA_DEVICE float slot_fma(float a, float b, float c) {
  float r;
  asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
FA_DEVICE float slot_mul(float a, float b) {
  float r;
  asm volatile("v_mul_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
FA_DEVICE float slot_exp2(float x) {
  float r;
  asm volatile("v_exp_f32 %0, %1" : "=v"(r) : "v"(x));
  return r;
}
FA_DEVICE float slot_max3(float a, float b, float c) {
  float r;
  asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
FA_DEVICE float slot_max2(float a, float b) {
  float r;
  asm volatile("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
FA_DEVICE void slot_add(float& acc, float x) { asm volatile("v_add_f32 %0, %0, %1" : "+v"(acc) : "v"(x)); }
// x where bound <= C, else 0 (a select, so that an infinite x leaves no NaN); C an inline integer constant.
// Writes vcc.  x must not be the result of the instruction right before (the compiler adds no wait state here).
template <int C>
FA_DEVICE float slot_keep_if_at_least(float x, int bound) {
  static_assert(C >= -16 && C <= 64, "inline constant");
  asm volatile("v_cmp_ge_i32 vcc, %2, %1\n\tv_cndmask_b32 %0, 0, %0, vcc" : "+v"(x) : "v"(bound), "n"(C) : "vcc");
  return x;
}
// x where C < bound, else 0: the same for a mask that ends inside the tile.
template <int C>
FA_DEVICE float slot_keep_if_below(float x, int bound) {
  static_assert(C >= -16 && C <= 64, "inline constant");
  asm volatile("v_cmp_lt_i32 vcc, %2, %1\n\tv_cndmask_b32 %0, 0, %0, vcc" : "+v"(x) : "v"(bound), "n"(C) : "vcc");
  return x;
}
FA_DEVICE uint32_t slot_pack2(half_t, float a, float b) {
  uint32_t r;
  asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
FA_DEVICE uint32_t slot_pack2(bf16_t, float a, float b) {
  uint32_t r;
  asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// Two fp32 values rounded to T and packed (lo = a, hi = b), and acc + lo + hi of such a pair.
FA_DEVICE uint32_t pack2(half_t, float a, float b) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 v; v[0] = (_Float16)a; v[1] = (_Float16)b;
  return __builtin_bit_cast(uint32_t, v);
}
FA_DEVICE uint32_t pack2(bf16_t, float a, float b) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  b2 v; v[0] = (__bf16)a; v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

}  // namespace hw
#include "pinned_regs.hpp"
#endif  // FLAGATTN_HOST_SIM

namespace hw {

template <int V> struct int_tag { static constexpr int value = V; };

template <class T> struct Elem;
template <> struct Elem<half_t> { using v8 = half8; };
template <> struct Elem<bf16_t> { using v8 = bf16x8; };

// 16 bytes of raw bits <-> 8 elements
template <class T> FA_DEVICE typename Elem<T>::v8 as_v8(u32x4 raw) {
  return __builtin_bit_cast(typename Elem<T>::v8, raw);
}
template <class T> FA_DEVICE typename Elem<T>::v8 join_v8(short4v lo, short4v hi) {
  short8v s = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename Elem<T>::v8, s);
}
template <class T> FA_DEVICE uint16_t bits16(float x) {
  T t = (T)x;
  return __builtin_bit_cast(uint16_t, t);
}
template <class T> FA_DEVICE float from_bits16(uint16_t b) {
  return (float)__builtin_bit_cast(T, b);
}

}  // namespace hw
