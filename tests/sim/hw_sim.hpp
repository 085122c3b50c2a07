// Host stand-in for csrc/hw.hpp: runs a HIP kernel body lane by lane on the CPU.
//
// TEST INFRASTRUCTURE.  Each lane of a workgroup is a ucontext fiber; a wavefront's 64 fibers are
// run in turn up to their next collective operation (matrix multiply, transposing LDS read, lane
// exchange, workgroup barrier), the operation is evaluated for the whole wavefront with the operand
// layouts measured on gfx950, and the fibers resume.  The order in which the wavefronts of a workgroup
// advance between barriers is selectable (Schedule below), to expose a missing barrier.  LDS is a heap block of exactly the requested
// size, so AddressSanitizer sees every out-of-range LDS or global access a kernel would make.
#pragma once
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <ucontext.h>
#include <functional>
#include <vector>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define HWSIM_ASAN 1
extern "C" void __sanitizer_start_switch_fiber(void** fake_stack_save, const void* bottom, size_t size);
extern "C" void __sanitizer_finish_switch_fiber(void* fake_stack_save, const void** bottom_old, size_t* size_old);
#endif
#endif

typedef void* hipStream_t;
struct dim3 { unsigned x, y, z; dim3(unsigned a = 1, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {} };

// The few host-side HIP calls the library makes, for a "device" that is this process: one device with
// 256 compute units, device symbols are ordinary globals, a launch runs the grid to completion.
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize };
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount };
inline hipError_t hipGetDevice(int* dev) { *dev = 0; return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 256; return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void** p, const void* symbol) { *p = const_cast<void*>(symbol); return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))
#define __device__
#define __align__(n) __attribute__((aligned(n)))
#define hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, ...) \
  ::hwsim::run_grid(grid, (int)(block).x, lds_bytes, [&]() { kern(__VA_ARGS__); })

namespace hwsim {

enum Op { OP_NONE, OP_DONE, OP_BARRIER, OP_MFMA32, OP_MFMA16, OP_TR, OP_SHFL, OP_WAVESYNC };

struct Lane {
  ucontext_t ctx;
  char* stack = nullptr;
  Op op = OP_NONE;
  float a[8], b[8], c[16], out[16];
  const void* addr = nullptr;
  uint16_t tr[4];
  float sh_in = 0, sh_out = 0;
  int mask = 0;
  void* fake = nullptr;
};

constexpr size_t kStack = 256 * 1024;
inline std::vector<Lane> lanes;
inline int cur = 0;
inline ucontext_t sched_ctx;
inline void* sched_fake = nullptr;
inline const void* sched_bottom = nullptr;
inline size_t sched_size = 0;
inline int bx, by, bz, gx, gz;
inline unsigned char* lds = nullptr;
inline std::function<void()> body;

inline void to_sched() {
#ifdef HWSIM_ASAN
  __sanitizer_start_switch_fiber(&lanes[cur].fake, sched_bottom, sched_size);
#endif
  swapcontext(&lanes[cur].ctx, &sched_ctx);
#ifdef HWSIM_ASAN
  __sanitizer_finish_switch_fiber(lanes[cur].fake, &sched_bottom, &sched_size);
#endif
}
inline void yield(Op op) { lanes[cur].op = op; to_sched(); }

inline void entry() {
#ifdef HWSIM_ASAN
  __sanitizer_finish_switch_fiber(nullptr, &sched_bottom, &sched_size);
#endif
  body();
  lanes[cur].op = OP_DONE;
#ifdef HWSIM_ASAN
  __sanitizer_start_switch_fiber(nullptr, sched_bottom, sched_size);
#endif
  swapcontext(&lanes[cur].ctx, &sched_ctx);
}

inline void resume(int l) {
  cur = l;
#ifdef HWSIM_ASAN
  __sanitizer_start_switch_fiber(&sched_fake, lanes[l].stack, kStack);
#endif
  swapcontext(&sched_ctx, &lanes[l].ctx);
#ifdef HWSIM_ASAN
  __sanitizer_finish_switch_fiber(sched_fake, nullptr, nullptr);
#endif
}

inline void die(const char* msg) { fprintf(stderr, "hwsim: %s\n", msg); abort(); }

inline void eval_wave(int base, Op op) {
  Lane* L = &lanes[base];
  if (op == OP_MFMA32) {
    for (int i = 0; i < 32; ++i)
      for (int j = 0; j < 32; ++j) {
        int h = (i % 8) / 4, r = 4 * (i / 8) + i % 4;
        float s = L[h * 32 + j].c[r];
        for (int k = 0; k < 16; ++k) s += L[(k / 8) * 32 + i].a[k % 8] * L[(k / 8) * 32 + j].b[k % 8];
        L[h * 32 + j].out[r] = s;
      }
  } else if (op == OP_MFMA16) {
    for (int i = 0; i < 16; ++i)
      for (int j = 0; j < 16; ++j) {
        int q = i / 4, r = i % 4;
        float s = L[q * 16 + j].c[r];
        for (int k = 0; k < 32; ++k) s += L[(k / 8) * 16 + i].a[k % 8] * L[(k / 8) * 16 + j].b[k % 8];
        L[q * 16 + j].out[r] = s;
      }
  } else if (op == OP_TR) {
    for (int l = 0; l < 64; ++l) {
      int g = l / 16, i = l % 16;
      for (int e = 0; e < 4; ++e) {
        const uint16_t* src = (const uint16_t*)L[g * 16 + 4 * e + i / 4].addr;
        L[l].tr[e] = src[i % 4];
      }
    }
  } else if (op == OP_SHFL) {
    for (int l = 0; l < 64; ++l) L[l].sh_out = L[l ^ L[l].mask].sh_in;
  }
}

// How the wavefronts of a workgroup interleave.  Correctly synchronised kernels give the same result
// under every schedule; HWSIM_SCHEDULE picks one: "lockstep" (default: each wavefront in turn up to its
// next collective operation), "ahead" / "ahead_descending" (each wavefront runs on alone until it waits
// at a barrier or exits, lowest or highest index first: the largest skew barriers allow), "random"
// (runs of random length in random order, seeded by HWSIM_SEED).
enum ScheduleMode { kLockstep, kAheadAscending, kAheadDescending, kRandom };
struct Schedule {
  ScheduleMode mode = kLockstep;
  uint64_t rng = 1;
  uint64_t next() { rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17; return rng; }
};
inline Schedule schedule_from_env() {
  Schedule s;
  const char* m = getenv("HWSIM_SCHEDULE");
  if (!m || !*m || !strcmp(m, "lockstep")) s.mode = kLockstep;
  else if (!strcmp(m, "ahead")) s.mode = kAheadAscending;
  else if (!strcmp(m, "ahead_descending")) s.mode = kAheadDescending;
  else if (!strcmp(m, "random")) s.mode = kRandom;
  else die("HWSIM_SCHEDULE must be lockstep, ahead, ahead_descending or random");
  const char* seed = getenv("HWSIM_SEED");
  s.rng = 0x9E3779B97F4A7C15ull ^ (seed ? strtoull(seed, nullptr, 10) : 0);
  if (!s.rng) s.rng = 1;
  return s;
}

// Runs `fn` once per lane of every workgroup of the grid, one workgroup at a time.
inline void run_grid(dim3 grid, int threads, size_t lds_bytes, std::function<void()> fn) {
  if (threads % 64) die("workgroup size must be a multiple of the wavefront size");
  Schedule sched = schedule_from_env();
  body = fn;
  gx = (int)grid.x;
  gz = (int)grid.z;
  lanes.resize(threads);
  for (auto& ln : lanes)
    if (!ln.stack) ln.stack = (char*)malloc(kStack);
  int waves = threads / 64;
  std::vector<int> state(waves);  // 0 running, 1 at barrier, 2 done
  for (unsigned z = 0; z < grid.z; ++z)
    for (unsigned y = 0; y < grid.y; ++y)
      for (unsigned x = 0; x < grid.x; ++x) {
        bx = (int)x; by = (int)y; bz = (int)z;
        lds = (unsigned char*)malloc(lds_bytes ? lds_bytes : 1);
        memset(lds, 0xA5, lds_bytes);
        for (int t = 0; t < threads; ++t) {
          getcontext(&lanes[t].ctx);
          lanes[t].ctx.uc_stack.ss_sp = lanes[t].stack;
          lanes[t].ctx.uc_stack.ss_size = kStack;
          lanes[t].ctx.uc_link = nullptr;
          lanes[t].op = OP_NONE;
          makecontext(&lanes[t].ctx, (void (*)())entry, 0);
        }
        for (auto& s : state) s = 0;
        for (;;) {
          // One pass over the wavefronts in the order and with the run lengths of the chosen schedule.
          for (int i = 0; i < waves; ++i) {
            int w = sched.mode == kAheadDescending ? waves - 1 - i : sched.mode == kRandom ? (int)(sched.next() % waves) : i;
            long run = sched.mode == kLockstep ? 1 : sched.mode == kRandom ? 1 + (long)(sched.next() % 48) : (1L << 60);
            while (run-- > 0 && state[w] == 0) {
              for (int l = 0; l < 64; ++l) resume(w * 64 + l);
              Op op = lanes[w * 64].op;
              for (int l = 1; l < 64; ++l)
                if (lanes[w * 64 + l].op != op) die("lanes of one wavefront reached different collective operations");
              if (op == OP_DONE) state[w] = 2;
              else if (op == OP_BARRIER) state[w] = 1;
              else eval_wave(w * 64, op);
            }
          }
          int done = 0, waiting = 0;
          for (int s : state) { done += s == 2; waiting += s == 1; }
          if (done == waves) break;
          if (done + waiting == waves) {
            if (done) die("workgroup barrier reached by some wavefronts after others exited");
            for (auto& s : state) s = 0;
          }
        }
        free(lds);
        lds = nullptr;
      }
}

}  // namespace hwsim

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

#define FA_DEVICE inline
#define FA_KERNEL
#define FA_LAUNCH_BOUNDS(n)
#define FA_LAUNCH_BOUNDS2(n, w)
#define FA_LDS_DECL(name) unsigned char* name = ::hwsim::lds

inline int thread_id() { return hwsim::cur; }
inline int block_x() { return hwsim::bx; }
inline int block_y() { return hwsim::by; }
inline int block_z() { return hwsim::bz; }
inline void store_streaming(void* p, u32x4 v) { *(u32x4*)p = v; }
inline u32x4 load_streaming(const void* p) { return *(const u32x4*)p; }
inline void wait_global_loads() {}
template <int N>
inline void wait_lds_pending() {}
inline int uniform(int x) { return x; }
inline int grid_z() { return hwsim::gz; }
inline void block_sync() { hwsim::yield(hwsim::OP_BARRIER); }
inline void barrier_only() { hwsim::yield(hwsim::OP_BARRIER); }
inline void wave_sync() { hwsim::yield(hwsim::OP_WAVESYNC); }

template <class V8> inline f32x16 mfma32_any(V8 a, V8 b, f32x16 c) {
  hwsim::Lane& ln = hwsim::lanes[hwsim::cur];
  for (int e = 0; e < 8; ++e) { ln.a[e] = (float)a[e]; ln.b[e] = (float)b[e]; }
  for (int r = 0; r < 16; ++r) ln.c[r] = c[r];
  hwsim::yield(hwsim::OP_MFMA32);
  hwsim::Lane& l2 = hwsim::lanes[hwsim::cur];
  f32x16 d;
  for (int r = 0; r < 16; ++r) d[r] = l2.out[r];
  return d;
}
inline f32x16 mfma32(half8 a, half8 b, f32x16 c) { return mfma32_any(a, b, c); }
inline f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) { return mfma32_any(a, b, c); }
inline f32x16 zero16() { f32x16 z; for (int r = 0; r < 16; ++r) z[r] = 0.f; return z; }
// accumulator tuples that the GPU build pins to fixed physical registers: plain values here
using o_tuples = f32x16[2][4];
template <int I, class V8> inline void pinned_o_mfma(V8 a, V8 b, o_tuples& o) { o[I / 4][I % 4] = mfma32_any(a, b, o[I / 4][I % 4]); }
template <int I, class V8> inline void pinned_s_mfma_first(V8 a, V8 b, f32x16& c, o_tuples&) { c = mfma32_any(a, b, zero16()); }
template <int I, class V8> inline void pinned_s_mfma(V8 a, V8 b, f32x16& c, o_tuples&) { c = mfma32_any(a, b, c); }
template <int I> inline void pinned_o_clear(o_tuples& o) { o[I / 4][I % 4] = zero16(); }
template <int I> inline void pinned_o_scale(o_tuples& o, float f) { for (int r = 0; r < 16; ++r) o[I / 4][I % 4][r] *= f; }
template <int I, int R> inline float pinned_o_read(const o_tuples& o) { return o[I / 4][I % 4][R]; }
inline void mfma_drain() {}
inline f32x16 mfma32_vacc(half8 a, half8 b, f32x16 c) { return mfma32_any(a, b, c); }
inline f32x16 mfma32_vacc(bf16x8 a, bf16x8 b, f32x16 c) { return mfma32_any(a, b, c); }

template <class V8> inline f32x4 mfma16_any(V8 a, V8 b, f32x4 c) {
  hwsim::Lane& ln = hwsim::lanes[hwsim::cur];
  for (int e = 0; e < 8; ++e) { ln.a[e] = (float)a[e]; ln.b[e] = (float)b[e]; }
  for (int r = 0; r < 4; ++r) ln.c[r] = c[r];
  hwsim::yield(hwsim::OP_MFMA16);
  hwsim::Lane& l2 = hwsim::lanes[hwsim::cur];
  f32x4 d;
  for (int r = 0; r < 4; ++r) d[r] = l2.out[r];
  return d;
}
inline f32x4 mfma16(half8 a, half8 b, f32x4 c) { return mfma16_any(a, b, c); }
inline f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) { return mfma16_any(a, b, c); }

inline short4v lds_read_tr16(const void* p) {
  hwsim::lanes[hwsim::cur].addr = p;
  // touch the 8 bytes here so the sanitizer attributes a bad address to the lane that passed it
  volatile uint16_t probe = ((const uint16_t*)p)[0] ^ ((const uint16_t*)p)[3];
  (void)probe;
  hwsim::yield(hwsim::OP_TR);
  hwsim::Lane& ln = hwsim::lanes[hwsim::cur];
  short4v r;
  for (int e = 0; e < 4; ++e) r[e] = (short)ln.tr[e];
  return r;
}

inline u32x4 lds_load16(uint32_t addr) { return *(const u32x4*)(hwsim::lds + addr); }
inline short4v lds_read_tr16_at(uint32_t addr) { return lds_read_tr16(hwsim::lds + addr); }

inline float shfl_xor(float x, int mask) {
  hwsim::Lane& ln = hwsim::lanes[hwsim::cur];
  ln.sh_in = x;
  ln.mask = mask;
  hwsim::yield(hwsim::OP_SHFL);
  return hwsim::lanes[hwsim::cur].sh_out;
}
inline float xor32(float x) { return shfl_xor(x, 32); }
// integer exchanges ride on the float one (values are small enough to be exact)
inline int shfl_up(int x, int delta) {
  // value of lane l - delta: gather through xor exchanges of every source lane bit pattern
  int result = x;
  const int me = hwsim::cur & 63;
  for (int m = 1; m < 64; ++m) {
    const int got = (int)shfl_xor((float)x, m);
    if ((me ^ m) == me - delta) result = got;
  }
  return result;
}
inline int lane_value(int x, int lane) {
  int result = x;
  const int me = hwsim::cur & 63;
  for (int m = 1; m < 64; ++m) {
    const int got = (int)shfl_xor((float)x, m);
    if ((me ^ m) == lane) result = got;
  }
  return result;
}
inline uint64_t ballot(bool pred) {
  uint64_t mask = 0;
  const int me = hwsim::cur & 63;
  for (int m = 0; m < 64; ++m) {
    const float got = m == 0 ? (pred ? 1.f : 0.f) : shfl_xor(pred ? 1.f : 0.f, m);
    if (got > 0.f) mask |= (uint64_t)1 << (me ^ m);
  }
  return mask;
}
inline void swap_halves(float& a, float& b) {
  const bool upper = (hwsim::cur & 63) >= 32;
  const float xa = shfl_xor(a, 32), xb = shfl_xor(b, 32);
  // a' = [a.lo, b.lo], b' = [a.hi, b.hi]
  const float na = upper ? xb : a, nb = upper ? b : xa;
  a = na;
  b = nb;
}
inline void swap_halves_in_slot(float& a, float& b) { swap_halves(a, b); }
inline float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }
inline float max2(float a, float b) { return fmaxf(a, b); }
inline uint32_t lds_address(const void* p) { return (uint32_t)((const unsigned char*)p - hwsim::lds); }
inline void dma_load16(const void* base, uint32_t lane_offset, uint32_t lds_base) {
  memcpy(hwsim::lds + lds_base + 16 * (hwsim::cur & 63), (const char*)base + lane_offset, 16);
}
template <int LDS_OFFSET> inline void dma_load16_at(const void* base, uint32_t lane_offset, uint32_t lds_base) {
  dma_load16(base, lane_offset, lds_base + LDS_OFFSET);
}
inline uint32_t pack2(half_t, float a, float b) {
  half_t v[2] = {(half_t)a, (half_t)b};
  uint32_t r; memcpy(&r, v, 4); return r;
}
inline uint32_t pack2(bf16_t, float a, float b) {
  bf16_t v[2] = {(bf16_t)a, (bf16_t)b};
  uint32_t r; memcpy(&r, v, 4); return r;
}
inline bool wave_any(bool pred) {
  float v = pred ? 1.f : 0.f;
  for (int m = 1; m < 64; m <<= 1) v = fmaxf(v, shfl_xor(v, m));
  return v > 0.f;
}

inline void sched_fence() {}
inline void pin(float&) {}
inline void pin(uint32_t&) {}
template <class V> inline void keep_in_agprs(V&) {}
inline void keep_branch() {}
template <int N, int DEPTH, int RPM = 1, int EXTRA = 0> inline void sched_prefetched_operands() {}
inline float exp2_fast(float x) { return exp2f(x); }
inline float log_nat(float x) { return logf(x); }
inline float slot_fma(float a, float b, float c) { return fmaf(a, b, c); }
inline float slot_mul(float a, float b) { return a * b; }
inline float slot_exp2(float x) { return exp2f(x); }
inline float slot_max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }
inline float slot_max2(float a, float b) { return fmaxf(a, b); }
inline void slot_add(float& acc, float x) { acc += x; }
template <int C>
inline float slot_keep_if_at_least(float x, int bound) { return bound <= C ? x : 0.f; }
template <int C>
inline float slot_keep_if_below(float x, int bound) { return C < bound ? x : 0.f; }
inline uint32_t slot_pack2(half_t t, float a, float b) { return pack2(t, a, b); }
inline uint32_t slot_pack2(bf16_t t, float a, float b) { return pack2(t, a, b); }

}  // namespace hw
