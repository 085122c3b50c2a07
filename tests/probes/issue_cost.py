#!/usr/bin/env python3
"""Issue-cost probe for gfx950: what one instruction of each kind costs a wavefront that shares its SIMD with
nobody (or with one other wavefront) while the matrix pipe is busy.

A *slot* is one ``v_mfma_f32_32x32x16_bf16`` followed by a literal list of other instructions; a kernel runs
16 slots per loop iteration, written as ONE assembly block so that the compiler adds nothing, on one workgroup per
compute unit (96 KB of LDS keeps a second one away) of 256 threads (one wavefront per SIMD) or 512 (two).  The
program prints, per variant, nanoseconds and shader clocks (``s_memtime``) per slot.  The kernels compute nothing
and touch no global memory except one float per thread at the end.

    python tests/probes/issue_cost.py --build      # writes build/issue_cost.hip and compiles it (no GPU needed)
    tests/probes/build/issue_cost                  # on the GPU: prints the table

Measurement infrastructure for the design notes; nothing in the package uses it.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
BUILD = os.path.join(HERE, "build")
variants = []   # (name, threads, mfma(bool), per-slot instruction list as function of slot index m)
def V(name, threads, mf, fn): variants.append((name, threads, mf, fn))

def rep(tmpl, n):
    return lambda m: [tmpl.format(i=i, a=100 + (i % 8), b=108 + (i % 8), c=116 + (i % 8), m=m) for i in range(n)]

kinds = {
  'fma':      'v_fma_f32 v{a}, v{b}, v{c}, v{a}',
  'exp':      'v_exp_f32 v{a}, v{b}',
  'snop':     's_nop 0',
  'salu':     's_add_u32 s40, s40, 1',
  'waitcnt':  's_waitcnt lgkmcnt(15)',
  'cvtpk':    'v_cvt_pk_bf16_f32 v{a}, v{b}, v{c}',
  'max3':     'v_max3_f32 v100, v100, v{b}, v{c}',
  'accread':  'v_accvgpr_read_b32 v{a}, a{i}',
  'mov':      'v_mov_b32 v{a}, v{b}',
  'dsread':   'ds_read_b128 v[{q}:{q3}], v124 offset:1024',
}
def dsread(n):
    def f(m):
        out = []
        for i in range(n):
            q = 100 + 4 * ((m * n + i) % 4)
            out.append(f'ds_read_b128 v[{q}:{q+3}], v124 offset:1024')
        if m % 4 == 3: out.append(f's_waitcnt lgkmcnt({min(15, 2 * n)})')
        return out
    return f
def mix(extra_valu=0, extra_salu=0, extra_ds=0):
    def f(m):
        out = ['v_fma_f32 v100, v108, v109, v110', f'v_exp_f32 v{101 + m % 2}, v111', f'v_add_f32 v{103 + m % 2}, v{103 + m % 2}, v112']
        out.append('v_cvt_pk_bf16_f32 v105, v112, v113' if m % 2 else 'v_max3_f32 v106, v106, v108, v109')
        for i in range(extra_valu): out.append(f'v_fma_f32 v{116 + i % 4}, v108, v109, v{116 + i % 4}')
        for i in range(extra_salu): out.append('s_add_u32 s40, s40, 1')
        if extra_ds:
            q = 120; out.append(f'ds_read_b128 v[{100 + 20}:{100 + 23}], v124 offset:1024') if m % 4 < extra_ds else None
            if m % 4 == 3: out.append('s_waitcnt lgkmcnt(4)')
        return out
    return f

for t in (256, 512):
    V('mfma only', t, True, lambda m: [])
for kind in ('fma', 'exp', 'snop', 'salu', 'waitcnt', 'cvtpk', 'max3', 'accread', 'mov'):
    V(f'no mfma, 8 x {kind}', 256, False, rep(kinds[kind], 8))
V('no mfma, 4 x dsread', 256, False, dsread(4))
for kind in ('fma', 'exp', 'salu'):
    V(f'no mfma, 8 x {kind}', 512, False, rep(kinds[kind], 8))
for kind in ('fma', 'exp', 'snop', 'salu', 'waitcnt', 'cvtpk', 'accread'):
    for n in (1, 2, 4, 6, 7, 8, 10, 12):
        V(f'mfma + {n:2d} x {kind}', 256, True, rep(kinds[kind], n))
for n in (1, 2, 3, 4): V(f'mfma + {n} x dsread', 256, True, dsread(n))
V('mfma + softmax mix (3 valu + exp)', 256, True, mix())
for ev in (1, 2, 3): V(f'mfma + mix + {ev} valu', 256, True, mix(ev))
for es in (2, 4, 6): V(f'mfma + mix + {es} salu', 256, True, mix(0, es))
V('mfma + mix + 2 valu + 3 salu + ds', 256, True, mix(2, 3, 3))
# two wavefronts per SIMD
for kind in ('fma', 'exp', 'salu', 'snop'):
    for n in (1, 2, 4, 6, 8, 12):
        V(f'mfma + {n:2d} x {kind}', 512, True, rep(kinds[kind], n))
for n in (1, 2): V(f'mfma + {n} x dsread', 512, True, dsread(n))
V('mfma + softmax mix (3 valu + exp)', 512, True, mix())
for ev in (1, 2, 3): V(f'mfma + mix + {ev} valu', 512, True, mix(ev))
for es in (2, 4, 6): V(f'mfma + mix + {es} salu', 512, True, mix(0, es))
V('mfma + mix + 2 valu + 3 salu + ds', 512, True, mix(2, 3, 3))

src = ['''#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %d\\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
#define CLOB "memory", "s40", ''' + ', '.join(f'"v{i}"' for i in range(100, 128)) + ', ' + ', '.join(f'"a{i}"' for i in range(64)) + '''
''']
for idx, (name, threads, mf, fn) in enumerate(variants):
    body = []
    for m in range(16):
        if mf: body.append(f'v_mfma_f32_32x32x16_bf16 a[{16 * (m % 4)}:{16 * (m % 4) + 15}], %0, %1, a[{16 * (m % 4)}:{16 * (m % 4) + 15}]')
        body += [x for x in fn(m) if x]
    text = '\\n\\t'.join(body) if body else 's_nop 0'
    init = '\\n\\t'.join([f'v_accvgpr_write_b32 a{i}, 0' for i in range(64)] + [f'v_mov_b32 v{i}, 0x3c000000' for i in range(100, 124)] +
                         ['v_mov_b32 v124, %2', 's_mov_b32 s40, 0'])
    src.append(f'''__global__ void __launch_bounds__({threads}) k{idx}(float* out, long long* cyc, int iters) {{
  extern __shared__ unsigned char smem[];
  for (int i = threadIdx.x; i < 4096; i += {threads}) ((unsigned*)smem)[i] = i;
  __syncthreads();
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {{ a[i] = (__bf16)(float)((threadIdx.x + i) & 3); b[i] = (__bf16)((i & 1) ? 0.5f : -0.5f); }}
  const unsigned lds_addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem + (threadIdx.x & 63) * 16;
  long long t0 = 0, t1 = 0;
  asm volatile("{init}" : : "v"(a), "v"(b), "v"(lds_addr) : CLOB);
  t0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; ++it) {{
    asm volatile("{text}" : : "v"(a), "v"(b), "v"(lds_addr) : CLOB);
  }}
  asm volatile("s_waitcnt lgkmcnt(0)\\n\\ts_nop 15\\n\\ts_nop 15" : : : CLOB);
  t1 = __builtin_readcyclecounter();
  float s; asm volatile("v_accvgpr_read_b32 %0, a5\\n\\tv_add_f32 %0, %0, v100\\n\\tv_add_f32 %0, %0, v106" : "=v"(s) : : CLOB);
  out[(size_t)blockIdx.x * {threads} + threadIdx.x] = s;
  if (threadIdx.x == 0) cyc[blockIdx.x] = t1 - t0;
}}
''')
src.append('''static float* d_out; static long long* d_cyc; static long long h_cyc[256];
typedef void (*kern_t)(float*, long long*, int);
static void run(kern_t kf, int threads, const char* name) {
  const int iters = 4000;
  hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
  CHECK(hipFuncSetAttribute((const void*)kf, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));   // one workgroup per CU
  hipLaunchKernelGGL(kf, dim3(256), dim3(threads), 96 * 1024, 0, d_out, d_cyc, 50);
  CHECK(hipEventRecord(e0));
  hipLaunchKernelGGL(kf, dim3(256), dim3(threads), 96 * 1024, 0, d_out, d_cyc, iters);
  CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1)); CHECK(hipGetLastError());
  float ms; CHECK(hipEventElapsedTime(&ms, e0, e1));
  CHECK(hipMemcpy(h_cyc, d_cyc, sizeof(h_cyc), hipMemcpyDeviceToHost));
  double c = 0; for (int i = 0; i < 256; ++i) c += (double)h_cyc[i];
  c /= 256.0;
  const double slots = iters * 16.0, waves = threads / 256.0;
  printf("%-40s waves/SIMD %d : %7.2f ns/slot %7.1f ticks/slot | per SIMD %6.2f ns per slot\\n", name, threads / 256,
         ms * 1e6 / slots, c / slots, ms * 1e6 / slots / waves);
  fflush(stdout);
}
int main() {
  CHECK(hipMalloc(&d_out, 256 * 1024 * sizeof(float)));
  CHECK(hipMalloc(&d_cyc, 256 * sizeof(long long)));
''')
src.append(f'  run(k0, 256, "warm-up"); run(k0, 256, "warm-up");\n')
for idx, (name, threads, mf, fn) in enumerate(variants):
    src.append(f'  run(k{idx}, {threads}, "{name}");\n')
src.append('  return 0;\n}\n')


def main():
    os.makedirs(BUILD, exist_ok=True)
    path = os.path.join(BUILD, "issue_cost.hip")
    with open(path, "w") as f:
        f.write("".join(src))
    print(f"{len(variants)} variants -> {path}")
    if "--build" in sys.argv:
        subprocess.run(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
                        "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", path, "-o",
                        os.path.join(BUILD, "issue_cost")], check=True, stderr=subprocess.DEVNULL)


if __name__ == "__main__":
    main()
