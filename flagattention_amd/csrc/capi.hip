// extern "C" surface of the library: validates arguments, fills the kernels' parameter blocks and
// forwards to the launchers.  Declarations and the reference interfaces they replace are in
// include/flagattn.h.
#include "../../include/flagattn.h"
#include "params.hpp"

namespace {

constexpr int kVersion = 1;

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

extern "C" {

int fa_version(void) { return kVersion; }

int fa_num_cus(void) {
#ifdef FLAGATTN_HOST_SIM
  return 256;
#else
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
  return n;
#endif
}

int fa_fwd(int dtype, const fa_view4* q, const fa_view4* k, const fa_view4* v, const fa_view4* o,
           float* lse, int B, int H, int Hk, int M, int N, int D, int causal, float sm_scale,
           void* stream) {
  if (!view_ok(q) || !view_ok(k) || !view_ok(v) || !view_ok(o) || !lse) return FA_ERR_BAD_ARGUMENT;
  if (!head_dim_ok(D)) return FA_ERR_UNSUPPORTED;
  if (Hk <= 0 || H % Hk) return FA_ERR_BAD_ARGUMENT;
  fa::FwdParams p = {};
  p.q = to_view(q); p.k = to_view(k); p.v = to_view(v); p.o = to_view(o);
  p.lse = lse;
  p.B = B; p.H = H; p.M = M; p.N = N; p.D = D;
  p.group = H / Hk;
  p.causal = causal; p.w = 0; p.sm_scale = sm_scale; p.dtype = dtype;
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

}  // extern "C"
