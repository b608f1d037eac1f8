// extern "C" surface of the library: argument validation (before any HIP call), error text, dispatch.
#include "../../include/corope_amd.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>

#include "kernels.hpp"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr float kLog2e = 1.4426950408889634f;

int check_ptrs(const char* what, std::initializer_list<const void*> ptrs) {
  for (const void* p : ptrs) {
    if (p == nullptr) return fail(COROPE_E_BADARG, "%s: null pointer argument", what);
    if (!aligned16(p)) return fail(COROPE_E_ALIGN, "%s: pointer %p is not 16-byte aligned", what, p);
  }
  return COROPE_OK;
}

int launch_status(const char* what, hipError_t e) {
  if (e == hipSuccess) return COROPE_OK;
  return fail(COROPE_E_LAUNCH, "%s: HIP error %d (%s)", what, (int)e, hipGetErrorString(e));
}

corope::BwdParams make_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                           const float* lse, float* delta, const float* c, const float* s, int64_t fstride, void* dq,
                           void* dk, void* dv, int B, int H, int N, float sm_scale) {
  corope::BwdParams p{};
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<const uint16_t*>(o);
  p.d_o = static_cast<const uint16_t*>(d_o);
  p.cos = c;
  p.sin = s;
  p.lse = lse;
  p.delta = delta;
  p.dq = static_cast<uint16_t*>(dq);
  p.dk = static_cast<uint16_t*>(dk);
  p.dv = static_cast<uint16_t*>(dv);
  p.fstride = fstride;
  p.sm_scale = sm_scale;
  p.qk_scale = sm_scale * kLog2e;
  p.N = N;
  p.BH = B * H;
  return p;
}

}  // namespace

extern "C" {

int corope_amd_version(void) { return 1; }

const char* corope_amd_last_error(void) { return g_err; }

int corope_rope_attn_check(int B, int H, int N, int D, int64_t freq_row_stride, float sm_scale, int backward) {
  (void)backward;
  if (B <= 0 || H <= 0 || N <= 0) return fail(COROPE_E_BADARG, "rope_attn: B, H, N must be positive (got %d, %d, %d)", B, H, N);
  if (D != 64 && D != 128) return fail(COROPE_E_UNSUPPORTED, "rope_attn: head dim %d not built (64 and 128 are)", D);
  if (freq_row_stride < D / 2 || freq_row_stride % 4 != 0)
    return fail(COROPE_E_BADARG, "rope_attn: freq_row_stride %lld must be >= D/2 and a multiple of 4", (long long)freq_row_stride);
  if (!(sm_scale > 0.f) || !std::isfinite(sm_scale)) return fail(COROPE_E_BADARG, "rope_attn: sm_scale must be positive and finite");
  if ((int64_t)B * H * N * D >= ((int64_t)1 << 40)) return fail(COROPE_E_UNSUPPORTED, "rope_attn: tensor too large");
  g_err[0] = 0;
  return COROPE_OK;
}

int corope_gqa_check(int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0) return fail(COROPE_E_BADARG, "corope_gqa: sizes must be positive");
  if (Hq % Hkv != 0) return fail(COROPE_E_BADARG, "corope_gqa: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  if (Hq / Hkv > 8) return fail(COROPE_E_UNSUPPORTED, "corope_gqa: group size %d exceeds 8", Hq / Hkv);
  if (D != 64 && D != 128) return fail(COROPE_E_UNSUPPORTED, "corope_gqa: head dim %d not built (64 and 128 are)", D);
  if (!std::isfinite(sm_scale)) return fail(COROPE_E_BADARG, "corope_gqa: sm_scale must be finite");
  if (!(theta > 0.f) || !std::isfinite(theta)) return fail(COROPE_E_BADARG, "corope_gqa: theta must be positive and finite");
  g_err[0] = 0;
  return COROPE_OK;
}

int corope_rope_attn_fwd(const void* q, const void* k, const void* v, const float* freqs_cos, const float* freqs_sin,
                         int64_t freq_row_stride, void* o, float* lse, int B, int H, int N, int D, float sm_scale,
                         int causal, void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 0);
  if (rc) return rc;
  rc = check_ptrs("rope_attn_fwd", {q, k, v, freqs_cos, freqs_sin, o, lse});
  if (rc) return rc;
  corope::FwdParams p{};
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.cos = freqs_cos;
  p.sin = freqs_sin;
  p.o = static_cast<uint16_t*>(o);
  p.lse = lse;
  p.fstride = freq_row_stride;
  p.qk_scale = sm_scale * kLog2e;
  p.N = N;
  p.BH = B * H;
  return launch_status("rope_attn_fwd", corope::launch_rope_attn_fwd(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

int corope_rope_attn_bwd_preprocess(const void* o, const void* d_o, float* delta, int B, int H, int N, int D,
                                    void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, D, 1.f, 1);
  if (rc) return rc;
  rc = check_ptrs("rope_attn_bwd_preprocess", {o, d_o, delta});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(nullptr, nullptr, nullptr, o, d_o, nullptr, delta, nullptr, nullptr, D, nullptr,
                                 nullptr, nullptr, B, H, N, 1.f);
  return launch_status("rope_attn_bwd_preprocess", corope::launch_bwd_preprocess(p, D, static_cast<hipStream_t>(stream)));
}

int corope_rope_attn_bwd_dv(const void* q, const void* k, const void* d_o, const float* lse, const float* freqs_cos,
                            const float* freqs_sin, int64_t freq_row_stride, void* dv, int B, int H, int N, int D,
                            float sm_scale, int causal, void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs("rope_attn_bwd_dv", {q, k, d_o, lse, freqs_cos, freqs_sin, dv});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q, k, nullptr, nullptr, d_o, lse, nullptr, freqs_cos, freqs_sin, freq_row_stride,
                                 nullptr, nullptr, dv, B, H, N, sm_scale);
  return launch_status("rope_attn_bwd_dv", corope::launch_bwd_dv(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

int corope_rope_attn_bwd_dk(const void* q, const void* k, const void* v, const void* d_o, const float* lse,
                            const float* delta, const float* freqs_cos, const float* freqs_sin,
                            int64_t freq_row_stride, void* dk, int B, int H, int N, int D, float sm_scale, int causal,
                            void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs("rope_attn_bwd_dk", {q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, dk});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q, k, v, nullptr, d_o, lse, const_cast<float*>(delta), freqs_cos, freqs_sin,
                                 freq_row_stride, nullptr, dk, nullptr, B, H, N, sm_scale);
  return launch_status("rope_attn_bwd_dk", corope::launch_bwd_dk(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

int corope_rope_attn_bwd_dkdv(const void* q, const void* k, const void* v, const void* d_o, const float* lse,
                              const float* delta, const float* freqs_cos, const float* freqs_sin,
                              int64_t freq_row_stride, void* dk, void* dv, int B, int H, int N, int D, float sm_scale,
                              int causal, void* stream) {
  int rc = check_ptrs("rope_attn_bwd_dkdv", {v, delta, dk, dv});
  if (rc) return rc;
  rc = corope_rope_attn_bwd_dv(q, k, d_o, lse, freqs_cos, freqs_sin, freq_row_stride, dv, B, H, N, D, sm_scale, causal,
                               stream);
  if (rc) return rc;
  return corope_rope_attn_bwd_dk(q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dk, B, H, N, D,
                                 sm_scale, causal, stream);
}

int corope_rope_attn_bwd_dq(const void* q, const void* k, const void* v, const void* d_o, const float* lse,
                            const float* delta, const float* freqs_cos, const float* freqs_sin,
                            int64_t freq_row_stride, void* dq, int B, int H, int N, int D, float sm_scale, int causal,
                            void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs("rope_attn_bwd_dq", {q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, dq});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q, k, v, nullptr, d_o, lse, const_cast<float*>(delta), freqs_cos, freqs_sin,
                                 freq_row_stride, dq, nullptr, nullptr, B, H, N, sm_scale);
  return launch_status("rope_attn_bwd_dq", corope::launch_bwd_dq(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

int corope_rope_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                         float* delta, const float* freqs_cos, const float* freqs_sin, int64_t freq_row_stride,
                         void* dq, void* dk, void* dv, int B, int H, int N, int D, float sm_scale, int causal,
                         void* stream) {
  int rc = corope_rope_attn_bwd_preprocess(o, d_o, delta, B, H, N, D, stream);
  if (rc) return rc;
  rc = corope_rope_attn_bwd_dkdv(q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dk, dv, B, H, N, D,
                                 sm_scale, causal, stream);
  if (rc) return rc;
  return corope_rope_attn_bwd_dq(q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dq, B, H, N, D,
                                 sm_scale, causal, stream);
}

int corope_rope_freqs(float* freqs_cos, float* freqs_sin, int n_pos, int D, int width, int64_t freq_row_stride, int pos0,
                      float theta, void* stream) {
  if (n_pos <= 0 || D <= 0 || D % 2 != 0) return fail(COROPE_E_BADARG, "rope_freqs: n_pos must be positive and D even");
  if (D > 128) return fail(COROPE_E_UNSUPPORTED, "rope_freqs: head dim %d exceeds 128", D);
  if (width != D && width != D / 2) return fail(COROPE_E_BADARG, "rope_freqs: width must be D or D/2 (got %d)", width);
  if (freq_row_stride < width) return fail(COROPE_E_BADARG, "rope_freqs: row stride smaller than the row");
  if (pos0 < 0 || !(theta > 0.f) || !std::isfinite(theta)) return fail(COROPE_E_BADARG, "rope_freqs: bad pos0 or theta");
  if ((int64_t)n_pos * (D / 2) >= ((int64_t)1 << 31)) return fail(COROPE_E_UNSUPPORTED, "rope_freqs: table too large");
  if (freqs_cos == nullptr || freqs_sin == nullptr) return fail(COROPE_E_BADARG, "rope_freqs: null pointer argument");
  g_err[0] = 0;
  return launch_status("rope_freqs", corope::launch_rope_freqs(freqs_cos, freqs_sin, n_pos, D, width, freq_row_stride,
                                                               pos0, theta, static_cast<hipStream_t>(stream)));
}

int corope_gqa_fwd(const void* q, const void* k, const void* v, void* o, int B, int Hq, int Hkv, int N, int D,
                   float sm_scale, float theta, void* stream) {
  int rc = corope_gqa_check(B, Hq, Hkv, N, D, sm_scale, theta);
  if (rc) return rc;
  rc = check_ptrs("corope_gqa_fwd", {q, k, v, o});
  if (rc) return rc;
  corope::CoropeParams p{};
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<uint16_t*>(o);
  p.sm_scale = sm_scale;
  p.theta = theta;
  p.B = B;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.N = N;
  return launch_status("corope_gqa_fwd", corope::launch_corope_gqa_fwd(p, D, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
