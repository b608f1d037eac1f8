// extern "C" surface of the library: argument validation (before any HIP call), error text, dispatch.
#include "../../include/corope_amd.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>

#include "kernels.hpp"

#ifdef COROPE_TRACE
// Measurement builds only (libcorope_amd_trace.so): where the attention kernels write their time stamps, or null.
namespace corope { uint64_t* g_trace_buf = nullptr; }
extern "C" void corope_debug_trace(void* buf) { corope::g_trace_buf = static_cast<uint64_t*>(buf); }
#endif

namespace corope {
namespace {
// An environment variable that must hold one of `allowed` (anything else, or unset: 0 = the library's own choice).
int env_choice(const char* name, std::initializer_list<int> allowed) {
  const char* e = getenv(name);
  if (e == nullptr) return 0;
  const int v = atoi(e);
  for (int a : allowed)
    if (v == a) return v;
  return 0;
}
}  // namespace
// Kernel forms are picked by shape.  For diagnostics two environment variables, read ONCE when the library is loaded,
// override the pick for the whole process: COROPE_AMD_TILE_ROWS (128 or 256 rows per workgroup item) and
// COROPE_AMD_FWD_WAVE_ROWS (32 or 64 query rows per wave, or 128: 128-row items with two workgroups per compute unit, in the two-launch forward at D = 128).  The shipped library has
// no call that changes them afterwards; the measurement build (libcorope_amd_trace.so) has one, for the tests.
std::atomic<int> g_tile_rows{env_choice("COROPE_AMD_TILE_ROWS", {128, 256})};
std::atomic<int> g_fwd_wave_rows{env_choice("COROPE_AMD_FWD_WAVE_ROWS", {32, 64, 128})};
}  // namespace corope

#ifdef COROPE_TRACE
extern "C" int corope_debug_set_forms(int tile_rows, int fwd_wave_rows) {
  if ((tile_rows != 0 && tile_rows != 128 && tile_rows != 256) || (fwd_wave_rows != 0 && fwd_wave_rows != 32 && fwd_wave_rows != 64 && fwd_wave_rows != 128))
    return COROPE_E_BADARG;
  corope::g_tile_rows.store(tile_rows);
  corope::g_fwd_wave_rows.store(fwd_wave_rows);
  return COROPE_OK;
}
#endif

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
  p.H = p.Hkv = H;
  return p;
}

}  // namespace

extern "C" {

int corope_amd_version(void) { return 3; }

const char* corope_amd_last_error(void) { return g_err; }

int corope_rope_attn_check(int B, int H, int N, int D, int64_t freq_row_stride, float sm_scale, int backward) {
  (void)backward;
  if (B <= 0 || H <= 0 || N <= 0) return fail(COROPE_E_BADARG, "rope_attn: B, H, N must be positive (got %d, %d, %d)", B, H, N);
  if (D != 64 && D != 128 && D != 256)
    return fail(COROPE_E_UNSUPPORTED, "rope_attn: head dim %d not built (64, 128 and 256 are)", D);
  if (freq_row_stride < D / 2 || freq_row_stride % 4 != 0)
    return fail(COROPE_E_BADARG, "rope_attn: freq_row_stride %lld must be >= D/2 and a multiple of 4", (long long)freq_row_stride);
  if (!(sm_scale > 0.f) || !std::isfinite(sm_scale)) return fail(COROPE_E_BADARG, "rope_attn: sm_scale must be positive and finite");
  if ((int64_t)B * H * N * D >= ((int64_t)1 << 40)) return fail(COROPE_E_UNSUPPORTED, "rope_attn: tensor too large");
  // one workgroup per (batch, head, 64-row tile) on a single grid axis in the rotation pass, fewer in the other kernels
  if ((int64_t)B * H * ((N + 63) / 64) >= ((int64_t)1 << 31))
    return fail(COROPE_E_UNSUPPORTED, "rope_attn: B * H * ceil(N / 64) = %lld workgroups exceed the grid",
                (long long)B * H * ((N + 63) / 64));
  // staging loads address a (batch, head) slab and the tables with 32-bit byte offsets
  if ((int64_t)N * D * 2 >= ((int64_t)1 << 32) || (int64_t)N * freq_row_stride * 4 >= ((int64_t)1 << 32))
    return fail(COROPE_E_UNSUPPORTED, "rope_attn: one (batch, head) slab or a cos/sin table exceeds 4 GiB");
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
  // one workgroup per (batch, kv head, query row) on a single grid axis; slabs addressed with 32-bit byte offsets
  if ((int64_t)B * Hkv * N >= ((int64_t)1 << 31) || (int64_t)N * D * 2 >= ((int64_t)1 << 32))
    return fail(COROPE_E_UNSUPPORTED, "corope_gqa: B * Hkv * N = %lld rows exceed the grid, or one slab exceeds 4 GiB",
                (long long)B * Hkv * N);
  g_err[0] = 0;
  return COROPE_OK;
}

}  // extern "C" (reopened below)

namespace {

// Workspace of the two-launch forward: rotated K (bf16, same shape as k), then one float per 64-key tile.
int64_t fwd_ws_krot_bytes(int B, int H, int N, int D) { return (((int64_t)B * H * N * D * 2) + 255) / 256 * 256; }
int64_t fwd_ws_bytes(int B, int H, int N, int D) {
  return fwd_ws_krot_bytes(B, H, N, D) + (int64_t)B * H * ((N + 63) / 64) * 4;
}

// k_rot / tile_kmax null: single launch.  workspace non-null: rotate K into it first.
int rope_attn_fwd_impl(const char* what, const void* q, const void* k, const void* v, const float* freqs_cos,
                       const float* freqs_sin, int64_t freq_row_stride, void* o, float* lse, int B, int H, int N, int D,
                       float sm_scale, int causal, const void* k_rot, const float* tile_kmax, void* q_rot_out,
                       void* workspace, int64_t workspace_bytes, void* stream, int Hkv = 0) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 0);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, freqs_cos, freqs_sin, o, lse});
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
  p.H = H;
  p.Hkv = Hkv > 0 ? Hkv : H;
  p.contiguous(D);
  p.k_rot = static_cast<const uint16_t*>(k_rot);
  p.tile_kmax = tile_kmax;
  p.q_rot_out = static_cast<uint16_t*>(q_rot_out);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (workspace != nullptr) {
    rc = check_ptrs(what, {workspace});
    if (rc) return rc;
    if (workspace_bytes < fwd_ws_bytes(B, H, N, D))
      return fail(COROPE_E_BADARG, "%s: workspace of %lld bytes, %lld needed", what, (long long)workspace_bytes,
                  (long long)fwd_ws_bytes(B, H, N, D));
    uint16_t* ws_k = static_cast<uint16_t*>(workspace);
    float* ws_max = reinterpret_cast<float*>(static_cast<char*>(workspace) + fwd_ws_krot_bytes(B, H, N, D));
    rc = launch_status(what, corope::launch_rope_rotate(p.k, p.cos, p.sin, p.fstride, ws_k, ws_max, p.BH, N, D, st));
    if (rc) return rc;
    p.k_rot = ws_k;
    p.tile_kmax = ws_max;
  }
  if (p.k_rot != nullptr) return launch_status(what, corope::launch_rope_attn_fwd_prerotated(p, D, causal != 0, st));
  return launch_status(what, corope::launch_rope_attn_fwd(p, D, causal != 0, st));
}

}  // namespace

extern "C" {

int corope_rope_attn_fwd(const void* q, const void* k, const void* v, const float* freqs_cos, const float* freqs_sin,
                         int64_t freq_row_stride, void* o, float* lse, int B, int H, int N, int D, float sm_scale,
                         int causal, void* stream) {
  return rope_attn_fwd_impl("rope_attn_fwd", q, k, v, freqs_cos, freqs_sin, freq_row_stride, o, lse, B, H, N, D, sm_scale,
                            causal, nullptr, nullptr, nullptr, nullptr, 0, stream);
}

// ---- the forward for callers that cannot allocate -------------------------------------------------------------------
// Scratch of corope_rope_attn_fwd_noalloc: the rotated K and the per-tile key norms that corope_rope_attn_fwd_ws keeps in
// a caller-supplied workspace.  One copy per GPU the library is loaded on, held until the process ends.  In host code the
// array's name only stands for the symbol: the device address comes from hipGetSymbolAddress, once per device.
}  // extern "C" (reopened below)

#define COROPE_NOALLOC_MAX_BYTES (65ll << 20)
static __device__ __align__(256) unsigned char scratch[COROPE_NOALLOC_MAX_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];   // per device: address of that device's copy of `scratch`

// Device address of the current device's scratch array (null + error text on failure).
void* scratch_address(const char* what) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) {
    launch_status(what, e);
    return nullptr;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    fail(COROPE_E_UNSUPPORTED, "%s: device ordinal %d outside [0, %d)", what, dev, kMaxDevices);
    return nullptr;
  }
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr != nullptr) return ptr;
  if (hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)); e != hipSuccess || ptr == nullptr) {
    launch_status(what, e != hipSuccess ? e : hipErrorInvalidSymbol);
    return nullptr;
  }
  g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // two threads racing here store the same address
  return ptr;
}

}  // namespace

extern "C" {

int64_t corope_rope_attn_fwd_noalloc_max_bytes(void) { return COROPE_NOALLOC_MAX_BYTES; }

int corope_rope_attn_fwd_noalloc(const void* q, const void* k, const void* v, const float* freqs_cos, const float* freqs_sin,
                                 int64_t freq_row_stride, void* o, float* lse, int B, int H, int N, int D, float sm_scale,
                                 int causal, void* stream) {
  const char* what = "rope_attn_fwd_noalloc";
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 0);
  if (rc) return rc;
  const int64_t need = fwd_ws_bytes(B, H, N, D);
  if (need > COROPE_NOALLOC_MAX_BYTES)
    return fail(COROPE_E_UNSUPPORTED,
                "%s: B*H*N*D = %lld needs %lld bytes of scratch, the built-in buffer holds %lld; use corope_rope_attn_fwd_ws "
                "with a workspace of your own",
                what, (long long)B * H * N * D, (long long)need, (long long)COROPE_NOALLOC_MAX_BYTES);
  rc = check_ptrs(what, {q, k, v, freqs_cos, freqs_sin, o, lse});
  if (rc) return rc;
  void* ptr = scratch_address(what);
  if (ptr == nullptr) return COROPE_E_LAUNCH;
  return rope_attn_fwd_impl(what, q, k, v, freqs_cos, freqs_sin, freq_row_stride, o, lse, B, H, N, D, sm_scale, causal,
                            nullptr, nullptr, nullptr, ptr, COROPE_NOALLOC_MAX_BYTES, stream);
}

int64_t corope_rope_attn_fwd_workspace_bytes(int B, int H, int N, int D) {
  if (corope_rope_attn_check(B, H, N, D, D, 1.f, 0)) return -1;
  return fwd_ws_bytes(B, H, N, D);
}

int corope_rope_attn_fwd_ws(const void* q, const void* k, const void* v, const float* freqs_cos, const float* freqs_sin,
                            int64_t freq_row_stride, void* o, float* lse, int B, int H, int N, int D, float sm_scale,
                            int causal, void* workspace, int64_t workspace_bytes, void* stream) {
  if (workspace == nullptr) return fail(COROPE_E_BADARG, "rope_attn_fwd_ws: null workspace");
  return rope_attn_fwd_impl("rope_attn_fwd_ws", q, k, v, freqs_cos, freqs_sin, freq_row_stride, o, lse, B, H, N, D,
                            sm_scale, causal, nullptr, nullptr, nullptr, workspace, workspace_bytes, stream);
}

int corope_rope_attn_fwd_prerotated(const void* q, const void* k_rot, const float* tile_kmax, const void* v,
                                    const float* freqs_cos, const float* freqs_sin, int64_t freq_row_stride, void* o,
                                    float* lse, void* q_rot_out, int B, int H, int N, int D, float sm_scale, int causal,
                                    void* stream) {
  int rc = check_ptrs("rope_attn_fwd_prerotated", {k_rot});
  if (rc) return rc;
  if (q_rot_out != nullptr && !aligned16(q_rot_out))
    return fail(COROPE_E_ALIGN, "rope_attn_fwd_prerotated: q_rot_out %p is not 16-byte aligned", q_rot_out);
  if (tile_kmax == nullptr || (reinterpret_cast<uintptr_t>(tile_kmax) & 3u))
    return fail(tile_kmax ? COROPE_E_ALIGN : COROPE_E_BADARG, "rope_attn_fwd_prerotated: tile_kmax %p is null or misaligned",
                (const void*)tile_kmax);
  return rope_attn_fwd_impl("rope_attn_fwd_prerotated", q, k_rot, v, freqs_cos, freqs_sin, freq_row_stride, o, lse, B, H,
                            N, D, sm_scale, causal, k_rot, tile_kmax, q_rot_out, nullptr, 0, stream);
}

int corope_rope_attn_fwd_train(const void* q, const void* k, const void* v, const float* freqs_cos, const float* freqs_sin,
                               int64_t freq_row_stride, void* o, float* lse, void* q_rot, void* k_rot, float* tile_kmax,
                               int B, int H, int N, int D, float sm_scale, int causal, void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 0);
  if (rc) return rc;
  rc = check_ptrs("rope_attn_fwd_train", {q, k, v, freqs_cos, freqs_sin, o, lse, q_rot, k_rot});
  if (rc) return rc;
  if (tile_kmax == nullptr || (reinterpret_cast<uintptr_t>(tile_kmax) & 3u))
    return fail(tile_kmax ? COROPE_E_ALIGN : COROPE_E_BADARG, "rope_attn_fwd_train: tile_kmax %p is null or misaligned",
                (const void*)tile_kmax);
  rc = corope_rope_rotate(k, freqs_cos, freqs_sin, freq_row_stride, k_rot, tile_kmax, B, H, N, D, 1.f, stream);
  if (rc) return rc;
  return corope_rope_attn_fwd_prerotated(q, k_rot, tile_kmax, v, freqs_cos, freqs_sin, freq_row_stride, o, lse, q_rot, B, H,
                                         N, D, sm_scale, causal, stream);
}

int corope_rope_rotate(const void* x, const float* freqs_cos, const float* freqs_sin, int64_t freq_row_stride, void* y,
                       float* tile_max, int B, int H, int N, int D, float scale, void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, 1.f, 0);
  if (rc) return rc;
  rc = check_ptrs("rope_rotate", {x, freqs_cos, freqs_sin, y});
  if (rc) return rc;
  if (!(scale > 0.f) || !std::isfinite(scale)) return fail(COROPE_E_BADARG, "rope_rotate: scale %g must be positive and finite", (double)scale);
  if (tile_max != nullptr && (reinterpret_cast<uintptr_t>(tile_max) & 3u))
    return fail(COROPE_E_ALIGN, "rope_rotate: tile_max %p is not 4-byte aligned", (void*)tile_max);
  return launch_status("rope_rotate",
                       corope::launch_rope_rotate(static_cast<const uint16_t*>(x), freqs_cos, freqs_sin, freq_row_stride,
                                                  static_cast<uint16_t*>(y), tile_max, B * H, N, D,
                                                  static_cast<hipStream_t>(stream), scale));
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

}  // extern "C" (reopened below)

namespace {

int64_t bwd_ws_tensor_bytes(int B, int H, int N, int D) { return (((int64_t)B * H * N * D * 2) + 255) / 256 * 256; }

// prerot: q and k are copies that corope_rope_rotate rotated.
void mark_prerotated(corope::BwdParams& p, bool prerot) {
  if (prerot) {
    p.q_rot = p.q;
    p.k_rot = p.k;
  }
}

// Everything a whole backward takes, checked before the first launch of a composite entry point: sizes, then every
// pointer (null and alignment).  `o` may be null only where the caller says so.
int validate_bwd(const char* what, int B, int H, int N, int D, int64_t freq_row_stride, float sm_scale,
                 std::initializer_list<const void*> ptrs) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  return check_ptrs(what, ptrs);
}

int bwd_dv_impl(const char* what, bool prerot, const void* q, const void* k, const void* d_o, const float* lse,
                const float* freqs_cos, const float* freqs_sin, int64_t freq_row_stride, void* dv, int B, int H, int N,
                int D, float sm_scale, int causal, void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, d_o, lse, freqs_cos, freqs_sin, dv});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q, k, nullptr, nullptr, d_o, lse, nullptr, freqs_cos, freqs_sin, freq_row_stride,
                                 nullptr, nullptr, dv, B, H, N, sm_scale);
  mark_prerotated(p, prerot);
  return launch_status(what, corope::launch_bwd_dv(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

int bwd_dk_impl(const char* what, bool prerot, const void* q, const void* k, const void* v, const void* d_o,
                const float* lse, const float* delta, const float* freqs_cos, const float* freqs_sin,
                int64_t freq_row_stride, void* dk, int B, int H, int N, int D, float sm_scale, int causal, void* stream) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, dk});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q, k, v, nullptr, d_o, lse, const_cast<float*>(delta), freqs_cos, freqs_sin,
                                 freq_row_stride, nullptr, dk, nullptr, B, H, N, sm_scale);
  mark_prerotated(p, prerot);
  return launch_status(what, corope::launch_bwd_dk(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

// o non-null: the kernel computes delta from o and d_o for its rows and WRITES it to `delta`.
int bwd_dq_impl(const char* what, bool prerot, const void* q, const void* k, const void* v, const void* d_o,
                const float* lse, const float* delta, const float* freqs_cos, const float* freqs_sin,
                int64_t freq_row_stride, void* dq, int B, int H, int N, int D, float sm_scale, int causal, void* stream,
                const void* o = nullptr) {
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, dq});
  if (rc) return rc;
  if (o != nullptr && !aligned16(o)) return fail(COROPE_E_ALIGN, "%s: pointer %p is not 16-byte aligned", what, o);
  corope::BwdParams p = make_bwd(q, k, v, o, d_o, lse, const_cast<float*>(delta), freqs_cos, freqs_sin,
                                 freq_row_stride, dq, nullptr, nullptr, B, H, N, sm_scale);
  mark_prerotated(p, prerot);
  return launch_status(what, corope::launch_bwd_dq(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

}  // namespace

extern "C" {

int corope_rope_attn_bwd_dv(const void* q, const void* k, const void* d_o, const float* lse, const float* freqs_cos,
                            const float* freqs_sin, int64_t freq_row_stride, void* dv, int B, int H, int N, int D,
                            float sm_scale, int causal, void* stream) {
  return bwd_dv_impl("rope_attn_bwd_dv", false, q, k, d_o, lse, freqs_cos, freqs_sin, freq_row_stride, dv, B, H, N, D,
                     sm_scale, causal, stream);
}

int corope_rope_attn_bwd_dk(const void* q, const void* k, const void* v, const void* d_o, const float* lse,
                            const float* delta, const float* freqs_cos, const float* freqs_sin,
                            int64_t freq_row_stride, void* dk, int B, int H, int N, int D, float sm_scale, int causal,
                            void* stream) {
  return bwd_dk_impl("rope_attn_bwd_dk", false, q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dk, B,
                     H, N, D, sm_scale, causal, stream);
}

int corope_rope_attn_bwd_dkdv(const void* q, const void* k, const void* v, const void* d_o, const float* lse,
                              const float* delta, const float* freqs_cos, const float* freqs_sin,
                              int64_t freq_row_stride, void* dk, void* dv, int B, int H, int N, int D, float sm_scale,
                              int causal, void* stream) {
  int rc = validate_bwd("rope_attn_bwd_dkdv", B, H, N, D, freq_row_stride, sm_scale,
                        {q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, dk, dv});
  if (rc) return rc;
  if (D == 64) {   // both sets of accumulators and the rotation's table values fit a wave's registers: one launch
    corope::BwdParams p = make_bwd(q, k, v, nullptr, d_o, lse, const_cast<float*>(delta), freqs_cos, freqs_sin,
                                   freq_row_stride, nullptr, dk, dv, B, H, N, sm_scale);
    return launch_status("rope_attn_bwd_dkdv", corope::launch_bwd_dkdv_fused(p, D, causal != 0, static_cast<hipStream_t>(stream)));
  }
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
  return bwd_dq_impl("rope_attn_bwd_dq", false, q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dq, B,
                     H, N, D, sm_scale, causal, stream);
}

int corope_rope_attn_bwd_dv_prerotated(const void* q_rot, const void* k_rot, const void* d_o, const float* lse,
                                       const float* freqs_cos, const float* freqs_sin, int64_t freq_row_stride, void* dv,
                                       int B, int H, int N, int D, float sm_scale, int causal, void* stream) {
  return bwd_dv_impl("rope_attn_bwd_dv_prerotated", true, q_rot, k_rot, d_o, lse, freqs_cos, freqs_sin, freq_row_stride,
                     dv, B, H, N, D, sm_scale, causal, stream);
}

int corope_rope_attn_bwd_dk_prerotated(const void* q_rot, const void* k_rot, const void* v, const void* d_o,
                                       const float* lse, const float* delta, const float* freqs_cos,
                                       const float* freqs_sin, int64_t freq_row_stride, void* dk, int B, int H, int N,
                                       int D, float sm_scale, int causal, void* stream) {
  return bwd_dk_impl("rope_attn_bwd_dk_prerotated", true, q_rot, k_rot, v, d_o, lse, delta, freqs_cos, freqs_sin,
                     freq_row_stride, dk, B, H, N, D, sm_scale, causal, stream);
}

int corope_rope_attn_bwd_dkdv_prerotated(const void* q_rot, const void* k_rot, const void* v, const void* d_o,
                                         const float* lse, const float* delta, const float* freqs_cos,
                                         const float* freqs_sin, int64_t freq_row_stride, void* dk, void* dv, int B, int H,
                                         int N, int D, float sm_scale, int causal, void* stream) {
  const char* what = "rope_attn_bwd_dkdv_prerotated";
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs(what, {q_rot, k_rot, v, d_o, lse, delta, freqs_cos, freqs_sin, dk, dv});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q_rot, k_rot, v, nullptr, d_o, lse, const_cast<float*>(delta), freqs_cos, freqs_sin,
                                 freq_row_stride, nullptr, dk, dv, B, H, N, sm_scale);
  mark_prerotated(p, true);
  return launch_status(what, corope::launch_bwd_dkdv_fused(p, D, causal != 0, static_cast<hipStream_t>(stream)));
}

int corope_rope_attn_bwd_dq_prerotated(const void* q_rot, const void* k_rot, const void* v, const void* o, const void* d_o,
                                       const float* lse, float* delta, const float* freqs_cos, const float* freqs_sin,
                                       int64_t freq_row_stride, void* dq, int B, int H, int N, int D, float sm_scale,
                                       int causal, void* stream) {
  return bwd_dq_impl("rope_attn_bwd_dq_prerotated", true, q_rot, k_rot, v, d_o, lse, delta, freqs_cos, freqs_sin,
                     freq_row_stride, dq, B, H, N, D, sm_scale, causal, stream, o);
}

int corope_rope_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                         float* delta, const float* freqs_cos, const float* freqs_sin, int64_t freq_row_stride,
                         void* dq, void* dk, void* dv, int B, int H, int N, int D, float sm_scale, int causal,
                         void* stream) {
  int rc = validate_bwd("rope_attn_bwd", B, H, N, D, freq_row_stride, sm_scale,
                        {q, k, v, o, d_o, lse, delta, freqs_cos, freqs_sin, dq, dk, dv});
  if (rc) return rc;
  rc = corope_rope_attn_bwd_preprocess(o, d_o, delta, B, H, N, D, stream);
  if (rc) return rc;
  rc = corope_rope_attn_bwd_dkdv(q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dk, dv, B, H, N, D,
                                 sm_scale, causal, stream);
  if (rc) return rc;
  return corope_rope_attn_bwd_dq(q, k, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dq, B, H, N, D,
                                 sm_scale, causal, stream);
}

int corope_rope_attn_bwd_prerotated(const void* q_rot, const void* k_rot, const void* v, const void* o, const void* d_o,
                                    const float* lse, float* delta, const float* freqs_cos, const float* freqs_sin,
                                    int64_t freq_row_stride, void* dq, void* dk, void* dv, int B, int H, int N, int D,
                                    float sm_scale, int causal, void* stream) {
  // two launches: the dQ kernel computes delta for the rows it owns on its way (no separate pass over o and dO), the
  // fused dK+dV kernel reads it afterwards
  int rc = validate_bwd("rope_attn_bwd_prerotated", B, H, N, D, freq_row_stride, sm_scale,
                        {q_rot, k_rot, v, o, d_o, lse, delta, freqs_cos, freqs_sin, dq, dk, dv});
  if (rc) return rc;
  rc = corope_rope_attn_bwd_dq_prerotated(q_rot, k_rot, v, o, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dq, B,
                                          H, N, D, sm_scale, causal, stream);
  if (rc) return rc;
  return corope_rope_attn_bwd_dkdv_prerotated(q_rot, k_rot, v, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dk,
                                              dv, B, H, N, D, sm_scale, causal, stream);
}

int64_t corope_rope_attn_bwd_workspace_bytes(int B, int H, int N, int D) {
  if (corope_rope_attn_check(B, H, N, D, D, 1.f, 1)) return -1;
  return 2 * bwd_ws_tensor_bytes(B, H, N, D);
}

int corope_rope_attn_bwd_ws(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                            const float* lse, float* delta, const float* freqs_cos, const float* freqs_sin,
                            int64_t freq_row_stride, void* dq, void* dk, void* dv, int B, int H, int N, int D,
                            float sm_scale, int causal, void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = validate_bwd("rope_attn_bwd_ws", B, H, N, D, freq_row_stride, sm_scale,
                        {q, k, v, o, d_o, lse, delta, freqs_cos, freqs_sin, dq, dk, dv, workspace});
  if (rc) return rc;
  if (workspace_bytes < 2 * bwd_ws_tensor_bytes(B, H, N, D))
    return fail(COROPE_E_BADARG, "rope_attn_bwd_ws: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                (long long)(2 * bwd_ws_tensor_bytes(B, H, N, D)));
  void* q_rot = workspace;
  void* k_rot = static_cast<char*>(workspace) + bwd_ws_tensor_bytes(B, H, N, D);
  rc = corope_rope_rotate(q, freqs_cos, freqs_sin, freq_row_stride, q_rot, nullptr, B, H, N, D, sm_scale * kLog2e, stream);
  if (rc) return rc;
  rc = corope_rope_rotate(k, freqs_cos, freqs_sin, freq_row_stride, k_rot, nullptr, B, H, N, D, 1.f, stream);
  if (rc) return rc;
  return corope_rope_attn_bwd_prerotated(q_rot, k_rot, v, o, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dq, dk,
                                         dv, B, H, N, D, sm_scale, causal, stream);
}

int corope_rope_attn_fwd_gqa(const void* q, const void* k, const void* v, const float* freqs_cos, const float* freqs_sin,
                             int64_t freq_row_stride, void* o, float* lse, void* q_rot, void* k_rot, float* tile_kmax, int B,
                             int Hq, int Hkv, int N, int D, float sm_scale, int causal, void* stream) {
  const char* what = "rope_attn_fwd_gqa";
  if (Hkv <= 0 || Hq % Hkv != 0) return fail(COROPE_E_BADARG, "%s: Hq=%d is not a multiple of Hkv=%d", what, Hq, Hkv);
  if (k_rot == nullptr) {
    if (q_rot != nullptr) return fail(COROPE_E_BADARG, "%s: q_rot without k_rot", what);
    return rope_attn_fwd_impl(what, q, k, v, freqs_cos, freqs_sin, freq_row_stride, o, lse, B, Hq, N, D, sm_scale, causal,
                              nullptr, nullptr, nullptr, nullptr, 0, stream, Hkv);
  }
  int rc = corope_rope_attn_check(B, Hq, N, D, freq_row_stride, sm_scale, 0);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, freqs_cos, freqs_sin, o, lse, k_rot});
  if (rc) return rc;
  if (q_rot != nullptr && !aligned16(q_rot)) return fail(COROPE_E_ALIGN, "%s: q_rot %p is not 16-byte aligned", what, q_rot);
  if (tile_kmax == nullptr || (reinterpret_cast<uintptr_t>(tile_kmax) & 3u))
    return fail(tile_kmax ? COROPE_E_ALIGN : COROPE_E_BADARG, "%s: tile_kmax %p is null or misaligned", what,
                (const void*)tile_kmax);
  rc = corope_rope_rotate(k, freqs_cos, freqs_sin, freq_row_stride, k_rot, tile_kmax, B, Hkv, N, D, 1.f, stream);
  if (rc) return rc;
  return rope_attn_fwd_impl(what, q, k_rot, v, freqs_cos, freqs_sin, freq_row_stride, o, lse, B, Hq, N, D, sm_scale, causal,
                            k_rot, tile_kmax, q_rot, nullptr, 0, stream, Hkv);
}

int corope_rope_attn_bwd_gqa(const void* q, const void* k, int prerotated, const void* v, const void* o, const void* d_o,
                             const float* lse, float* delta, const float* freqs_cos, const float* freqs_sin,
                             int64_t freq_row_stride, void* dq, void* dk, void* dv, int B, int Hq, int Hkv, int N, int D,
                             float sm_scale, int causal, void* stream) {
  const char* what = "rope_attn_bwd_gqa";
  if (Hkv <= 0 || Hq % Hkv != 0) return fail(COROPE_E_BADARG, "%s: Hq=%d is not a multiple of Hkv=%d", what, Hq, Hkv);
  int rc = corope_rope_attn_check(B, Hq, N, D, freq_row_stride, sm_scale, 1);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, o, d_o, lse, delta, freqs_cos, freqs_sin, dq, dk, dv});
  if (rc) return rc;
  rc = corope_rope_attn_bwd_preprocess(o, d_o, delta, B, Hq, N, D, stream);
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q, k, v, nullptr, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dq, dk, dv, B, Hq,
                                 N, sm_scale);
  p.Hkv = Hkv;
  mark_prerotated(p, prerotated != 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (prerotated) {
    rc = launch_status(what, corope::launch_bwd_dkdv_fused(p, D, causal != 0, st));
  } else {
    rc = launch_status(what, corope::launch_bwd_dv(p, D, causal != 0, st));
    if (rc == 0) rc = launch_status(what, corope::launch_bwd_dk(p, D, causal != 0, st));
  }
  if (rc) return rc;
  return launch_status(what, corope::launch_bwd_dq(p, D, causal != 0, st));
}

// ---- fp16 tensors (the reference's dtype): the same kernels built for fp16 elements -------------------------------------
int corope_rope_attn_fwd_f16(const void* q, const void* k, const void* v, const float* freqs_cos, const float* freqs_sin,
                             int64_t freq_row_stride, void* o, float* lse, void* q_rot, void* k_rot, float* tile_kmax, int B,
                             int H, int Hkv, int N, int D, float sm_scale, int causal, void* stream) {
  const char* what = "rope_attn_fwd_f16";
  if (Hkv <= 0 || H % Hkv != 0) return fail(COROPE_E_BADARG, "%s: H=%d is not a multiple of Hkv=%d", what, H, Hkv);
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 0);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, freqs_cos, freqs_sin, o, lse});
  if (rc) return rc;
  if (k_rot == nullptr && q_rot != nullptr) return fail(COROPE_E_BADARG, "%s: q_rot without k_rot", what);
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
  p.H = H;
  p.Hkv = Hkv;
  p.contiguous(D);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (k_rot == nullptr) return launch_status(what, corope_f16::launch_rope_attn_fwd(p, D, causal != 0, st));
  // two launches: K rotated once into k_rot (with the largest key norm of every 64-key tile), then the attention kernel
  // on it, which leaves its rotated, scaled Q rows in q_rot if asked to (the operands of a backward on rotated copies)
  rc = check_ptrs(what, {k_rot});
  if (rc) return rc;
  if (q_rot != nullptr && !aligned16(q_rot)) return fail(COROPE_E_ALIGN, "%s: q_rot %p is not 16-byte aligned", what, q_rot);
  // tile_kmax null: the attention kernel is the single-launch one on the rotated copy (probabilities in fp16 against an fp16 V)
  if (reinterpret_cast<uintptr_t>(tile_kmax) & 3u) return fail(COROPE_E_ALIGN, "%s: tile_kmax %p is misaligned", what, (const void*)tile_kmax);
  rc = launch_status(what, corope_f16::launch_rope_rotate(p.k, p.cos, p.sin, p.fstride, static_cast<uint16_t*>(k_rot), tile_kmax,
                                                          B * Hkv, N, D, st, 1.f, 1, 0, 0, 0));
  if (rc) return rc;
  p.k_rot = static_cast<const uint16_t*>(k_rot);
  p.tile_kmax = tile_kmax;
  p.q_rot_out = static_cast<uint16_t*>(q_rot);
  return launch_status(what, corope_f16::launch_rope_attn_fwd_prerotated(p, D, causal != 0, st));
}

int corope_rope_attn_bwd_f16(const void* q, const void* k, int prerotated, const void* v, const void* o, const void* d_o,
                             const float* lse, float* delta, const float* freqs_cos, const float* freqs_sin,
                             int64_t freq_row_stride, void* dq, void* dk, void* dv, int B, int H, int Hkv, int N, int D,
                             float sm_scale, int causal, void* workspace, int64_t workspace_bytes, void* stream) {
  const char* what = "rope_attn_bwd_f16";
  if (Hkv <= 0 || H % Hkv != 0) return fail(COROPE_E_BADARG, "%s: H=%d is not a multiple of Hkv=%d", what, H, Hkv);
  int rc = validate_bwd(what, B, H, N, D, freq_row_stride, sm_scale,
                        {q, k, v, o, d_o, lse, delta, freqs_cos, freqs_sin, dq, dk, dv});
  if (rc) return rc;
  corope::BwdParams p = make_bwd(q, k, v, o, d_o, lse, delta, freqs_cos, freqs_sin, freq_row_stride, dq, dk, dv, B, H, N,
                                 sm_scale);
  p.Hkv = Hkv;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (prerotated) {
    // q, k are the rotated copies a two-launch forward kept: the dQ kernel computes delta on its way, dK and dV come
    // from one kernel
    mark_prerotated(p, true);
    rc = launch_status(what, corope_f16::launch_bwd_dq(p, D, causal != 0, st));
    if (rc) return rc;
    return launch_status(what, corope_f16::launch_bwd_dkdv_fused(p, D, causal != 0, st));
  }
  if (workspace != nullptr) {
    // as corope_rope_attn_bwd_ws: q (scaled) and k are rotated once, then as above
    if (!aligned16(workspace)) return fail(COROPE_E_ALIGN, "%s: pointer %p is not 16-byte aligned", what, workspace);
    const int64_t each = bwd_ws_tensor_bytes(B, H, N, D);
    if (workspace_bytes < 2 * each)
      return fail(COROPE_E_BADARG, "%s: workspace of %lld bytes, %lld needed", what, (long long)workspace_bytes,
                  (long long)(2 * each));
    uint16_t* q_rot = static_cast<uint16_t*>(workspace);
    uint16_t* k_rot = reinterpret_cast<uint16_t*>(static_cast<char*>(workspace) + each);
    rc = launch_status(what, corope_f16::launch_rope_rotate(p.q, p.cos, p.sin, p.fstride, q_rot, nullptr, p.BH, N, D, st,
                                                            p.qk_scale, 1, 0, 0, 0));
    if (rc) return rc;
    rc = launch_status(what, corope_f16::launch_rope_rotate(p.k, p.cos, p.sin, p.fstride, k_rot, nullptr, B * Hkv, N, D, st, 1.f, 1, 0, 0, 0));
    if (rc) return rc;
    p.q = p.q_rot = q_rot;
    p.k = p.k_rot = k_rot;
    rc = launch_status(what, corope_f16::launch_bwd_dq(p, D, causal != 0, st));
    if (rc) return rc;
    return launch_status(what, corope_f16::launch_bwd_dkdv_fused(p, D, causal != 0, st));
  }
  rc = launch_status(what, corope_f16::launch_bwd_preprocess(p, D, st));
  if (rc) return rc;
  p.o = nullptr;   // delta comes from the pass above, not from the dQ kernel
  rc = launch_status(what, corope_f16::launch_bwd_dv(p, D, causal != 0, st));
  if (rc) return rc;
  rc = launch_status(what, corope_f16::launch_bwd_dk(p, D, causal != 0, st));
  if (rc) return rc;
  return launch_status(what, corope_f16::launch_bwd_dq(p, D, causal != 0, st));
}

int corope_rope_attn_fwd_strided(const void* q, const int64_t* q_strides, const void* k, const int64_t* k_strides, const void* v,
                                 const int64_t* v_strides, const float* freqs_cos, const float* freqs_sin,
                                 int64_t freq_row_stride, void* o, float* lse, void* q_rot, void* k_rot, float* tile_kmax, int B,
                                 int H, int Hkv, int N, int D, float sm_scale, int causal, int fp16, void* stream) {
  const char* what = "rope_attn_fwd_strided";
  if (Hkv <= 0 || H % Hkv != 0) return fail(COROPE_E_BADARG, "%s: H=%d is not a multiple of Hkv=%d", what, H, Hkv);
  int rc = corope_rope_attn_check(B, H, N, D, freq_row_stride, sm_scale, 0);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, freqs_cos, freqs_sin, o, lse});
  if (rc) return rc;
  if (q_strides == nullptr || k_strides == nullptr || v_strides == nullptr) return fail(COROPE_E_BADARG, "%s: null strides", what);
  for (const int64_t* st : {q_strides, k_strides, v_strides}) {
    // rows start on 16-byte boundaries and one (batch, head) slice stays below 4 GiB (32-bit offsets inside it)
    if (st[2] < D || st[0] < 0 || st[1] < 0 || st[0] % 8 != 0 || st[1] % 8 != 0 || st[2] % 8 != 0)
      return fail(COROPE_E_BADARG, "%s: strides (%lld, %lld, %lld) must be non-negative multiples of 8 elements, rows at least D apart",
                  what, (long long)st[0], (long long)st[1], (long long)st[2]);
    if ((int64_t)N * st[2] * 2 >= ((int64_t)1 << 32) || st[2] >= ((int64_t)1 << 30))
      return fail(COROPE_E_UNSUPPORTED, "%s: one (batch, head) slice spans 4 GiB or more at row stride %lld", what, (long long)st[2]);
  }
  if (k_rot == nullptr && q_rot != nullptr) return fail(COROPE_E_BADARG, "%s: q_rot without k_rot", what);
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
  p.H = H;
  p.Hkv = Hkv;
  p.q_sb = q_strides[0], p.q_sh = q_strides[1], p.q_sn = (int)q_strides[2];
  p.k_sb = k_strides[0], p.k_sh = k_strides[1], p.k_sn = (int)k_strides[2];
  p.v_sb = v_strides[0], p.v_sh = v_strides[1], p.v_sn = (int)v_strides[2];
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (k_rot == nullptr)
    return launch_status(what, fp16 ? corope_f16::launch_rope_attn_fwd(p, D, causal != 0, st)
                                    : corope::launch_rope_attn_fwd(p, D, causal != 0, st));
  rc = check_ptrs(what, {k_rot});
  if (rc) return rc;
  if (q_rot != nullptr && !aligned16(q_rot)) return fail(COROPE_E_ALIGN, "%s: q_rot %p is not 16-byte aligned", what, q_rot);
  // tile_kmax null: the attention kernel is the single-launch one on the rotated copy (no lazy reference value; for fp16
  // tensors: probabilities in fp16 against an fp16 V)
  if (reinterpret_cast<uintptr_t>(tile_kmax) & 3u) return fail(COROPE_E_ALIGN, "%s: tile_kmax %p is misaligned", what, (const void*)tile_kmax);
  uint16_t* kr = static_cast<uint16_t*>(k_rot);
  rc = launch_status(what, fp16 ? corope_f16::launch_rope_rotate(p.k, p.cos, p.sin, p.fstride, kr, tile_kmax, B * Hkv, N, D, st, 1.f,
                                                                 Hkv, p.k_sb, p.k_sh, p.k_sn)
                                : corope::launch_rope_rotate(p.k, p.cos, p.sin, p.fstride, kr, tile_kmax, B * Hkv, N, D, st, 1.f, Hkv,
                                                             p.k_sb, p.k_sh, p.k_sn));
  if (rc) return rc;
  p.k_rot = kr;
  p.tile_kmax = tile_kmax;
  p.q_rot_out = static_cast<uint16_t*>(q_rot);
  return launch_status(what, fp16 ? corope_f16::launch_rope_attn_fwd_prerotated(p, D, causal != 0, st)
                                  : corope::launch_rope_attn_fwd_prerotated(p, D, causal != 0, st));
}

int corope_rope_freqs(float* freqs_cos, float* freqs_sin, int n_pos, int D, int width, int64_t freq_row_stride, int pos0,
                      float theta, void* stream) {
  if (n_pos <= 0 || D <= 0 || D % 2 != 0) return fail(COROPE_E_BADARG, "rope_freqs: n_pos must be positive and D even");
  if (D > 256) return fail(COROPE_E_UNSUPPORTED, "rope_freqs: head dim %d exceeds 256", D);
  if (width != D && width != D / 2) return fail(COROPE_E_BADARG, "rope_freqs: width must be D or D/2 (got %d)", width);
  if (freq_row_stride < width) return fail(COROPE_E_BADARG, "rope_freqs: row stride smaller than the row");
  if (pos0 < 0 || !(theta > 0.f) || !std::isfinite(theta)) return fail(COROPE_E_BADARG, "rope_freqs: bad pos0 or theta");
  if ((int64_t)n_pos * (D / 2) >= ((int64_t)1 << 31)) return fail(COROPE_E_UNSUPPORTED, "rope_freqs: table too large");
  if (freqs_cos == nullptr || freqs_sin == nullptr) return fail(COROPE_E_BADARG, "rope_freqs: null pointer argument");
  g_err[0] = 0;
  return launch_status("rope_freqs", corope::launch_rope_freqs(freqs_cos, freqs_sin, n_pos, D, width, freq_row_stride,
                                                               pos0, theta, static_cast<hipStream_t>(stream)));
}

}  // extern "C" (reopened below)

namespace {

int corope_gqa_fwd_impl(const char* what, bool f16, const void* q, const void* k, const void* v, void* o, int B, int Hq, int Hkv,
                        int N, int D, float sm_scale, float theta, void* stream) {
  int rc = corope_gqa_check(B, Hq, Hkv, N, D, sm_scale, theta);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, o});
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
  hipStream_t st = static_cast<hipStream_t>(stream);
  return launch_status(what, f16 ? corope_f16::launch_corope_gqa_fwd(p, D, st) : corope::launch_corope_gqa_fwd(p, D, st));
}

}  // namespace

extern "C" {

int corope_gqa_fwd(const void* q, const void* k, const void* v, void* o, int B, int Hq, int Hkv, int N, int D,
                   float sm_scale, float theta, void* stream) {
  return corope_gqa_fwd_impl("corope_gqa_fwd", false, q, k, v, o, B, Hq, Hkv, N, D, sm_scale, theta, stream);
}

int corope_gqa_fwd_f16(const void* q, const void* k, const void* v, void* o, int B, int Hq, int Hkv, int N, int D,
                       float sm_scale, float theta, void* stream) {
  return corope_gqa_fwd_impl("corope_gqa_fwd_f16", true, q, k, v, o, B, Hq, Hkv, N, D, sm_scale, theta, stream);
}

int64_t corope_gqa_bwd_workspace_bytes(int B, int Hq, int Hkv, int N, int D) {
  if (corope_gqa_check(B, Hq, Hkv, N, D, 1.f, 2.f)) return -1;
  return 4 * corope::corope_gqa_bwd_workspace_floats(B, Hq, Hkv, N, D);
}

int64_t corope_gqa_bwd_min_workspace_bytes(int B, int Hq, int Hkv, int N, int D) {
  if (corope_gqa_check(B, Hq, Hkv, N, D, 1.f, 2.f)) return -1;
  return 4 * corope::corope_gqa_bwd_workspace_floats(1, Hq / Hkv, 1, N, D);
}

}  // extern "C" (reopened below)

namespace {

int corope_gqa_bwd_impl(const char* what, bool f16, const void* q, const void* k, const void* v, const void* o, const void* d_o,
                        void* dq, void* dk, void* dv, int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta,
                        void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = corope_gqa_check(B, Hq, Hkv, N, D, sm_scale, theta);
  if (rc) return rc;
  rc = check_ptrs(what, {q, k, v, d_o, dq, dk, dv, workspace});
  if (rc) return rc;
  if (o != nullptr && !aligned16(o)) return fail(COROPE_E_ALIGN, "%s: pointer %p is not 16-byte aligned", what, o);
  const int64_t need = 4 * corope::corope_gqa_bwd_workspace_floats(1, Hq / Hkv, 1, N, D);
  if (workspace_bytes < need)
    return fail(COROPE_E_BADARG, "%s: workspace of %lld bytes, at least %lld needed (one group's matrices)", what,
                (long long)workspace_bytes, (long long)need);
  corope::CoropeBwdParams p{};
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<const uint16_t*>(o);
  p.d_o = static_cast<const uint16_t*>(d_o);
  p.dq = static_cast<uint16_t*>(dq);
  p.dk = static_cast<uint16_t*>(dk);
  p.dv = static_cast<uint16_t*>(dv);
  p.sm_scale = sm_scale;
  p.theta = theta;
  p.B = B;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.N = N;
  float* ws = static_cast<float*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  return launch_status(what, f16 ? corope_f16::launch_corope_gqa_bwd(p, D, ws, workspace_bytes / 4, st)
                                 : corope::launch_corope_gqa_bwd(p, D, ws, workspace_bytes / 4, st));
}

}  // namespace

extern "C" {

int corope_gqa_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, void* dq, void* dk, void* dv,
                   int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta, void* workspace,
                   int64_t workspace_bytes, void* stream) {
  return corope_gqa_bwd_impl("corope_gqa_bwd", false, q, k, v, o, d_o, dq, dk, dv, B, Hq, Hkv, N, D, sm_scale, theta, workspace,
                             workspace_bytes, stream);
}

int corope_gqa_bwd_f16(const void* q, const void* k, const void* v, const void* o, const void* d_o, void* dq, void* dk,
                       void* dv, int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta, void* workspace,
                       int64_t workspace_bytes, void* stream) {
  return corope_gqa_bwd_impl("corope_gqa_bwd_f16", true, q, k, v, o, d_o, dq, dk, dv, B, Hq, Hkv, N, D, sm_scale, theta,
                             workspace, workspace_bytes, stream);
}


}  // extern "C"
