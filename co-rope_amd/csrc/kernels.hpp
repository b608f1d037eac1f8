// Parameter blocks and host-side launchers of the gfx950 kernels (internal to the library).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace corope {

// Raises a kernel's dynamic-LDS limit once per (kernel, device): `done` is a per-kernel word, bit d set = device d has it.
// Safe to call from several host threads (at worst the attribute is set twice to the same value).
inline hipError_t allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}


#ifdef COROPE_TRACE
// Experiment builds only: per-workgroup time stamps (100 MHz counter) for splitting a launch into its phases.
extern uint64_t* g_trace_buf;
#define COROPE_TRACE_FIELD uint64_t* trace;
#define COROPE_STAMP(slot, tid)                                                                              \
  do {                                                                                                       \
    if (p.trace != nullptr && threadIdx.x == (tid)) p.trace[(int64_t)blockIdx.x * 16 + (slot)] = __builtin_amdgcn_s_memrealtime(); \
  } while (0)
#define COROPE_STAMP_ID(tid, extra)                                                                          \
  do {                                                                                                       \
    if (p.trace != nullptr && threadIdx.x == (tid)) {                                                        \
      p.trace[(int64_t)blockIdx.x * 16 + 14] = (uint64_t)__builtin_amdgcn_s_getreg(63492) | ((uint64_t)__builtin_amdgcn_s_getreg(63508) << 32); \
      p.trace[(int64_t)blockIdx.x * 16 + 15] = (uint64_t)(extra);                                              \
    }                                                                                                        \
  } while (0)
// the same for persistent kernels: stamps are filed under the item (variables `item` and `TT` of the kernel)
#define COROPE_ISTAMP(slot)                                                                                   \
  do {                                                                                                        \
    if (p.trace != nullptr && threadIdx.x == TT) p.trace[(int64_t)item * 16 + (slot)] = __builtin_amdgcn_s_memrealtime(); \
  } while (0)
#define COROPE_ISTAMP_ID(extra)                                                                               \
  do {                                                                                                        \
    if (p.trace != nullptr && threadIdx.x == TT) {                                                            \
      p.trace[(int64_t)item * 16 + 14] = (uint64_t)__builtin_amdgcn_s_getreg(63492) | ((uint64_t)__builtin_amdgcn_s_getreg(63508) << 32); \
      p.trace[(int64_t)item * 16 + 15] = (uint64_t)(extra);                                                    \
    }                                                                                                         \
  } while (0)
#else
#define COROPE_TRACE_FIELD
#define COROPE_STAMP(slot, tid) do {} while (0)
#define COROPE_STAMP_ID(tid, extra) do {} while (0)
#define COROPE_ISTAMP(slot) do {} while (0)
#define COROPE_ISTAMP_ID(extra) do {} while (0)
#endif

// Compute units of the current device (cached per device; 256 on an MI355X): the size of a persistent launch, one
// workgroup per compute unit.
inline int device_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  int n = cached[dev & 63].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  cached[dev & 63].store(n, std::memory_order_relaxed);
  return n;
}

// Rows per workgroup of the attention kernels: 256 (8 waves) or 128 (4 waves).  By shape: a launch whose 256-row items
// number fewer than the compute units takes the 128-row form, which doubles the items and halves the time the heaviest
// of them runs; `g_tile_rows` (0 = by shape, 128, 256; set from the environment when the library is loaded) overrides the rule.
extern std::atomic<int> g_tile_rows;
// Query rows per wave of the two-launch forward at D = 128 with 256-row items: 32 (8 waves, two per SIMD) or 64 (4 waves,
// one per SIMD, every LDS fragment feeding two MFMAs); 0 = the default.
extern std::atomic<int> g_fwd_wave_rows;
// Whether two 4-wave workgroups of lds_bytes each fit a compute unit (the attention kernels are compiled for two waves
// per SIMD).
constexpr bool fits_twice(int lds_bytes) { return 2 * lds_bytes <= 160 * 1024; }
// small_lds_bytes: LDS of the kernel's 4-wave form.  Where two of those fit a compute unit, 128-row items pay as long as
// the 256-row items make fewer than two rounds (measured at D = 64: +15 % with one item per compute unit, +4 % with one
// and a half, -3 % with two); where only one fits, as long as they make less than one.
inline bool use_small_tiles(int n_rows, int slabs, int small_lds_bytes = 160 * 1024) {
  const int forced = g_tile_rows.load(std::memory_order_relaxed);
  if (forced == 128) return true;
  if (forced == 256) return false;
  return (int64_t)((n_rows + 255) / 256) * slabs < (int64_t)device_cu_count() * (fits_twice(small_lds_bytes) ? 2 : 1);
}

// Workgroups of a persistent launch: one per compute unit -- two where two fit (4-wave workgroups whose LDS leaves room
// for a second one) -- or one per item if those are fewer.  (Letting the two workgroups of a compute unit take its rounds in
// turn, so that every compute unit gets the same total, was measured and not kept: what counts is that both stay busy at the
// same time -- at one and a half rounds it cost 15 %, at exactly one it gained 3 %.)
inline unsigned persistent_grid(int64_t n_items, int waves, int lds_bytes) {
  const int per_cu = (waves <= 4 && fits_twice(lds_bytes)) ? 2 : 1;
  const int64_t slots = (int64_t)device_cu_count() * per_cu;
  return (unsigned)(n_items < slots ? n_items : slots);
}

struct FwdParams {
  COROPE_TRACE_FIELD
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* k_rot;   // K already rotated (same layout as k), or null: rotate K tiles inside the kernel
  const float* tile_kmax;  // with k_rot: largest rotated-key norm of every 64-key tile, [BH][ceil(N / 64)]
  uint16_t* q_rot_out;     // with k_rot, optional: receives the rotated Q times qk_scale (same layout as q), for a backward on rotated operands
  const float* cos;
  const float* sin;
  uint16_t* o;
  float* lse;
  int64_t fstride;   // elements between rows of the cos/sin tables
  float qk_scale;    // sm_scale * log2(e)
  int N;
  int BH;            // batch * query heads
  int H, Hkv;        // query heads and key/value heads per batch (grouped-query attention when Hkv < H; k, v, k_rot and
                     // tile_kmax then have B * Hkv slabs and query head h reads key/value head h / (H / Hkv))
  int num_m_blocks;  // filled in by the launcher
  // Layout of q, k, v (the forward only; o, lse, k_rot, q_rot_out are contiguous): elements between batches, heads and
  // rows; the last dimension is contiguous.  contiguous(D) fills in (B, H, N, D) row-major.
  int64_t q_sb, q_sh, k_sb, k_sh, v_sb, v_sh;
  int q_sn, k_sn, v_sn;
  void contiguous(int D) {
    q_sn = k_sn = v_sn = D;
    q_sh = k_sh = v_sh = (int64_t)N * D;
    q_sb = (int64_t)H * N * D;
    k_sb = v_sb = (int64_t)Hkv * N * D;
  }
#if defined(__HIPCC__)
  __device__ __forceinline__ const uint16_t* q_slab(int bh) const { return q + (bh / H) * q_sb + (bh % H) * q_sh; }
  __device__ __forceinline__ const uint16_t* k_slab(int kvs) const { return k + (kvs / Hkv) * k_sb + (kvs % Hkv) * k_sh; }
  __device__ __forceinline__ const uint16_t* v_slab(int kvs) const { return v + (kvs / Hkv) * v_sb + (kvs % Hkv) * v_sh; }
#endif
};

struct BwdParams {
  COROPE_TRACE_FIELD
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* o;
  const uint16_t* d_o;
  const uint16_t* q_rot;  // Q and K already rotated (same layout as q, k), or both null: rotate tiles inside the kernels;
  const uint16_t* k_rot;  // q_rot carries the factor qk_scale (rotated, scaled, rounded once), k_rot none
  const float* cos;
  const float* sin;
  const float* lse;
  float* delta;
  uint16_t* dq;
  uint16_t* dk;
  uint16_t* dv;
  int64_t fstride;
  float sm_scale;
  float qk_scale;  // sm_scale * log2(e)
  int N;
  int BH;          // batch * query heads
  int H, Hkv;      // as in FwdParams; dk, dv have B * Hkv slabs and sum over the query heads of their group
  int num_blocks;  // filled in by the launcher
};

struct CoropeParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* o;
  float sm_scale;
  float theta;  // RoPE base; inverse frequencies are theta^(-2d/D)
  int B, Hq, Hkv, N;
  int num_m_blocks;
};

struct CoropeBwdParams {
  const uint16_t* q;    // (B, Hq, N, D)
  const uint16_t* k;    // (B, Hkv, N, D)
  const uint16_t* v;
  const uint16_t* o;    // (B, Hq, N, D) forward output, or null: only a reference value for rowsum(P o dP) is taken from it
  const uint16_t* d_o;  // (B, Hq, N, D)
  uint16_t* dq;
  uint16_t* dk;
  uint16_t* dv;
  float sm_scale;
  float theta;
  int B, Hq, Hkv, N;
};

}  // namespace corope

#ifdef COROPE_F16
#define COROPE_NS corope_f16
#else
#define COROPE_NS corope
#endif

namespace COROPE_NS {
using namespace corope;

// y = out_scale * rotated x for a (BH, N, D) tensor; tile_max (may be null) receives [BH][ceil(N / 64)] largest row norms.
// (x_sb, x_sh, x_sn: elements between batches, heads and rows of x, with H heads per batch; 0, 0, 0: contiguous)
hipError_t launch_rope_rotate(const uint16_t* x, const float* cosp, const float* sinp, int64_t fstride, uint16_t* y,
                              float* tile_max, int BH, int N, int D, hipStream_t stream, float out_scale = 1.f, int H = 1,
                              int64_t x_sb = 0, int64_t x_sh = 0, int x_sn = 0);
hipError_t launch_rope_attn_fwd_prerotated(const FwdParams& p, int D, bool causal, hipStream_t stream);  // needs k_rot
// the same with 64 query rows per wave, one wave per SIMD (D = 128)
hipError_t launch_rope_attn_fwd_prerotated_rows64(const FwdParams& p, int D, bool causal, hipStream_t stream);
// head dim 256 (bf16): 32 query rows per wave, one wave per SIMD, 32-key tiles
hipError_t launch_rope_attn_fwd_prerotated_pipe256(const FwdParams& p, bool causal, hipStream_t stream);
// head dim 128 in that form (128-row items, 32-key tiles), two workgroups per compute unit
hipError_t launch_rope_attn_fwd_prerotated_pipe32x2(const FwdParams& p, bool causal, hipStream_t stream);
hipError_t launch_rope_attn_fwd(const FwdParams& p, int D, bool causal, hipStream_t stream);
// the single-launch kernel on a rotated key copy (p.k_rot; no key norms needed): no rotation in its loop
hipError_t launch_rope_attn_fwd_single_prerotated(const FwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_bwd_preprocess(const BwdParams& p, int D, hipStream_t stream);
hipError_t launch_bwd_dv(const BwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_bwd_dk(const BwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_bwd_dkdv_fused(const BwdParams& p, int D, bool causal, hipStream_t stream);  // dK and dV in one launch
hipError_t launch_bwd_dq(const BwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_corope_gqa_fwd(const CoropeParams& p, int D, hipStream_t stream);
int64_t corope_gqa_bwd_workspace_floats(int B, int Hq, int Hkv, int N, int D);
hipError_t launch_corope_gqa_bwd(const CoropeBwdParams& p, int D, float* workspace, int64_t workspace_floats,
                                 hipStream_t stream);   // any workspace that holds at least one group's matrices
hipError_t launch_rope_freqs(float* cosp, float* sinp, int n_pos, int D, int width, int64_t row_stride, int pos0,
                             float theta, hipStream_t stream);

}  // namespace COROPE_NS

// The launchers of the fp16 build of the attention kernels (the sources compiled with -DCOROPE_F16): fp16 q, k, v, dO,
// fp16 matrix-core operands, fp16 outputs; same parameter blocks.
namespace corope_f16 {
hipError_t launch_rope_attn_fwd(const corope::FwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_rope_attn_fwd_prerotated(const corope::FwdParams& p, int D, bool causal, hipStream_t stream);  // needs k_rot
hipError_t launch_bwd_preprocess(const corope::BwdParams& p, int D, hipStream_t stream);
hipError_t launch_bwd_dv(const corope::BwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_bwd_dk(const corope::BwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_bwd_dq(const corope::BwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_bwd_dkdv_fused(const corope::BwdParams& p, int D, bool causal, hipStream_t stream);
hipError_t launch_rope_rotate(const uint16_t* x, const float* cosp, const float* sinp, int64_t fstride, uint16_t* y,
                              float* tile_max, int BH, int N, int D, hipStream_t stream, float out_scale, int H, int64_t x_sb,
                              int64_t x_sh, int x_sn);
hipError_t launch_corope_gqa_fwd(const corope::CoropeParams& p, int D, hipStream_t stream);
hipError_t launch_corope_gqa_bwd(const corope::CoropeBwdParams& p, int D, float* workspace, int64_t workspace_floats,
                                 hipStream_t stream);
}  // namespace corope_f16
