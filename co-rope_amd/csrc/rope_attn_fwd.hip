// Fused half-layout-RoPE flash-attention forward for gfx950.
//
// Device counterpart of the reference's _attn_fwd / _attn_fwd_inner
// (fused-rope/fused_rope_attn.py:222-320, :48-138).
//
// One workgroup owns BLOCK_M = 32 * NWAVES query rows of one (batch, head); each wave owns 32 of them.
// Scores are produced transposed, S^T = K_r Q_r^T, with 32x32x16 bf16 MFMAs: the rotated K tile is the A
// operand (read from LDS), the rotated Q rows are the B operand (registers, loaded and rotated once).  In
// the 32x32 accumulator every lane then holds 16 keys of ONE query, so the online-softmax row statistics
// are a per-lane reduction plus one exchange between the two halves of the wave, and the bf16 P^T values
// are already laid out as the B operand of O^T += V^T P^T (V^T read from a transposed LDS tile).
//
// K tiles are rotated while they are staged global -> registers -> LDS, once per workgroup per tile
// (the reference re-rotates per program: :82-99); the next tile's global loads are issued before the
// current tile's MFMAs and written to the other LDS buffer afterwards (one barrier per tile).
#include "common.hpp"
#include "kernels.hpp"

namespace corope {

template <int D, int NWAVES, int BLOCK_N>
struct FwdCfg {
  static constexpr int kThreads = NWAVES * kWave;
  static constexpr int kBlockM = NWAVES * 32;
  static constexpr int kKBytes = RowTile<D>::bytes(BLOCK_N);
  static constexpr int kVBytes = TransTile<BLOCK_N>::bytes(D);
  static constexpr int kStageBytes = kKBytes + kVBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
};

template <int D, int NWAVES, int BLOCK_N, bool CAUSAL>
__global__ __launch_bounds__(NWAVES* kWave) void rope_attn_fwd_kernel(FwdParams p) {
  using Cfg = FwdCfg<D, NWAVES, BLOCK_N>;
  constexpr int NT = Cfg::kThreads;
  constexpr int KC = D / 16;        // contraction chunks of QK^T
  constexpr int NKB = BLOCK_N / 32; // 32-key blocks per tile
  constexpr int NDB = D / 32;       // 32-column blocks of O
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  // Heaviest query blocks first; consecutive workgroup ids walk over (batch, head) so that all blocks of one
  // head land on the same XCD (ids are dealt round-robin to the 8 XCDs) and share its L2.
  const int bh = blockIdx.x % p.BH;
  const int mb = p.num_m_blocks - 1 - blockIdx.x / p.BH;
  const int m0 = mb * Cfg::kBlockM;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lq = lane % 32, lh = lane / 32;
  const int N = p.N;

  const uint16_t* qg = p.q + (int64_t)bh * N * D;
  const uint16_t* kg = p.k + (int64_t)bh * N * D;
  const uint16_t* vg = p.v + (int64_t)bh * N * D;

  const int n_tiles = CAUSAL ? min((m0 + Cfg::kBlockM + BLOCK_N - 1) / BLOCK_N, (N + BLOCK_N - 1) / BLOCK_N)
                             : (N + BLOCK_N - 1) / BLOCK_N;

  RotStage<D, BLOCK_N, NT> kst;
  TransStage<D, BLOCK_N, NT> vst;
  kst.load(kg, p.cos, p.sin, p.fstride, 0, N);
  vst.load(vg, 0, N);

  // ---- Q rows of this wave: load, rotate, keep as the B operand ------------------------------------------
  const int q_row = m0 + wave * 32 + lq;           // absolute query index of this lane
  u32x4 qb[KC];
  {
    const int qr = min(q_row, N - 1);
    const uint16_t* qp = qg + (int64_t)qr * D + 8 * lh;
    const float* cp = p.cos + (int64_t)qr * p.fstride + 8 * lh;
    const float* sp = p.sin + (int64_t)qr * p.fstride + 8 * lh;
#pragma unroll
    for (int kc = 0; kc < KC / 2; ++kc) {
      u32x4 x1 = *reinterpret_cast<const u32x4*>(qp + 16 * kc);
      u32x4 x2 = *reinterpret_cast<const u32x4*>(qp + D / 2 + 16 * kc);
      f32x4 c0 = *reinterpret_cast<const f32x4*>(cp + 16 * kc), c1 = *reinterpret_cast<const f32x4*>(cp + 16 * kc + 4);
      f32x4 s0 = *reinterpret_cast<const f32x4*>(sp + 16 * kc), s1 = *reinterpret_cast<const f32x4*>(sp + 16 * kc + 4);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float a0 = bf16_lo(x1[w]), a1 = bf16_hi(x1[w]), b0 = bf16_lo(x2[w]), b1 = bf16_hi(x2[w]);
        float cc0 = w < 2 ? c0[2 * w] : c1[2 * w - 4], cc1 = w < 2 ? c0[2 * w + 1] : c1[2 * w - 3];
        float ss0 = w < 2 ? s0[2 * w] : s1[2 * w - 4], ss1 = w < 2 ? s0[2 * w + 1] : s1[2 * w - 3];
        qb[kc][w] = pack_bf16(a0 * cc0 - b0 * ss0, a1 * cc1 - b1 * ss1);
        qb[kc + KC / 2][w] = pack_bf16(b0 * cc0 + a0 * ss0, b1 * cc1 + a1 * ss1);
      }
    }
  }

  f32x16 oacc[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i) oacc[i] = f32x16{0};
  float m_run = -INFINITY;   // running row maximum of the raw scores (this lane's query)
  float l_run = 0.f;         // this lane's share of the running denominator

  auto ks = [&](int buf) { return reinterpret_cast<uint16_t*>(smem + buf * Cfg::kStageBytes); };
  auto vs = [&](int buf) { return reinterpret_cast<uint16_t*>(smem + buf * Cfg::kStageBytes + Cfg::kKBytes); };
  kst.store_rows(ks(0));
  vst.store(vs(0));
  __syncthreads();

  const float scale = p.qk_scale;
  const int wave_q_lo = m0 + wave * 32, wave_q_hi = wave_q_lo + 31;

  for (int t = 0; t < n_tiles; ++t) {
    const int n0 = t * BLOCK_N;
    const int cur = t & 1;
    if (t + 1 < n_tiles) {
      kst.load(kg, p.cos, p.sin, p.fstride, n0 + BLOCK_N, N);
      vst.load(vg, n0 + BLOCK_N, N);
    }
    // Tiles entirely above this wave's diagonal contribute nothing to it.
    const bool active = !CAUSAL || n0 <= wave_q_hi;
    if (active) {
      // ---- S^T = K_r Q_r^T -----------------------------------------------------------------------------
      f32x16 sacc[NKB];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        sacc[kb] = f32x16{0};
        const uint16_t* kp = ks(cur) + RowTile<D>::off(kb * 32 + lq, 8 * lh);
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
          u32x4 a = *reinterpret_cast<const u32x4*>(kp + 16 * kc);
          sacc[kb] = mfma32(a, qb[kc], sacc[kb]);
        }
      }
      // ---- masking (diagonal tiles, ragged tail) -----------------------------------------------------
      const bool need_mask = (CAUSAL && n0 + BLOCK_N - 1 > wave_q_lo) || (!CAUSAL && n0 + BLOCK_N > N);
      if (need_mask) {
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            int key = n0 + kb * 32 + acc_row(i, lh);
            bool dead = CAUSAL ? key > q_row : key >= N;
            if (dead) sacc[kb][i] = -INFINITY;
          }
      }
      // ---- online softmax (base 2) -----------------------------------------------------------------
      float mt = sacc[0][0];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mt = fmaxf(mt, sacc[kb][i]);
      mt = half_max(mt);
      const float m_new = fmaxf(m_run, mt);
      const float ms = m_new * scale;
      const float alpha = fast_exp2(m_run * scale - ms);
      m_run = m_new;
      float lsum = 0.f;
      u32x4 pb[BLOCK_N / 16];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          float p0 = fast_exp2(sacc[kb][i] * scale - ms);
          float p1 = fast_exp2(sacc[kb][i + 1] * scale - ms);
          lsum += p0 + p1;
          pb[2 * kb + i / 8][(i % 8) / 2] = pack_bf16(p0, p1);
        }
      l_run = l_run * alpha + lsum;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
      }
      // ---- O^T += V^T P^T ------------------------------------------------------------------------------
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        const uint16_t* vp = vs(cur) + (db * 32 + lq) * TransTile<BLOCK_N>::kStride + 8 * lh;
#pragma unroll
        for (int c = 0; c < BLOCK_N / 16; ++c) {
          u32x4 a = *reinterpret_cast<const u32x4*>(vp + 16 * c);
          oacc[db] = mfma32(a, pb[c], oacc[db]);
        }
      }
    }
    if (t + 1 < n_tiles) {
      kst.store_rows(ks(cur ^ 1));
      vst.store(vs(cur ^ 1));
    }
    __syncthreads();
  }

  // ---- epilogue: normalise, write O and the base-2 log-sum-exp ----------------------------------------------
  const float l_tot = half_sum(l_run);
  const float inv_l = 1.f / l_tot;
  if (q_row < N) {
    uint16_t* op = p.o + ((int64_t)bh * N + q_row) * D;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = pack_bf16(oacc[db][4 * g] * inv_l, oacc[db][4 * g + 1] * inv_l);
        w[1] = pack_bf16(oacc[db][4 * g + 2] * inv_l, oacc[db][4 * g + 3] * inv_l);
        *reinterpret_cast<u32x2*>(op + db * 32 + 8 * g + 4 * lh) = w;
      }
    if (lh == 0) p.lse[(int64_t)bh * N + q_row] = m_run * scale + fast_log2(l_tot);
  }
}

// ---- host-side launch -----------------------------------------------------------------------------------------
template <int D, int NWAVES, int BLOCK_N, bool CAUSAL>
static hipError_t launch_fwd_cfg(FwdParams p, hipStream_t stream) {
  using Cfg = FwdCfg<D, NWAVES, BLOCK_N>;
  auto kern = rope_attn_fwd_kernel<D, NWAVES, BLOCK_N, CAUSAL>;
  static bool attr_set = false;  // per instantiation; benign if raced (same value)
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       Cfg::kLdsBytes);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  p.num_m_blocks = (p.N + Cfg::kBlockM - 1) / Cfg::kBlockM;
  dim3 grid(p.num_m_blocks * p.BH);
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, p);
  return hipGetLastError();
}

hipError_t launch_rope_attn_fwd(const FwdParams& p, int D, bool causal, hipStream_t stream) {
  if (D == 128) {
    return causal ? launch_fwd_cfg<128, 8, 64, true>(p, stream) : launch_fwd_cfg<128, 8, 64, false>(p, stream);
  }
  return causal ? launch_fwd_cfg<64, 8, 64, true>(p, stream) : launch_fwd_cfg<64, 8, 64, false>(p, stream);
}

}  // namespace corope
