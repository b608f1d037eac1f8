// Co-RoPE grouped-query attention forward for gfx950 (causal).
//
// Device counterpart of the reference's _corope_fwd_backbone
// (corope-exp/flash_attn_co_rope_gqa_triton.py:48-400); the definition it must reproduce is
// corope-exp/corope_attn_gqa_pytorch.py:16-134.
//
//   z[i,j]     = sigmoid(s * q_leader[i] . k[j])                      (leader = first query head of the group)
//   delta[i,j] = sum_{j < t <= i} z[i,t]                              (the reference's a[i,i] - a[i,j])
//   score[i,j] = s * sum_d ( (q1 k1 + q2 k2) cos(delta w_d) - (q2 k1 - q1 k2) sin(delta w_d) )
//              = s * q[i] . R(delta[i,j]) k[j]      with R rotating each (k1, k2) pair by -delta w_d
//
// Two restatements keep the work down.  (1) delta is a suffix sum that starts at the diagonal, so key tiles are
// swept right to left and delta accumulates directly: the reference's extra pass over all keys (:103-135) and
// the cancellation in a[i,i] - a[i,j] disappear (online softmax does not care about tile order).  (2) The
// angle is shared by the whole group, so the key pair is rotated once per (i, j, d) and every head of the
// group is then a plain dot product with it: 4 + 2G multiply-adds instead of 6G.
//
// The kernel is bound by the D/2 sin/cos pairs per (query, key) and group, not by matrix math.  Mapping:
// one workgroup = 4 waves = one (batch, kv head) x a block of query rows; each wave owns R = 32/G rows, i.e.
// 32 (row, head) "virtual rows".  For one key tile (64 keys) a wave works in two domains:
//   lane = key:   the key row sits in registers (fp32); query values are wave-uniform and come in through
//                 scalar loads; per row: leader logit, gate, suffix scan across lanes, then the rotated dots
//                 for the G heads; raw scores go to an LDS scratch [virtual row][key];
//   lane = virtual row (MFMA layout): online softmax exactly as in the RoPE-attention forward, then
//                 O^T += V^T P^T with 32x32x16 bf16 MFMAs (V tile read transposed from LDS).
#include "common.hpp"
#include "kernels.hpp"

namespace corope {

constexpr int kCoBlockN = 64;   // keys per tile == lanes per wave
constexpr int kCoWaves = 4;

struct CoropeFreqs {
  float w[64];  // inverse frequencies divided by 2*pi (revolutions per unit of delta), D/2 entries used
};

template <int D, int G>
struct CoropeCfg {
  static constexpr int kR = 32 / G;                                    // query rows per wave
  static constexpr int kRowsWg = kR * kCoWaves;                        // query rows per workgroup
  static constexpr int kQW = 2 * G;                                    // floats per (row, rotation pair): (q1, q2) per head
  static constexpr int kSStride = kCoBlockN + 4;                       // floats per scratch row
  static constexpr int kKBytes = RowTile<D>::bytes(kCoBlockN);          // K tile, row-major bf16, read row-wise
  static constexpr int kVPad = 32;                                     // V tile is read only through the transposing load
  static constexpr int kVBytes = RowTile<D, kVPad>::bytes(kCoBlockN);
  static constexpr int kSBytes = 32 * kSStride * 4;                     // score scratch, per wave
  static constexpr int kQBytes = kRowsWg * (D / 2) * kQW * 4;           // the workgroup's queries as fp32, all heads
  static constexpr int kWBytes = (D / 2) * 4;                           // inverse frequencies
  static constexpr int kOffV = kKBytes;
  static constexpr int kOffS = kOffV + kVBytes;
  static constexpr int kOffQ = kOffS + kCoWaves * kSBytes;
  static constexpr int kOffW = kOffQ + kQBytes;
  static constexpr int kLdsBytes = kOffW + kWBytes;
};

template <int D, int G>
__global__ __launch_bounds__(kCoWaves* kWave) void corope_gqa_fwd_kernel(CoropeParams p, CoropeFreqs fr) {
  using Cfg = CoropeCfg<D, G>;
  constexpr int R = Cfg::kR;             // query rows per wave
  constexpr int VR = R * G;              // virtual rows in use (<= 32)
  constexpr int ROWS_WG = Cfg::kRowsWg;  // query rows per workgroup
  constexpr int HALF = D / 2, NDB = D / 32;
  constexpr int LSV = RowTile<D, Cfg::kVPad>::kStride;
  constexpr int NT = kCoWaves * kWave;
  constexpr int QW = Cfg::kQW;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t* ks = reinterpret_cast<uint16_t*>(smem);
  uint16_t* vs = reinterpret_cast<uint16_t*>(smem + Cfg::kOffV);
  float* qs = reinterpret_cast<float*>(smem + Cfg::kOffQ);
  float* ws = reinterpret_cast<float*>(smem + Cfg::kOffW);

  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  float* ss = reinterpret_cast<float*>(smem + Cfg::kOffS + wave * Cfg::kSBytes);

  const int n_groups = p.B * p.Hkv;
  const int grp = blockIdx.x % n_groups;                       // (batch, kv head)
  const int mb = p.num_m_blocks - 1 - blockIdx.x / n_groups;   // heaviest row blocks first
  const int b = grp / p.Hkv, kvh = grp % p.Hkv;
  const int N = p.N;
  const int m0 = mb * ROWS_WG;
  const int row0 = m0 + wave * R;                              // first query row of this wave
  const int row_hi = min(row0 + R - 1, N - 1);

  const uint16_t* kg = p.k + ((int64_t)b * p.Hkv + kvh) * N * D;
  const uint16_t* vg = p.v + ((int64_t)b * p.Hkv + kvh) * N * D;
  const uint32_t* qg = reinterpret_cast<const uint32_t*>(p.q + ((int64_t)b * p.Hq + (int64_t)kvh * G) * N * D);
  const int64_t q_head_words = (int64_t)N * D / 2;              // 32-bit words between consecutive heads

  // MFMA-domain identity of this lane
  const int lv = lane % 32, lh = lane / 32;                    // virtual row, lane half
  const int my_row = row0 + lv / G;                            // query row of the virtual row
  const int my_head = lv % G;

  f32x16 oacc[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i) oacc[i] = f32x16{0};
  float m_run = -INFINITY, l_run = 0.f;
  float carry_v = 0.f;                                         // lane r holds the mileage carried by row r

  const float scale2 = p.sm_scale * 1.4426950408889634f;
  const int t_hi = min(m0 + ROWS_WG - 1, N - 1) / kCoBlockN;

  // ---- the workgroup's query rows, all heads of the group, as fp32 in LDS: [row][pair d][head][q1, q2] -----------
  // (wave-uniform operands of the lane = key domain are read from here with broadcast LDS loads)
  for (int u = threadIdx.x; u < ROWS_WG * G * (HALF / 8); u += NT) {
    const int ch = u % (HALF / 8), g = (u / (HALF / 8)) % G, row = u / ((HALF / 8) * G);
    const uint32_t* src = qg + (int64_t)g * q_head_words + (int64_t)min(m0 + row, N - 1) * (D / 2) + ch * 4;
    u32x4 x1 = *reinterpret_cast<const u32x4*>(src);
    u32x4 x2 = *reinterpret_cast<const u32x4*>(src + HALF / 2);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = e % 2 ? bf16_hi(x1[e / 2]) : bf16_lo(x1[e / 2]);
      float b2 = e % 2 ? bf16_hi(x2[e / 2]) : bf16_lo(x2[e / 2]);
      *reinterpret_cast<f32x2*>(qs + ((row * HALF) + ch * 8 + e) * QW + 2 * g) = f32x2{a, b2};
    }
  }
  if (threadIdx.x < HALF) ws[threadIdx.x] = fr.w[threadIdx.x];

  CopyStage<D, kCoBlockN, NT> kst;
  CopyStage<D, kCoBlockN, NT, Cfg::kVPad> vst;
  for (int t = t_hi; t >= 0; --t) {
    const int n0 = t * kCoBlockN;
    kst.load(kg, n0, N);
    vst.load(vg, n0, N);
    __syncthreads();  // previous tile fully consumed
    kst.store_rows(ks);
    vst.store_rows(vs);
    __syncthreads();

    if (n0 <= row_hi) {
      // ------------------------------------------------------------------ lane = key
      float k1[HALF], k2[HALF];
      {
        const uint16_t* kr = ks + RowTile<D>::off(lane, 0);
#pragma unroll
        for (int c = 0; c < HALF / 8; ++c) {
          u32x4 a = *reinterpret_cast<const u32x4*>(kr + 8 * c);
          u32x4 bq = *reinterpret_cast<const u32x4*>(kr + HALF + 8 * c);
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            k1[8 * c + 2 * w] = bf16_lo(a[w]);
            k1[8 * c + 2 * w + 1] = bf16_hi(a[w]);
            k2[8 * c + 2 * w] = bf16_lo(bq[w]);
            k2[8 * c + 2 * w + 1] = bf16_hi(bq[w]);
          }
        }
      }
      const int key = n0 + lane;
#pragma unroll 1
      for (int r = 0; r < R; ++r) {
        const int row = min(row0 + r, N - 1);                   // wave-uniform
        const float* qrow = qs + (wave * R + r) * HALF * QW;     // fp32 (q1, q2) pairs of every head, broadcast reads
        // leader logit (head 0 of the group)
        float logit = 0.f;
        {
          // chunks of 8 pairs, fetched one chunk ahead; the scheduling barrier keeps the (fully unrolled) loop from
          // hoisting every LDS read to the top and drowning in registers
          f32x2 qc[8], qn[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) qc[e] = *reinterpret_cast<const f32x2*>(qrow + e * QW);
#pragma unroll
          for (int d8 = 0; d8 < HALF; d8 += 8) {
            if (d8 + 8 < HALF) {
#pragma unroll
              for (int e = 0; e < 8; ++e) qn[e] = *reinterpret_cast<const f32x2*>(qrow + (d8 + 8 + e) * QW);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              logit = __builtin_fmaf(qc[e][0], k1[d8 + e], logit);
              logit = __builtin_fmaf(qc[e][1], k2[d8 + e], logit);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < 8; ++e) qc[e] = qn[e];
          }
        }
        float z = 1.f / (1.f + __expf(-logit * p.sm_scale));
        if (key > row) z = 0.f;                                  // gates beyond the diagonal do not count
        // inclusive suffix sum over the lanes (keys to the right within the tile)
        float suf = z;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
          float o = __shfl_down(suf, off);
          if (lane + off < kWave) suf += o;
        }
        const float carry = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, carry_v), r));
        const float delta = carry + (suf - z);
        const float total = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, suf)));
        if (lane == r) carry_v = carry + total;

        float acc[G];
#pragma unroll
        for (int g = 0; g < G; ++g) acc[g] = 0.f;
        {
          constexpr int CH = G <= 4 ? 4 : 2;   // rotation pairs per chunk (bounds the registers of the look-ahead)
          typedef float wvec __attribute__((ext_vector_type(CH)));
          f32x2 qc[CH][G], qn[CH][G];
          wvec wc = *reinterpret_cast<const wvec*>(ws), wn = wc;
#pragma unroll
          for (int e = 0; e < CH; ++e)
#pragma unroll
            for (int g = 0; g < G; ++g) qc[e][g] = *reinterpret_cast<const f32x2*>(qrow + e * QW + 2 * g);
#pragma unroll
          for (int d0 = 0; d0 < HALF; d0 += CH) {
            if (d0 + CH < HALF) {
              wn = *reinterpret_cast<const wvec*>(ws + d0 + CH);
#pragma unroll
              for (int e = 0; e < CH; ++e)
#pragma unroll
                for (int g = 0; g < G; ++g) qn[e][g] = *reinterpret_cast<const f32x2*>(qrow + (d0 + CH + e) * QW + 2 * g);
            }
#pragma unroll
            for (int e = 0; e < CH; ++e) {
              const int d = d0 + e;
              float x = __builtin_amdgcn_fractf(delta * wc[e]);
              float sn = __builtin_amdgcn_sinf(x), cs = __builtin_amdgcn_cosf(x);
              float r1 = __builtin_fmaf(cs, k1[d], sn * k2[d]);
              float r2 = __builtin_fmaf(cs, k2[d], -(sn * k1[d]));
#pragma unroll
              for (int g = 0; g < G; ++g) {
                acc[g] = __builtin_fmaf(qc[e][g][0], r1, acc[g]);
                acc[g] = __builtin_fmaf(qc[e][g][1], r2, acc[g]);
              }
            }
            __builtin_amdgcn_sched_barrier(0);
            wc = wn;
#pragma unroll
            for (int e = 0; e < CH; ++e)
#pragma unroll
              for (int g = 0; g < G; ++g) qc[e][g] = qn[e][g];
          }
        }
#pragma unroll
        for (int g = 0; g < G; ++g) ss[(r * G + g) * Cfg::kSStride + lane] = acc[g] * scale2;
      }
    }
    __syncthreads();  // scratch written (each wave reads only its own scratch; the barrier orders LDS traffic)

    if (n0 <= row_hi) {
      // ------------------------------------------------------------------ lane = virtual row
      float sv[kCoBlockN / 16][8];
      const bool diag = n0 + kCoBlockN - 1 > row0;
      float mt = -INFINITY;
#pragma unroll
      for (int c = 0; c < kCoBlockN / 16; ++c) {
        const float* sp = ss + lv * Cfg::kSStride + 16 * c + 8 * lh;
        f32x4 a = *reinterpret_cast<const f32x4*>(sp), bq = *reinterpret_cast<const f32x4*>(sp + 4);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float x = j < 4 ? a[j] : bq[j - 4];
          if (diag && (n0 + 16 * c + 8 * lh + j) > my_row) x = -INFINITY;
          sv[c][j] = x;
          mt = fmaxf(mt, x);
        }
      }
      mt = half_max(mt);
      // A wave's rows may straddle a tile boundary: a row below the tile sees no key of it yet (all -inf).
      const float m_max = fmaxf(m_run, mt);
      const float m_new = m_max == -INFINITY ? 0.f : m_max;
      const float alpha = fast_exp2(m_run - m_new);
      m_run = m_max;
      float lsum = 0.f;
      u32x4 pb[kCoBlockN / 16];
#pragma unroll
      for (int c = 0; c < kCoBlockN / 16; ++c)
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
          float p0 = fast_exp2(sv[c][j] - m_new), p1 = fast_exp2(sv[c][j + 1] - m_new);
          lsum += p0 + p1;
          pb[c][j / 2] = pack_bf16(p0, p1);
        }
      l_run = l_run * alpha + lsum;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
#pragma unroll
      for (int c = 0; c < kCoBlockN / 16; ++c)
#pragma unroll
        for (int db = 0; db < NDB; ++db)
          oacc[db] = mfma32(load_a_trans_natural(vs, LSV, 16 * c, db * 32), pb[c], oacc[db]);
    }
  }

  const float l_tot = half_sum(l_run);
  const float inv_l = l_tot > 0.f ? 1.f / l_tot : 0.f;   // same guard as the reference's epilogue (:343-345)
  if (lv < VR && my_row < N) {
    uint16_t* op = p.o + (((int64_t)b * p.Hq + kvh * G + my_head) * N + my_row) * D;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w = {pack_bf16(oacc[db][4 * g] * inv_l, oacc[db][4 * g + 1] * inv_l),
                   pack_bf16(oacc[db][4 * g + 2] * inv_l, oacc[db][4 * g + 3] * inv_l)};
        *reinterpret_cast<u32x2*>(op + db * 32 + 8 * g + 4 * lh) = w;
      }
  }
}

template <int D, int G>
static hipError_t launch_corope_cfg(CoropeParams p, const CoropeFreqs& fr, hipStream_t stream) {
  using Cfg = CoropeCfg<D, G>;
  auto kern = corope_gqa_fwd_kernel<D, G>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       Cfg::kLdsBytes);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  constexpr int rows_wg = Cfg::kRowsWg;
  p.num_m_blocks = (p.N + rows_wg - 1) / rows_wg;
  hipLaunchKernelGGL(kern, dim3(p.num_m_blocks * p.B * p.Hkv), dim3(kCoWaves * kWave), Cfg::kLdsBytes, stream, p, fr);
  return hipGetLastError();
}

template <int D>
static hipError_t launch_corope_d(const CoropeParams& p, const CoropeFreqs& fr, hipStream_t stream) {
  switch (p.Hq / p.Hkv) {
    case 1: return launch_corope_cfg<D, 1>(p, fr, stream);
    case 2: return launch_corope_cfg<D, 2>(p, fr, stream);
    case 3: return launch_corope_cfg<D, 3>(p, fr, stream);
    case 4: return launch_corope_cfg<D, 4>(p, fr, stream);
    case 5: return launch_corope_cfg<D, 5>(p, fr, stream);
    case 6: return launch_corope_cfg<D, 6>(p, fr, stream);
    case 7: return launch_corope_cfg<D, 7>(p, fr, stream);
    case 8: return launch_corope_cfg<D, 8>(p, fr, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_corope_gqa_fwd(const CoropeParams& p, int D, hipStream_t stream) {
  CoropeFreqs fr{};
  // theta^(-2d/D) evaluated like the reference's torch expression (fp32 exponent, fp32 power), then / 2 pi
  for (int d = 0; d < D / 2; ++d) {
    float e = (float)(2 * d) / (float)D;
    float inv = 1.0f / powf(p.theta, e);
    fr.w[d] = (float)((double)inv / 6.283185307179586);
  }
  return D == 128 ? launch_corope_d<128>(p, fr, stream) : launch_corope_d<64>(p, fr, stream);
}

}  // namespace corope
