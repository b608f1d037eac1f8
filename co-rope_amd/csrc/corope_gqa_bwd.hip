// Co-RoPE grouped-query attention backward for gfx950.
//
// The reference's "fused" Co-RoPE operator falls back to a dense PyTorch backward that materialises (B, Hq, N, N, D/2)
// temporaries (corope-exp/flash_attn_co_rope_gqa_triton.py:459-577; same mathematics as the manual backward of
// corope-exp/corope_attn_gqa_pytorch.py:137-300).  This file computes the same gradients with O(N^2) scalars per head
// in a caller-supplied workspace and no D-sized temporaries.
//
// Mathematics (group = the Hq/Hkv query heads sharing one key/value head; leader = first head of the group;
// c = sm_scale; w_d = theta^(-2d/D); pairs (d, d + D/2) as in the forward):
//   z_it    = sigmoid(c qL_i . k_t)                      delta_ij = sum_{j < t <= i} z_it
//   S^h_ij  = c sum_d [ q1 (k1 cos phi + k2 sin phi) + q2 (k2 cos phi - k1 sin phi) ],   phi = delta_ij w_d
//           = c q^h_i . kt_ij  =  c k_j . qt^h_ij       (kt, qt: the key / the query rotated by -/+ phi)
//   P = softmax_j(S),  dP^h_ij = dO^h_i . v_j,  dS = P o (dP - rowsum(P o dP))
//   dv_j    = sum_{h,i} P^h_ij dO^h_i
//   dq^h_i  = c sum_j dS^h_ij kt_ij                      dk_j = c sum_{h,i} dS^h_ij qt^h_ij      (paths with delta fixed)
//   through delta:  g^h_ij = dS/ddelta = c sum_d w_d (q1 kt2 - q2 kt1),   G_ij = sum_h dS^h_ij g^h_ij,
//                   dz_it = sum_{j < t} G_ij,   W_it = dz_it z_it (1 - z_it)   (gradient of the leader's logit),
//                   dqL_i += c sum_t W_it k_t,   dk_t += c sum_i W_it qL_i.
//
// Four kernels, each a plain loop nest over (query row, key) pairs with one wave per row (or per few keys):
//   gates   (lane = key):   z, delta by a right-to-left suffix scan             -> DELTA, ZP   [group][N][N]
//   scores  (lane = key):   S, P, dP, dS for all heads of the group             -> P, DS       [head][N][N]
//   dq      (lane = pair):  dq, G and its prefix sum, W, leader's dq            -> W           [group][N][N]
//   dkdv    (lane = pair):  dk, dv for 32 keys per workgroup, tiles of the matrices staged through LDS
// "lane = key" makes every dot product over d a per-lane loop (no reductions); "lane = pair" makes every sum over keys
// or queries a per-lane accumulation (the only cross-lane reduction left is G_ij, one per (i, j)).
#include "common.hpp"
#include "kernels.hpp"

namespace corope {

struct CoropeBwdFreqs {
  float turns[64];   // w_d / (2 pi): phase in revolutions per unit of delta (what v_sin_f32 / v_cos_f32 take)
  float rad[64];     // w_d
};

// Workspace layout, in floats; NN = N * N.
struct CoropeBwdWs {
  float* base;
  int64_t NN;
  int n_groups, n_heads;
  __device__ __host__ float* delta(int g) const { return base + (int64_t)g * NN; }
  __device__ __host__ float* zp(int g) const { return base + (int64_t)(n_groups + g) * NN; }
  __device__ __host__ float* w(int g) const { return base + (int64_t)(2 * n_groups + g) * NN; }
  __device__ __host__ float* p(int h) const { return base + (int64_t)(3 * n_groups + h) * NN; }
  __device__ __host__ float* ds(int h) const { return base + (int64_t)(3 * n_groups + n_heads + h) * NN; }
};

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = fmaxf(x, __shfl_xor(x, m));
  return x;
}

// One (N, D) bf16 row as D/8 16-byte words in registers; element e as float.
template <int D>
struct RowRegs {
  u32x4 w[D / 8];
  __device__ __forceinline__ void load(const uint16_t* row) {
#pragma unroll
    for (int i = 0; i < D / 8; ++i) w[i] = *reinterpret_cast<const u32x4*>(row + 8 * i);
  }
  __device__ __forceinline__ float at(int e) const {   // e: compile-time after unrolling
    const uint32_t x = w[e / 8][(e % 8) / 2];
    return (e % 2) ? bf16_hi(x) : bf16_lo(x);
  }
};

__device__ __forceinline__ float bf16_to_f(uint16_t x) { return __builtin_bit_cast(float, (uint32_t)x << 16); }
__device__ __forceinline__ uint16_t f_to_bf16(float x) { return (uint16_t)(pack_bf16(x, 0.f) & 0xffffu); }

// ---------------------------------------------------------------------------------------------------- gates
// One wave per (group, query row i), lane = key inside a 64-key chunk, chunks from the diagonal to the left.
template <int D>
__global__ __launch_bounds__(kWave) void corope_bwd_gates_kernel(CoropeBwdParams p, CoropeBwdWs ws) {
  __shared__ float ql[D];
  const int i = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv, G = p.Hq / p.Hkv;
  const uint16_t* qrow = p.q + (((int64_t)b * p.Hq + kvh * G) * N + i) * D;   // the leader's row
  const uint16_t* kbase = p.k + (int64_t)g * N * D;
  for (int d = lane; d < D; d += kWave) ql[d] = bf16_to_f(qrow[d]);
  __syncthreads();
  float* drow = ws.delta(g) + (int64_t)i * N;
  float* zrow = ws.zp(g) + (int64_t)i * N;
  float carry = 0.f;   // sum of z over the keys to the right of the current chunk (up to the diagonal)
  for (int c = i / kWave; c >= 0; --c) {
    const int j = c * kWave + lane;
    const bool valid = j <= i;
    RowRegs<D> kr;
    kr.load(kbase + (int64_t)(valid ? j : i) * D);
    float dot = 0.f;
#pragma unroll
    for (int d = 0; d < D; ++d) dot = __builtin_fmaf(ql[d], kr.at(d), dot);
    const float z = valid ? 1.f / (1.f + __expf(-dot * p.sm_scale)) : 0.f;
    float s = z;   // inclusive suffix sum over the lanes (keys) at and to the right of this one
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const float t = __shfl_down(s, off);
      if (lane + off < kWave) s += t;
    }
    if (valid) {
      drow[j] = carry + s - z;   // z of the keys strictly to the right, up to and including the diagonal
      zrow[j] = z * (1.f - z);
    }
    carry += __shfl(s, 0);
  }
}

// ---------------------------------------------------------------------------------------------------- scores
// One wave per (group, query row i), all G heads at once, lane = key.  Four sweeps over the row's keys: raw scores and
// their maxima; exponentials and their sums; P, dP and rowsum(P o dP); dS.  Only the first sweep evaluates sines and
// cosines.  The row sum is taken from P and dP themselves, as the reference does (:526-528), so the forward's rounded
// output is not an input of the backward.
template <int D, int G>
__global__ __launch_bounds__(kWave) void corope_bwd_scores_kernel(CoropeBwdParams p, CoropeBwdWs ws, CoropeBwdFreqs fr) {
  constexpr int HALF = D / 2;
  __shared__ float qs[HALF][G][2];   // (q1, q2) of every head per rotation pair
  __shared__ float dos[D][G];        // dO of every head per column
  const int i = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv;
  const int head0 = b * p.Hq + kvh * G;   // first head of the group, as a (batch, head) slab index
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const int64_t off = ((int64_t)(head0 + h) * N + i) * D;
    for (int d = lane; d < D; d += kWave) {
      qs[d % HALF][h][d / HALF] = bf16_to_f(p.q[off + d]);
      dos[d][h] = bf16_to_f(p.d_o[off + d]);
    }
  }
  __syncthreads();
  const uint16_t* kbase = p.k + (int64_t)g * N * D;
  const uint16_t* vbase = p.v + (int64_t)g * N * D;
  const float* drow = ws.delta(g) + (int64_t)i * N;
  const int n_chunks = i / kWave + 1;

  // ---- sweep 1: raw scores ---------------------------------------------------------------------------------------
  float mx[G];
#pragma unroll
  for (int h = 0; h < G; ++h) mx[h] = -INFINITY;
  for (int c = 0; c < n_chunks; ++c) {
    const int j = c * kWave + lane;
    const bool valid = j <= i;
    RowRegs<D> kr;
    kr.load(kbase + (int64_t)(valid ? j : i) * D);
    const float delta = valid ? drow[j] : 0.f;
    float acc[G];
#pragma unroll
    for (int h = 0; h < G; ++h) acc[h] = 0.f;
#pragma unroll
    for (int d = 0; d < HALF; ++d) {
      const float x = __builtin_amdgcn_fractf(delta * fr.turns[d]);
      const float sn = __builtin_amdgcn_sinf(x), cs = __builtin_amdgcn_cosf(x);
      const float k1 = kr.at(d), k2 = kr.at(d + HALF);
      const float kt1 = __builtin_fmaf(cs, k1, sn * k2), kt2 = __builtin_fmaf(cs, k2, -(sn * k1));
#pragma unroll
      for (int h = 0; h < G; ++h) acc[h] = __builtin_fmaf(qs[d][h][0], kt1, __builtin_fmaf(qs[d][h][1], kt2, acc[h]));
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float s = acc[h] * p.sm_scale;
      if (valid) {
        ws.p(head0 + h)[(int64_t)i * N + j] = s;
        mx[h] = fmaxf(mx[h], s);
      }
    }
  }
#pragma unroll
  for (int h = 0; h < G; ++h) mx[h] = wave_max(mx[h]);

  // ---- sweep 2: exponentials -------------------------------------------------------------------------------------
  float inv_l[G];
#pragma unroll
  for (int h = 0; h < G; ++h) inv_l[h] = 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const int j = c * kWave + lane;
    if (j <= i) {
#pragma unroll
      for (int h = 0; h < G; ++h) {
        float* pp = ws.p(head0 + h) + (int64_t)i * N + j;
        const float e = __expf(*pp - mx[h]);
        *pp = e;
        inv_l[h] += e;
      }
    }
  }
#pragma unroll
  for (int h = 0; h < G; ++h) inv_l[h] = 1.f / wave_sum(inv_l[h]);

  // ---- sweep 3: P, dP = dO . v (parked in DS), rowsum(P o dP) ------------------------------------------------------
  float dsum[G];
#pragma unroll
  for (int h = 0; h < G; ++h) dsum[h] = 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const int j = c * kWave + lane;
    const bool valid = j <= i;
    RowRegs<D> vr;
    vr.load(vbase + (int64_t)(valid ? j : i) * D);
    float dp[G];
#pragma unroll
    for (int h = 0; h < G; ++h) dp[h] = 0.f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float vv = vr.at(d);
#pragma unroll
      for (int h = 0; h < G; ++h) dp[h] = __builtin_fmaf(dos[d][h], vv, dp[h]);
    }
    if (valid) {
#pragma unroll
      for (int h = 0; h < G; ++h) {
        const int64_t at = (int64_t)i * N + j;
        const float pr = ws.p(head0 + h)[at] * inv_l[h];
        ws.p(head0 + h)[at] = pr;
        ws.ds(head0 + h)[at] = dp[h];
        dsum[h] = __builtin_fmaf(pr, dp[h], dsum[h]);
      }
    }
  }
#pragma unroll
  for (int h = 0; h < G; ++h) dsum[h] = wave_sum(dsum[h]);

  // ---- sweep 4: dS = P (dP - rowsum(P o dP)) -----------------------------------------------------------------------
  for (int c = 0; c < n_chunks; ++c) {
    const int j = c * kWave + lane;
    if (j <= i) {
#pragma unroll
      for (int h = 0; h < G; ++h) {
        const int64_t at = (int64_t)i * N + j;
        ws.ds(head0 + h)[at] = ws.p(head0 + h)[at] * (ws.ds(head0 + h)[at] - dsum[h]);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------- dq
// One wave per (group, query row i), lane = rotation pair (d, d + D/2), keys in ascending order so that the prefix sum
// of G is a running scalar.  The key chunk is staged in LDS; the row's scalars (delta, z(1-z), dS per head) are loaded
// with lane = key and handed out with readlane.
template <int D, int G>
__global__ __launch_bounds__(kWave) void corope_bwd_dq_kernel(CoropeBwdParams p, CoropeBwdWs ws, CoropeBwdFreqs fr) {
  constexpr int HALF = D / 2;
  __shared__ __attribute__((aligned(16))) uint16_t kch[kWave][D];   // 64 keys x D, bf16
  const int i = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv;
  const int head0 = b * p.Hq + kvh * G;
  const bool act = lane < HALF;           // D = 64 leaves the upper half of the wave without a pair
  const int dpair = act ? lane : 0;
  const float w_turn = fr.turns[dpair], w_rad = act ? fr.rad[dpair] : 0.f;
  float q1[G], q2[G], dq1[G], dq2[G];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const int64_t off = ((int64_t)(head0 + h) * N + i) * D;
    q1[h] = bf16_to_f(p.q[off + dpair]);
    q2[h] = bf16_to_f(p.q[off + dpair + HALF]);
    dq1[h] = dq2[h] = 0.f;
  }
  float dql1 = 0.f, dql2 = 0.f;   // the leader's extra gradient through its logits
  float gprefix = 0.f;            // sum of G_ij over the keys already visited
  const uint16_t* kbase = p.k + (int64_t)g * N * D;
  const int64_t rowoff = (int64_t)i * N;
  const int n_chunks = i / kWave + 1;
  for (int c = 0; c < n_chunks; ++c) {
    const int j0 = c * kWave, jl = j0 + lane;
    const bool valid = jl <= i;
    __syncthreads();   // the previous chunk's keys are no longer needed
    {
      const uint16_t* src = kbase + (int64_t)(valid ? jl : i) * D;
#pragma unroll
      for (int v8 = 0; v8 < D / 8; ++v8)
        *reinterpret_cast<u32x4*>(&kch[lane][8 * v8]) = *reinterpret_cast<const u32x4*>(src + 8 * v8);
    }
    const float dvec = valid ? ws.delta(g)[rowoff + jl] : 0.f;
    const float zvec = valid ? ws.zp(g)[rowoff + jl] : 0.f;
    float dsvec[G];
#pragma unroll
    for (int h = 0; h < G; ++h) dsvec[h] = valid ? ws.ds(head0 + h)[rowoff + jl] : 0.f;
    __syncthreads();
    float wvec = 0.f;
    const int n_here = min(kWave, i - j0 + 1);
    for (int jj = 0; jj < n_here; ++jj) {
      const float delta = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, dvec), jj));
      const float zp = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zvec), jj));
      const float k1 = bf16_to_f(kch[jj][dpair]), k2 = bf16_to_f(kch[jj][dpair + HALF]);
      const float x = __builtin_amdgcn_fractf(delta * w_turn);
      const float sn = __builtin_amdgcn_sinf(x), cs = __builtin_amdgcn_cosf(x);
      const float kt1 = __builtin_fmaf(cs, k1, sn * k2), kt2 = __builtin_fmaf(cs, k2, -(sn * k1));
      float gacc = 0.f;
#pragma unroll
      for (int h = 0; h < G; ++h) {
        const float ds = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, dsvec[h]), jj));
        dq1[h] = __builtin_fmaf(ds, kt1, dq1[h]);
        dq2[h] = __builtin_fmaf(ds, kt2, dq2[h]);
        gacc = __builtin_fmaf(ds, q1[h] * kt2 - q2[h] * kt1, gacc);
      }
      const float gij = p.sm_scale * wave_sum(gacc * w_rad);   // G_ij: the one cross-lane reduction per (i, j)
      const float wij = gprefix * zp;                          // dz_it z'(t) with the sum over keys j < t
      gprefix += gij;
      dql1 = __builtin_fmaf(wij, k1, dql1);
      dql2 = __builtin_fmaf(wij, k2, dql2);
      wvec = lane == jj ? wij : wvec;
    }
    if (valid) ws.w(g)[rowoff + jl] = wvec;
  }
  if (act) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const int64_t off = ((int64_t)(head0 + h) * N + i) * D;
      const float a1 = dq1[h] + (h == 0 ? dql1 : 0.f), a2 = dq2[h] + (h == 0 ? dql2 : 0.f);
      p.dq[off + dpair] = f_to_bf16(a1 * p.sm_scale);
      p.dq[off + dpair + HALF] = f_to_bf16(a2 * p.sm_scale);
    }
  }
}

// ---------------------------------------------------------------------------------------------------- dk, dv
// One workgroup of 4 waves per (group, block of 32 keys); each wave owns 8 of the keys, lane = rotation pair.  Query
// rows are visited 16 at a time: the 16 x 32 tiles of DELTA, W, DS^h, P^h and the 16 rows of q and dO of every head are
// staged in LDS, so the column-wise access of the N x N matrices costs full 128-byte lines.
constexpr int kDkKeys = 32, kDkRows = 16, kDkWaves = 4, kDkKeysPerWave = kDkKeys / kDkWaves;

template <int D, int G>
struct CoropeDkCfg {
  static constexpr int kMats = 2 + 2 * G;                                   // DELTA, W, DS^h, P^h
  static constexpr int kMatBytes = kMats * kDkRows * kDkKeys * 4;
  static constexpr int kRowBytes = kDkRows * G * D * 2;                     // q rows (and as many dO rows), bf16
  static constexpr int kLdsBytes = kMatBytes + 2 * kRowBytes;
};

template <int D, int G>
__global__ __launch_bounds__(kDkWaves* kWave) void corope_bwd_dkdv_kernel(CoropeBwdParams p, CoropeBwdWs ws,
                                                                         CoropeBwdFreqs fr) {
  using Cfg = CoropeDkCfg<D, G>;
  constexpr int HALF = D / 2, NT = kDkWaves * kWave;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float (*mats)[kDkRows][kDkKeys] = reinterpret_cast<float (*)[kDkRows][kDkKeys]>(smem);
  uint16_t (*qrows)[G][D] = reinterpret_cast<uint16_t (*)[G][D]>(smem + Cfg::kMatBytes);
  uint16_t (*dorows)[G][D] = reinterpret_cast<uint16_t (*)[G][D]>(smem + Cfg::kMatBytes + Cfg::kRowBytes);

  const int jb = blockIdx.x * kDkKeys, g = blockIdx.y;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv;
  const int head0 = b * p.Hq + kvh * G;
  const bool act = lane < HALF;
  const int dpair = act ? lane : 0;
  const float w_turn = fr.turns[dpair];
  const int jw = jb + wave * kDkKeysPerWave;   // first key of this wave

  float dk1[kDkKeysPerWave], dk2[kDkKeysPerWave], dv1[kDkKeysPerWave], dv2[kDkKeysPerWave];
#pragma unroll
  for (int kk = 0; kk < kDkKeysPerWave; ++kk) dk1[kk] = dk2[kk] = dv1[kk] = dv2[kk] = 0.f;

  // rows i >= jb see at least one key of the block
  for (int i0 = (jb / kDkRows) * kDkRows; i0 < N; i0 += kDkRows) {
    __syncthreads();
    // ---- stage the tiles: element (m, r, c) <- matrix m at [i0 + r][jb + c] (zero outside the causal triangle / N) ----
    for (int e = threadIdx.x; e < Cfg::kMats * kDkRows * kDkKeys; e += NT) {
      const int m = e / (kDkRows * kDkKeys), r = (e / kDkKeys) % kDkRows, c = e % kDkKeys;
      const int i = i0 + r, j = jb + c;
      float val = 0.f;
      if (i < N && j <= i) {
        const int64_t at = (int64_t)i * N + j;
        const float* src = m == 0 ? ws.delta(g) : m == 1 ? ws.w(g) : m < 2 + G ? ws.ds(head0 + m - 2) : ws.p(head0 + m - 2 - G);
        val = src[at];
      }
      mats[m][r][c] = val;
    }
    for (int e = threadIdx.x; e < kDkRows * G * (D / 8); e += NT) {
      const int r = e / (G * (D / 8)), h = (e / (D / 8)) % G, v8 = e % (D / 8);
      const int i = min(i0 + r, N - 1);
      const int64_t off = ((int64_t)(head0 + h) * N + i) * D + 8 * v8;
      *reinterpret_cast<u32x4*>(&qrows[r][h][8 * v8]) = *reinterpret_cast<const u32x4*>(p.q + off);
      *reinterpret_cast<u32x4*>(&dorows[r][h][8 * v8]) = *reinterpret_cast<const u32x4*>(p.d_o + off);
    }
    __syncthreads();
    const int n_rows = min(kDkRows, N - i0);
    for (int r = 0; r < n_rows; ++r) {
      const int i = i0 + r;
      float q1[G], q2[G], o1[G], o2[G];
#pragma unroll
      for (int h = 0; h < G; ++h) {
        q1[h] = bf16_to_f(qrows[r][h][dpair]);
        q2[h] = bf16_to_f(qrows[r][h][dpair + HALF]);
        o1[h] = bf16_to_f(dorows[r][h][dpair]);
        o2[h] = bf16_to_f(dorows[r][h][dpair + HALF]);
      }
#pragma unroll
      for (int kk = 0; kk < kDkKeysPerWave; ++kk) {
        const int c = wave * kDkKeysPerWave + kk;
        if (jw + kk > i) continue;   // wave-uniform: keys above the diagonal of this row (their tiles are zero anyway)
        const float delta = mats[0][r][c], wij = mats[1][r][c];
        const float x = __builtin_amdgcn_fractf(delta * w_turn);
        const float sn = __builtin_amdgcn_sinf(x), cs = __builtin_amdgcn_cosf(x);
#pragma unroll
        for (int h = 0; h < G; ++h) {
          const float ds = mats[2 + h][r][c], pr = mats[2 + G + h][r][c];
          const float qt1 = __builtin_fmaf(cs, q1[h], -(sn * q2[h])), qt2 = __builtin_fmaf(cs, q2[h], sn * q1[h]);
          dk1[kk] = __builtin_fmaf(ds, qt1, dk1[kk]);
          dk2[kk] = __builtin_fmaf(ds, qt2, dk2[kk]);
          dv1[kk] = __builtin_fmaf(pr, o1[h], dv1[kk]);
          dv2[kk] = __builtin_fmaf(pr, o2[h], dv2[kk]);
        }
        dk1[kk] = __builtin_fmaf(wij, q1[0], dk1[kk]);   // the leader's logit path (unrotated q)
        dk2[kk] = __builtin_fmaf(wij, q2[0], dk2[kk]);
      }
    }
  }
  if (act) {
#pragma unroll
    for (int kk = 0; kk < kDkKeysPerWave; ++kk) {
      const int j = jw + kk;
      if (j >= N) continue;
      const int64_t off = ((int64_t)g * N + j) * D;
      p.dk[off + dpair] = f_to_bf16(dk1[kk] * p.sm_scale);
      p.dk[off + dpair + HALF] = f_to_bf16(dk2[kk] * p.sm_scale);
      p.dv[off + dpair] = f_to_bf16(dv1[kk]);
      p.dv[off + dpair + HALF] = f_to_bf16(dv2[kk]);
    }
  }
}

// ---------------------------------------------------------------------------------------------------- host side
int64_t corope_gqa_bwd_workspace_floats(int B, int Hq, int Hkv, int N) {
  return (int64_t)N * N * (3 * (int64_t)B * Hkv + 2 * (int64_t)B * Hq);
}

template <int D, int G>
static hipError_t launch_corope_bwd_cfg(const CoropeBwdParams& p, const CoropeBwdWs& ws, const CoropeBwdFreqs& fr,
                                        hipStream_t stream) {
  const dim3 rows(p.N, p.B * p.Hkv);
  hipLaunchKernelGGL(corope_bwd_gates_kernel<D>, rows, dim3(kWave), 0, stream, p, ws);
  hipLaunchKernelGGL((corope_bwd_scores_kernel<D, G>), rows, dim3(kWave), 0, stream, p, ws, fr);
  hipLaunchKernelGGL((corope_bwd_dq_kernel<D, G>), rows, dim3(kWave), 0, stream, p, ws, fr);
  using Cfg = CoropeDkCfg<D, G>;
  auto kern = corope_bwd_dkdv_kernel<D, G>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       Cfg::kLdsBytes);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3((p.N + kDkKeys - 1) / kDkKeys, p.B * p.Hkv), dim3(kDkWaves * kWave), Cfg::kLdsBytes, stream,
                     p, ws, fr);
  return hipGetLastError();
}

template <int D>
static hipError_t launch_corope_bwd_d(const CoropeBwdParams& p, const CoropeBwdWs& ws, const CoropeBwdFreqs& fr,
                                      hipStream_t stream) {
  switch (p.Hq / p.Hkv) {
    case 1: return launch_corope_bwd_cfg<D, 1>(p, ws, fr, stream);
    case 2: return launch_corope_bwd_cfg<D, 2>(p, ws, fr, stream);
    case 3: return launch_corope_bwd_cfg<D, 3>(p, ws, fr, stream);
    case 4: return launch_corope_bwd_cfg<D, 4>(p, ws, fr, stream);
    case 5: return launch_corope_bwd_cfg<D, 5>(p, ws, fr, stream);
    case 6: return launch_corope_bwd_cfg<D, 6>(p, ws, fr, stream);
    case 7: return launch_corope_bwd_cfg<D, 7>(p, ws, fr, stream);
    case 8: return launch_corope_bwd_cfg<D, 8>(p, ws, fr, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_corope_gqa_bwd(const CoropeBwdParams& p, int D, float* workspace, hipStream_t stream) {
  CoropeBwdFreqs fr{};
  // theta^(-2d/D) evaluated like the reference's torch expression (fp32 exponent, fp32 power), as in the forward
  for (int d = 0; d < D / 2; ++d) {
    const float e = (float)(2 * d) / (float)D;
    const float inv = 1.0f / powf(p.theta, e);
    fr.rad[d] = inv;
    fr.turns[d] = (float)((double)inv / 6.283185307179586);
  }
  CoropeBwdWs ws{workspace, (int64_t)p.N * p.N, p.B * p.Hkv, p.B * p.Hq};
  return D == 128 ? launch_corope_bwd_d<128>(p, ws, fr, stream) : launch_corope_bwd_d<64>(p, ws, fr, stream);
}

}  // namespace corope
