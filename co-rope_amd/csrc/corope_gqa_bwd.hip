// Co-RoPE grouped-query attention backward for gfx950.
//
// The reference's "fused" Co-RoPE operator falls back to a dense PyTorch backward that materialises (B, Hq, N, N, D/2)
// temporaries (corope-exp/flash_attn_co_rope_gqa_triton.py:459-577; same mathematics as the manual backward of
// corope-exp/corope_attn_gqa_pytorch.py:137-300).  This file computes the same gradients with O(N^2) scalars per head
// in a caller-supplied workspace (packed lower-triangular matrices) and no D-sized temporaries.
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
// Sines and cosines are evaluated in two places only, once per (i, j, d) each: where the key is rotated (scores kernel)
// and where the dS-weighted sum of the group's queries is rotated (dk kernel) - the angle is shared by the group and
// rotation is linear, so one vector is rotated per (i, j), not one per head.  Everything that is a dot product with an
// already rotated or an unrotated row runs on the matrix cores.  Launches, in order:
//   rowdot (x2)  leader logits qL K^T per group and dP = dO V^T per head, fp32 into the workspace (32x32x16 bf16 MFMA,
//                128 rows x 128 keys per workgroup, operands fetched with whole cache lines and parked in LDS)
//   scores       one wave per (group, query row), lane = key:
//                  right to left over 64-key chunks: z, delta by a scan, the rotated keys Kt -> LDS (fp16); on the matrix
//                  cores S = q Kt^T and dS/ddelta = [-w q2, w q1] Kt^T for all heads at once, then - with running softmax
//                  statistics, flash-attention style - the two sums that make dq: sum_j e_j dP_j kt_j and sum_j e_j kt_j;
//                  left to right: P, dS, G and its running sum, W;
//                  writes dq of the heads 1..G-1, the leader's dq without its gate path (fp32, workspace) and the workspace
//                  matrices DELTA, W [group] and P, DS [head] (packed lower triangles)
//   dq_leader    dq_leader = c (partial + W K): a plain product on the matrix cores, 128 rows per workgroup
//   dv           dv^T += dO^T P on the matrix cores, 128 keys per workgroup
//   dk           one workgroup per (group, 128 keys): sum_h dS^h q^h on the matrix cores, then lane = rotation pair x 16
//                keys rotates it per (i, j) and adds the gate path W qL; tiles of DELTA, W, DS staged through LDS
// Rounding: the rotated keys and what multiplies them (queries, the softmax weights e and e dP) are fp16 - the bf16
// queries convert exactly, and 11 significant bits keep scores accurate at sm_scale = 1 too; the products on unrotated
// rows (W K, P dO, the row dots) take bf16 operands; sums, statistics, delta, dS/ddelta and everything stored in the
// workspace are fp32.
#include <algorithm>

#include "common.hpp"
#include "kernels.hpp"

namespace COROPE_NS {

struct CoropeBwdFreqs {
  float turns[64];   // w_d / (2 pi): phase in revolutions per unit of delta (what v_sin_f32 / v_cos_f32 take)
  float rad[64];     // w_d
};

// Row i of a workspace matrix holds the keys j <= i only: rows are packed, each padded to the 64-key chunk it ends in
// (rows 64 c .. 64 c + 63 take 64 (c + 1) floats each), so every row starts on a 256-byte boundary.
__device__ __host__ inline int64_t tri_row_start(int i) {
  const int64_t c = i / 64, r = i % 64;
  return 2048 * c * (c + 1) + 64 * (c + 1) * r;
}

// Workspace layout, in floats; NN = tri_row_start(N) is the size of one packed lower-triangular matrix.
struct CoropeBwdWs {
  float* base;
  int64_t NN;
  int n_groups, n_heads;
  __device__ __host__ float* delta(int g) const { return base + (int64_t)g * NN; }
  __device__ __host__ float* w(int g) const { return base + (int64_t)(n_groups + g) * NN; }
  __device__ __host__ float* p(int h) const { return base + (int64_t)(2 * n_groups + h) * NN; }               // S, then P
  __device__ __host__ float* ds(int h) const { return base + (int64_t)(2 * n_groups + n_heads + h) * NN; }    // dS/ddelta, then dS
  __device__ __host__ float* dp(int h) const { return base + (int64_t)(2 * n_groups + 2 * n_heads + h) * NN; }
  // (N, D) per group: the leader head's dq without the gate path and without the factor sm_scale
  __device__ __host__ float* dql(int g, int N, int D) const {
    return base + (int64_t)(2 * n_groups + 3 * n_heads) * NN + (int64_t)g * N * D;
  }
};

// ---------------------------------------------------------------------------------------------------- row dots
// out[idx][i][j] = a[idx * a_mul][i] . b[idx / b_div][j] for the tiles that touch the causal triangle: the two plain
// matrix products of the backward (leader logits qL K^T per group: a_mul = G, b_div = 1; dP = dO V^T per head: a_mul
// = 1, b_div = G) on the matrix cores.  A workgroup of 4 waves owns 128 rows x 128 keys; the rows of both operands are
// fetched with whole cache lines and parked in LDS (an operand piece read straight from global memory is 16 bytes of a
// row per lane: every instruction would touch 64 different lines); one wave owns 32 rows and sweeps the keys in two
// halves of 64, the second half fetched while the first is multiplied.
constexpr int kRowdotRows = 128, kRowdotKeys = 64;

template <int D>
__global__ __launch_bounds__(4 * kWave) void corope_bwd_rowdot_kernel(const uint16_t* a, const uint16_t* b, float* out,
                                                                      int64_t NN, int N, int a_mul, int b_div) {
  constexpr int TS = D + 8, NT = 4 * kWave, PIECES = D / 8;
  constexpr int A_PER = kRowdotRows * PIECES / NT, B_PER = kRowdotKeys * PIECES / NT;
  __shared__ __attribute__((aligned(16))) uint16_t atile[kRowdotRows * TS];
  __shared__ __attribute__((aligned(16))) uint16_t btile[kRowdotKeys * TS];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r = lane % 32, hf = lane / 32;
  const int idx = blockIdx.z;
  const int ib = blockIdx.y * kRowdotRows, j0 = blockIdx.x * 128;
  if (j0 > ib + kRowdotRows - 1 || ib >= N) return;   // every key of the block lies beyond its rows (workgroup-uniform)
  const int i0 = ib + wave * 32;
  const uint16_t* arows = a + (int64_t)idx * a_mul * N * D;
  const uint16_t* brows = b + (int64_t)(idx / b_div) * N * D;
  u32x4 breg[B_PER];
  auto fetch_b = [&](int jh) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < B_PER; ++u) {
      const int e = threadIdx.x + u * NT;
      breg[u] = *reinterpret_cast<const u32x4*>(brows + (int64_t)min(jh + e / PIECES, N - 1) * D + 8 * (e % PIECES));
    }
  };
  auto park_b = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < B_PER; ++u) {
      const int e = threadIdx.x + u * NT;
      *reinterpret_cast<u32x4*>(btile + (e / PIECES) * TS + 8 * (e % PIECES)) = breg[u];
    }
  };
  fetch_b(j0);
#pragma unroll
  for (int u = 0; u < A_PER; ++u) {
    const int e = threadIdx.x + u * NT;
    *reinterpret_cast<u32x4*>(atile + (e / PIECES) * TS + 8 * (e % PIECES)) =
        *reinterpret_cast<const u32x4*>(arows + (int64_t)min(ib + e / PIECES, N - 1) * D + 8 * (e % PIECES));
  }
  park_b();
  __syncthreads();
  u32x4 af[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) af[ks] = *reinterpret_cast<const u32x4*>(atile + (wave * 32 + r) * TS + 16 * ks + 8 * hf);
  float* obase = out + (int64_t)idx * NN;
  // the 32 rows of the wave lie in one 64-row band, so they share a row length; a column <= i0 + 31 is inside the padded row
  const int64_t row0 = tri_row_start(min(i0, N - 1)), row_len = 64 * (i0 / 64 + 1);
#pragma unroll 1
  for (int half = 0; half < 2; ++half) {
    const int jh = j0 + kRowdotKeys * half;
    const bool more = half == 0 && jh + kRowdotKeys <= ib + kRowdotRows - 1 && jh + kRowdotKeys < N;   // workgroup-uniform
    if (more) fetch_b(jh + kRowdotKeys);
#pragma unroll
    for (int jt = 0; jt < kRowdotKeys / 32; ++jt) {
      const int jj0 = jh + 32 * jt;
      if (jj0 > i0 + 31 || jj0 >= N || i0 >= N) continue;   // wave-uniform
      f32x16 c = f32x16{0};
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks)
        c = mfma32(af[ks], *reinterpret_cast<const u32x4*>(btile + (32 * jt + r) * TS + 16 * ks + 8 * hf), c);
      const int col = jj0 + r;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int dr = acc_row(e, hf);
        if (i0 + dr < N && col < N) obase[row0 + row_len * dr + col] = c[e];
      }
    }
    if (!more) break;
    __syncthreads();   // every wave is done with the first half of the keys
    park_b();
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------------------- scores
// One wave per (group, query row i), all G heads at once, lane = key.  Per 64-key chunk the lanes rotate their keys
// (the only place sines and cosines are evaluated) and park them in LDS as fp16; everything that is a dot product with
// the rotated key then runs on the matrix cores: the raw scores q^h . kt and their derivatives with respect to delta
// (rows [-w q2, w q1] . kt) as one (2G x D) x (D x 64 keys) product, and the dq sums as (weights x keys) x (keys x D).
template <int D, int G>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(2, 2))) void corope_bwd_scores_kernel(CoropeBwdParams p, CoropeBwdWs ws, CoropeBwdFreqs fr) {
  constexpr int HALF = D / 2;
  constexpr int KS = D + 8, WS = kWave + 8, NVR = 2 * G, NDB = D / 32;
  constexpr int NI = 4 * ((2 * G - 1) / 8 + 1);                       // accumulator registers that hold rows < 2G
  __shared__ __attribute__((aligned(16))) uint16_t kt[kWave * KS];    // [key][d]: keys (bf16), rotated in place (fp16)
  __shared__ __attribute__((aligned(16))) uint16_t wts[NVR * WS];     // [virtual row][key] fp16 weights of the keys
  const int i = p.N - 1 - blockIdx.x, g = blockIdx.y, lane = threadIdx.x;   // longest rows first
  const int vr = lane % 32, hf = lane / 32;                                  // matrix-core identity of this lane
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv;
  const int head0 = b * p.Hq + kvh * G;   // first head of the group, as a (batch, head) slab index
  // A operand of the score products, constant over the row: lane (vr, hf) holds columns 16 ks + 8 hf .. + 7 of matrix row vr;
  // rows h < G are q^h, rows G + h are [-w q2^h, w q1^h] (the derivative with respect to delta), the rest zero
  u32x4 aop[D / 16];
  {
    const int h = vr < G ? vr : vr - G;
    const uint16_t* qrow = p.q + ((int64_t)(head0 + (vr < 2 * G ? h : 0)) * N + i) * D;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      const int d0 = 16 * ks + 8 * hf;                      // first of this lane's 8 columns
      u32x4 val = u32x4{0, 0, 0, 0};
      if (vr < G) {
        const u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + d0);
#pragma unroll
        for (int e = 0; e < 4; ++e) val[e] = pack_f16(elt_lo(raw[e]), elt_hi(raw[e]));   // exact
      } else if (vr < 2 * G) {
        const bool upper = d0 >= HALF;                       // columns of the second half take w q1, the first half -w q2
        const u32x4 src = *reinterpret_cast<const u32x4*>(qrow + (upper ? d0 - HALF : d0 + HALF));
        const float* wr = fr.rad + (upper ? d0 - HALF : d0);
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float qv = e % 2 ? elt_hi(src[e / 2]) : elt_lo(src[e / 2]);
          x[e] = upper ? wr[e] * qv : -wr[e] * qv;
        }
        val = u32x4{pack_f16(x[0], x[1]), pack_f16(x[2], x[3]), pack_f16(x[4], x[5]), pack_f16(x[6], x[7])};
      }
      aop[ks] = val;
    }
  }
  const uint16_t* kbase = p.k + (int64_t)g * N * D;
  const int64_t rowoff = tri_row_start(i);
  const int n_chunks = i / kWave + 1;
  // this row of every workspace matrix: wave-uniform bases, addressed with 32-bit byte offsets of the key index
  float* const d_row = ws.delta(g) + rowoff;
  float* const w_row = ws.w(g) + rowoff;
  float *p_row[G], *ds_row[G];
  const float* dp_row[G];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    p_row[h] = ws.p(head0 + h) + rowoff;
    ds_row[h] = ws.ds(head0 + h) + rowoff;
    dp_row[h] = ws.dp(head0 + h) + rowoff;
  }

  // ---- right to left: gates, delta, raw scores, dS/ddelta, softmax statistics, dq sums --------------------------------
  // dq^h = c sum_j dS_j kt_j = c (sum_j e_j dP_j kt_j - Delta sum_j e_j kt_j) / L with e_j = exp(s_j - m): both sums are
  // accumulated on the matrix cores as rows 2h and 2h + 1 of W (virtual rows x keys) times Kt (keys x d), rescaled
  // flash-attention style when the row's running maximum m moves.  The 2G <= 16 virtual rows are the columns of 16x16x32
  // products (half the matrix-pipe time and accumulator registers of the 32x32x16 form, whose other 16 columns would be
  // idle): dqa[db][e] belongs to virtual row `qv` = lane % 16 and column 16 db + 4 (lane / 16) + e.
  constexpr int NQB = D / 16;
  const int qv = lane % 16, qg = lane / 16;
  f32x4 dqa[NQB];
#pragma unroll
  for (int db = 0; db < NQB; ++db) dqa[db] = f32x4{0, 0, 0, 0};
  float m_run[G], l_run[G], pd_run[G];   // running maximum (wave-uniform); per lane: sum of exp(s - m), of exp(s - m) dP
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m_run[h] = -INFINITY;
    l_run[h] = pd_run[h] = 0.f;
  }
  float carry = 0.f;   // sum of z over the keys to the right of the current chunk (up to the diagonal)
  // Reference value for Delta = rowsum(P o dP), which is only known at the end of the row: the dq sums take e (dP - ref)
  // as weights and are corrected by (Delta - ref) afterwards, which is exact for any ref; the closer ref is to Delta, the
  // less the two sums cancel (rows dominated by one key would otherwise lose the 11 bits of the weights).  With the forward
  // output at hand ref = rowsum(O o dO), equal to Delta up to O's rounding; without it ref = 0.
  // The weights e (dP - ref) go to the matrix cores as fp16, whose 5 exponent bits would tie the result to the scale of
  // dO (overflow from |dP - ref| ~ 1e3 on, nothing left of a mean-reduced loss's 1e-7): they are divided by a power of two
  // w_scale >= 4 |dO_i| first (|dP_ij| <= |dO_i| |v_j|, so the scaled weights are at most e^4 |v_j| / 4 whatever dO is)
  // and the sum is multiplied back afterwards -- exact both ways.
  float dref[G];
  int w_exp[G];   // w_scale = 2^w_exp, wave-uniform (scalar registers)
#pragma unroll
  for (int h = 0; h < G; ++h) {
    float acc = 0.f, sq = 0.f;
    const int64_t off = ((int64_t)(head0 + h) * N + i) * D;
    for (int d = lane; d < D; d += kWave) {
      const float g_d = elt_to_f(p.d_o[off + d]);
      sq = __builtin_fmaf(g_d, g_d, sq);
      if (p.o != nullptr) acc = __builtin_fmaf(elt_to_f(p.o[off + d]), g_d, acc);
    }
    dref[h] = wave_sum(acc);
    int ex = 0;
    (void)frexpf(__builtin_sqrtf(wave_sum(sq)), &ex);       // |dO_i| = m 2^ex with m in [0.5, 1); 0 gives ex = 0
    w_exp[h] = __builtin_amdgcn_readfirstlane(max(-100, min(100, ex + 2)));
  }
  // A chunk's 64 key rows are one contiguous block of global memory: the wave fetches it with consecutive 16-byte pieces
  // per lane (full cache lines per instruction) and parks it in the LDS tile, where each lane then finds its own key's
  // row.  The block, the leader logits (from the row-dot pass; their slot then takes delta) and dP are each requested
  // for the next chunk at the point where the current values have been used up.
  constexpr int PIECES = D / 8;   // 16-byte pieces per row = fetch instructions per chunk
  u32x4 kv[PIECES];
  // may_run_past_end: only the chunk on the diagonal can; the form without the clamped variant keeps one address per
  // lane (with both forms present the compiler merges them into loads behind sixteen selected 64-bit addresses)
  auto fetch_keys = [&](int c, auto may_run_past_end) __attribute__((always_inline)) {
    const uint16_t* block = kbase + (int64_t)c * kWave * D;   // wave-uniform
    if (!decltype(may_run_past_end)::value || c * kWave + kWave <= N) {
#pragma unroll
      for (int it = 0; it < PIECES; ++it)
        kv[it] = *reinterpret_cast<const u32x4*>(byte_offset(block, 16u * lane + 1024u * it));
    } else {   // the block runs past the last key: clamp the rows (only the chunk on the diagonal can get here)
#pragma unroll
      for (int it = 0; it < PIECES; ++it) {
        const int row = (it * kWave + lane) / PIECES, piece = lane % PIECES;
        kv[it] = *reinterpret_cast<const u32x4*>(kbase + (int64_t)min(c * kWave + row, N - 1) * D + 8 * piece);
      }
    }
  };
  auto park_keys = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int it = 0; it < PIECES; ++it) {
      const int row = (it * kWave + lane) / PIECES, piece = lane % PIECES;
      *reinterpret_cast<u32x4*>(kt + row * KS + 8 * piece) = kv[it];
    }
  };
  float logit, dpv[G];
  {
    const int jc = min((n_chunks - 1) * kWave + lane, i);
    fetch_keys(n_chunks - 1, std::true_type{});
    logit = *byte_offset(d_row, 4u * jc);
#pragma unroll
    for (int h = 0; h < G; ++h) dpv[h] = *byte_offset(dp_row[h], 4u * jc);
  }
#pragma unroll 1
  for (int c = n_chunks - 1; c >= 0; --c) {
    const int j = c * kWave + lane;
    const bool valid = j <= i;
    park_keys();
    const float z = valid ? 1.f / (1.f + __expf(-logit * p.sm_scale)) : 0.f;
    const int jn = j - kWave;   // this lane's key in the next chunk: at or below the diagonal whenever that chunk exists
    if (c > 0) logit = *byte_offset(d_row, 4u * jn);
    const float zpre = wave_prefix_sum(z), ztot = wave_last(zpre);
    const float delta = carry + (ztot - zpre);   // gates strictly to the right, up to and including the diagonal
    carry += ztot;

    // the key rotated by -delta w_d replaces the key in LDS (bf16, row = this lane's key)
    lds_order();
    // one step of look-ahead in two alternating register sets; the scheduling barriers keep the reads from all moving up
    u32x2 wa[2][2];
    wa[0][0] = *reinterpret_cast<const u32x2*>(kt + lane * KS);
    wa[0][1] = *reinterpret_cast<const u32x2*>(kt + lane * KS + HALF);
    static_for<HALF / 4>([&](auto step_c) __attribute__((always_inline)) {
      constexpr int step = decltype(step_c)::value, d0 = step * 4;
      if (d0 + 4 < HALF) {
        wa[(step + 1) % 2][0] = *reinterpret_cast<const u32x2*>(kt + lane * KS + d0 + 4);
        wa[(step + 1) % 2][1] = *reinterpret_cast<const u32x2*>(kt + lane * KS + HALF + d0 + 4);
      }
      const u32x2 w1 = wa[step % 2][0], w2 = wa[step % 2][1];
      float r1v[4], r2v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x = __builtin_amdgcn_fractf(delta * fr.turns[d0 + e]);
        const float sn = __builtin_amdgcn_sinf(x), cs = __builtin_amdgcn_cosf(x);
        const float k1 = e % 2 ? elt_hi(w1[e / 2]) : elt_lo(w1[e / 2]);
        const float k2 = e % 2 ? elt_hi(w2[e / 2]) : elt_lo(w2[e / 2]);
        r1v[e] = __builtin_fmaf(cs, k1, sn * k2);
        r2v[e] = __builtin_fmaf(cs, k2, -(sn * k1));
      }
      *reinterpret_cast<u32x2*>(kt + lane * KS + d0) = u32x2{pack_f16(r1v[0], r1v[1]), pack_f16(r1v[2], r1v[3])};
      *reinterpret_cast<u32x2*>(kt + lane * KS + HALF + d0) = u32x2{pack_f16(r2v[0], r2v[1]), pack_f16(r2v[2], r2v[3])};
      __builtin_amdgcn_sched_barrier(0);
    });
    lds_order();   // rotated keys are in LDS

    // (2G rows x D) x (D x 64 keys): lane = (row vr, half hf) for the A operand, (key vr [+ 32], half hf) for B
    f32x16 c0 = f32x16{0}, c1 = f32x16{0};
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      c0 = mfma32_f16(aop[ks], *reinterpret_cast<const u32x4*>(kt + vr * KS + 16 * ks + 8 * hf), c0);
      c1 = mfma32_f16(aop[ks], *reinterpret_cast<const u32x4*>(kt + (32 + vr) * KS + 16 * ks + 8 * hf), c1);
    }
    // the results sit at lane = key % 32 with rows split over the lane halves; swapping the upper half of the keys-below-
    // 32 result with the lower half of the keys-from-32 result puts every key's rows into its own lane
    float lo_rows[NI], hi_rows[NI];   // rows 8 (n / 4) + n % 4 and the same + 4
#pragma unroll
    for (int n = 0; n < NI; ++n) {
      const float x0 = c0[n], x1 = c1[n];   // (a bit_cast applied directly to a vector element reads element 0)
      const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, x0), __builtin_bit_cast(uint32_t, x1),
                                                      false, false);
      lo_rows[n] = __builtin_bit_cast(float, (uint32_t)r[0]);
      hi_rows[n] = __builtin_bit_cast(float, (uint32_t)r[1]);
    }
    // the registers of the product are free again: request the next chunk's keys (a chunk left of the diagonal one lies
    // inside the sequence)
    if (c > 0) fetch_keys(c - 1, std::false_type{});
    float acc[G], gacc[G];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const int ra = h, rb = G + h;
      acc[h] = (ra / 4) % 2 ? hi_rows[4 * (ra / 8) + ra % 4] : lo_rows[4 * (ra / 8) + ra % 4];
      gacc[h] = (rb / 4) % 2 ? hi_rows[4 * (rb / 8) + rb % 4] : lo_rows[4 * (rb / 8) + rb % 4];
    }
    if (valid) {
      *byte_offset(d_row, 4u * j) = delta;
      *byte_offset(w_row, 4u * j) = z * (1.f - z);   // the sigmoid's slope; replaced by W in the second sweep
    }
    // The reference value m_run[h] of the exponentials only has to keep them in range, it need not be the running
    // maximum (any value gives the same P once the row is normalised): it moves, to the exact maximum so far and with the
    // usual rescaling, only when some score of the chunk lies more than kLazyMargin above it -- rare after the first
    // chunks of a row -- and the common case costs one comparison per head instead of a cross-lane maximum.  The margin
    // bounds the weights e (dP - ref) that go to the matrix cores as fp16.
    constexpr float kLazyMargin = 4.f;
    bool exceeds = false;
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float sc = acc[h] * p.sm_scale;
      if (valid) {
        *byte_offset(p_row[h], 4u * j) = sc;
        *byte_offset(ds_row[h], 4u * j) = gacc[h] * p.sm_scale;
      }
      acc[h] = valid ? sc : -INFINITY;
      exceeds |= acc[h] > m_run[h] + kLazyMargin;   // m_run starts at -inf: the first chunk always moves it
    }
    if (__builtin_amdgcn_ballot_w64(exceeds) != 0) {   // wave-uniform
      float al = 1.f;          // this lane's virtual row's rescale factor
#pragma unroll
      for (int h = 0; h < G; ++h) {
        const float m_new = fmaxf(m_run[h], wave_max(acc[h]));   // finite: the chunk holds a key <= i
        const float a = __expf(m_run[h] - m_new);
        m_run[h] = m_new;
        l_run[h] *= a;
        pd_run[h] *= a;
        al = qv / 2 == h ? a : al;
      }
#pragma unroll
      for (int db = 0; db < NQB; ++db)
#pragma unroll
        for (int e = 0; e < 4; ++e) dqa[db][e] *= al;
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float e = __expf(acc[h] - m_run[h]);   // 0 for the keys beyond the diagonal
      l_run[h] += e;
      pd_run[h] = __builtin_fmaf(e, dpv[h], pd_run[h]);
      // (clamped to fp16's range: a value row |v_j| in the thousands saturates instead of turning into infinity)
      wts[(2 * h) * WS + lane] = f_to_f16(fminf(fmaxf(e * ldexpf(dpv[h] - dref[h], -w_exp[h]), -65504.f), 65504.f));
      wts[(2 * h + 1) * WS + lane] = f_to_f16(e);
    }
    if (c > 0) {
#pragma unroll
      for (int h = 0; h < G; ++h) dpv[h] = *byte_offset(dp_row[h], 4u * jn);
    }
    lds_order();   // rotated keys and weights are in LDS
#pragma unroll
    for (int ks = 0; ks < kWave / 32; ++ks) {   // 32 keys per product
      u32x4 bop = u32x4{0, 0, 0, 0};
      if (qv < 2 * G) bop = *reinterpret_cast<const u32x4*>(wts + qv * WS + 32 * ks + 8 * qg);
#pragma unroll
      for (int db = 0; db < NQB; ++db) dqa[db] = mfma16_f16(load_a_trans16(kt, KS, 32 * ks, 16 * db), bop, dqa[db]);
    }
    lds_order();   // ... and consumed: the next chunk may overwrite them
  }
  // row statistics: largest score, 1 / sum of exponentials, rowsum(P o dP)
  float m_row[G], inv_l[G], dsum[G];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m_row[h] = m_run[h];
    const float l = wave_sum(l_run[h]), pd = wave_sum(pd_run[h]);
    inv_l[h] = 1.f / l;
    dsum[h] = pd * inv_l[h];
  }

  // even virtual row 2h: (sum e (dP - ref) kt - (Delta - ref) sum e kt) / L, the second sum sitting in the neighbouring lane; the rows from
  // 2G on are idle
  {
    float my_inv = 0.f, my_dsum = 0.f;
    int my_exp = 0;
#pragma unroll
    for (int h = 0; h < G; ++h) {
      my_inv = qv / 2 == h ? inv_l[h] : my_inv;
      my_dsum = qv / 2 == h ? dsum[h] - dref[h] : my_dsum;
      my_exp = qv / 2 == h ? w_exp[h] : my_exp;
    }
#pragma unroll
    for (int db = 0; db < NQB; ++db)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float other = __shfl_xor(dqa[db][e], 1);
        if (qv < 2 * G) dqa[db][e] = (ldexpf(dqa[db][e], my_exp) - my_dsum * other) * my_inv;
      }
  }
  // dq of the heads 1..G-1 is final; the leader's still lacks the gate path W K, which a separate plain matrix product
  // adds (corope_bwd_dq_leader_kernel): its row goes to the workspace in fp32, unscaled
  if (qv < 2 * G && qv % 2 == 0) {
    if (qv == 0) {
      float* op = ws.dql(g, N, D) + (int64_t)i * D;
#pragma unroll
      for (int db = 0; db < NQB; ++db) *reinterpret_cast<f32x4*>(op + db * 16 + 4 * qg) = dqa[db];
    } else {
      uint16_t* op = p.dq + ((int64_t)(head0 + qv / 2) * N + i) * D;
#pragma unroll
      for (int db = 0; db < NQB; ++db) {
        const u32x2 w = {pack_elts(dqa[db][0] * p.sm_scale, dqa[db][1] * p.sm_scale),
                         pack_elts(dqa[db][2] * p.sm_scale, dqa[db][3] * p.sm_scale)};
        *reinterpret_cast<u32x2*>(op + db * 16 + 4 * qg) = w;
      }
    }
  }

  // ---- left to right: P, dS, G_ij = sum_h dS dS/ddelta, its running sum over the keys, W ------------------------------
  float gcarry = 0.f;
  // one chunk of look-ahead here too
  float sl_n, sv_n[G], gv_n[G], dp_n[G];
  auto fetch = [&](int c) __attribute__((always_inline)) {
    const int j = c * kWave + lane;
    const int jc = min(j, i);
    sl_n = *byte_offset(w_row, 4u * jc);
#pragma unroll
    for (int h = 0; h < G; ++h) {
      sv_n[h] = *byte_offset(p_row[h], 4u * jc);
      gv_n[h] = *byte_offset(ds_row[h], 4u * jc);
      dp_n[h] = *byte_offset(dp_row[h], 4u * jc);
    }
  };
  fetch(0);
#pragma unroll 1
  for (int c = 0; c < n_chunks; ++c) {
    const int j = c * kWave + lane;
    const bool valid = j <= i;
    // take this chunk's values out of the look-ahead registers and request the next chunk's before anything is stored,
    // so that waiting for them never waits for this chunk's stores
    const float slope = sl_n;
    float sv[G], gv[G], dpc[G];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      sv[h] = sv_n[h];
      gv[h] = gv_n[h];
      dpc[h] = dp_n[h];
    }
    if (c + 1 < n_chunks) fetch(c + 1);
    float gij = 0.f;
    float prv[G], dsv[G];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      prv[h] = __expf(sv[h] - m_row[h]) * inv_l[h];
      dsv[h] = prv[h] * (dpc[h] - dsum[h]);
      gij = __builtin_fmaf(dsv[h], gv[h], gij);
    }
    gij = valid ? gij : 0.f;
    const float pre = wave_prefix_sum(gij);   // over the keys at and to the left of this one
    const float wij = valid ? (gcarry + pre - gij) * slope : 0.f;   // (sum of G over the keys j < t) z'(t)
    gcarry += wave_last(pre);
    if (valid) {
#pragma unroll
      for (int h = 0; h < G; ++h) {
        *byte_offset(p_row[h], 4u * j) = prv[h];
        *byte_offset(ds_row[h], 4u * j) = dsv[h];
      }
      *byte_offset(w_row, 4u * j) = wij;
    }
  }
}

// ---------------------------------------------------------------------------------------------------- leader's dq
// dq_leader_i = c (partial_i + sum_{t <= i} W_it k_t): a plain (rows x keys) x (keys x D) product on the matrix cores,
// computed transposed (dq^T += K^T W^T) so that W is read along its packed rows: lane = query row, 8 consecutive keys per
// step, each value split into two bf16 parts (the keys are exact, so the product carries W to about 16 bits).  One
// workgroup of 4 waves owns 128 rows (32 per wave) of one group; the 16 key rows of a step are staged in LDS and read
// transposed.
template <int D>
__global__ __launch_bounds__(4 * kWave) void corope_bwd_dq_leader_kernel(CoropeBwdParams p, CoropeBwdWs ws) {
  constexpr int TS = D + 16, NDB = D / 32, NT = 4 * kWave, STEP = 16;
  __shared__ __attribute__((aligned(16))) uint16_t tile[STEP * TS];
  const int g = blockIdx.y;
  const int rb = (int)gridDim.x - 1 - (int)blockIdx.x;            // the last row blocks see the most keys: first
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r = lane % 32, hf = lane / 32;
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv, G = p.Hq / p.Hkv;
  const int iw = rb * 128 + 32 * wave, i = iw + r;                // this wave's first row, this lane's row
  const uint16_t* kbase = p.k + (int64_t)g * N * D;
  const float* wrow = ws.w(g) + tri_row_start(min(i, N - 1));
  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) acc[db] = f32x16{0};
  const int t_end = min(N, rb * 128 + 128);                       // keys up to the block's last row
  // the key rows and this lane's W values of a step are fetched into registers one step ahead (the workgroup of the last
  // row block walks N / 16 steps one after the other)
  constexpr int UNITS = STEP * (D / 8), PER = (UNITS + NT - 1) / NT;
  u32x4 kreg[PER];
  f32x4 w0 = f32x4{0.f, 0.f, 0.f, 0.f}, w1 = w0;
  auto fetch = [&](int t0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = min((int)threadIdx.x + u * NT, UNITS - 1);
      kreg[u] = *reinterpret_cast<const u32x4*>(kbase + (int64_t)min(t0 + e / (D / 8), N - 1) * D + 8 * (e % (D / 8)));
    }
    const int t = t0 + 8 * hf;     // first of this lane's 8 keys; t <= i keeps the 32-byte read inside the padded row
    w0 = w1 = f32x4{0.f, 0.f, 0.f, 0.f};
    if (t0 <= iw + 31 && iw < N && i < N && t <= i) {
      w0 = *reinterpret_cast<const f32x4*>(wrow + t);
      w1 = *reinterpret_cast<const f32x4*>(wrow + t + 4);
    }
  };
  if (t_end > 0) fetch(0);
#pragma unroll 1
  for (int t0 = 0; t0 < t_end; t0 += STEP) {
    __syncthreads();   // the previous step's reads of the tile are done
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = threadIdx.x + u * NT;
      if (UNITS % NT == 0 || e < UNITS) *reinterpret_cast<u32x4*>(tile + (e / (D / 8)) * TS + 8 * (e % (D / 8))) = kreg[u];
    }
    const int t = t0 + 8 * hf;
    float hi[8], lo[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      const float wv = (i < N && t + x <= i) ? (x < 4 ? w0[x] : w1[x - 4]) : 0.f;   // nothing beyond the diagonal is defined
      hi[x] = elt_to_f(f_to_elt(wv));
      lo[x] = wv - hi[x];
    }
    const u32x4 bhi = {pack_elts(hi[0], hi[1]), pack_elts(hi[2], hi[3]), pack_elts(hi[4], hi[5]), pack_elts(hi[6], hi[7])};
    const u32x4 blo = {pack_elts(lo[0], lo[1]), pack_elts(lo[2], lo[3]), pack_elts(lo[4], lo[5]), pack_elts(lo[6], lo[7])};
    if (t0 + STEP < t_end) fetch(t0 + STEP);
    __syncthreads();
    if (t0 <= iw + 31 && iw < N) {   // wave-uniform: some row of this wave sees a key of the step
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        const u32x4 a = load_a_trans_natural(tile, TS, 0, 32 * db);
        acc[db] = mfma32(a, bhi, acc[db]);
        acc[db] = mfma32(a, blo, acc[db]);
      }
    }
  }
  if (i < N) {
    const float* part = ws.dql(g, N, D) + (int64_t)i * D;
    uint16_t* op = p.dq + ((int64_t)(b * p.Hq + kvh * G) * N + i) * D;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const f32x4 pv = *reinterpret_cast<const f32x4*>(part + db * 32 + 8 * g4 + 4 * hf);
        const u32x2 w = {pack_elts((acc[db][4 * g4] + pv[0]) * p.sm_scale, (acc[db][4 * g4 + 1] + pv[1]) * p.sm_scale),
                         pack_elts((acc[db][4 * g4 + 2] + pv[2]) * p.sm_scale, (acc[db][4 * g4 + 3] + pv[3]) * p.sm_scale)};
        *reinterpret_cast<u32x2*>(op + db * 32 + 8 * g4 + 4 * hf) = w;
      }
  }
}

// ---------------------------------------------------------------------------------------------------- dv
// dv_j = sum_{h, i} P^h_ij dO^h_i on the matrix cores: dv^T (d x keys) += dO^T (d x rows) P (rows x keys), 16 rows per
// step.  One workgroup of 4 waves owns 128 keys (32 per wave) of one group; the 16 dO rows of every head are staged in
// LDS and read transposed; P comes straight from the workspace (lane = key: 128-byte lines) and is rounded to bf16.
template <int D, int G>
__global__ __launch_bounds__(4 * kWave) void corope_bwd_dv_kernel(CoropeBwdParams p, CoropeBwdWs ws) {
  constexpr int TS = D + 16, NDB = D / 32, NT = 4 * kWave, ROWS = 16;
  constexpr int UNITS = G * ROWS * (D / 8), PER = (UNITS + NT - 1) / NT;   // 16-byte pieces of a dO tile, per thread
  __shared__ __attribute__((aligned(16))) uint16_t tile[G * ROWS * TS];
  const int jb = blockIdx.x * 128, g = blockIdx.y;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r = lane % 32, hf = lane / 32;
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv;
  const int head0 = b * p.Hq + kvh * G;
  const int jw = jb + 32 * wave, j = jw + r;
  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) acc[db] = f32x16{0};

  // Both streams run one step ahead in registers: the workgroup of the first key block walks N / 16 steps one after the
  // other, and with a step's loads issued only when the step begins its time is N / 16 memory latencies.
  u32x4 dreg[PER];
  float pnext[G][8];
  auto fetch = [&](int i0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = min((int)threadIdx.x + u * NT, UNITS - 1);
      const int h = e / (ROWS * (D / 8)), rr = (e / (D / 8)) % ROWS, v8 = e % (D / 8);
      dreg[u] = *reinterpret_cast<const u32x4*>(p.d_o + ((int64_t)(head0 + h) * N + min(i0 + rr, N - 1)) * D + 8 * v8);
    }
    const bool wave_on = i0 + ROWS - 1 >= jw && jw < N;   // wave-uniform: some row of the step sees a key of this wave
    const int64_t row_len = 64 * (i0 / 64 + 1);           // the 16 rows of a step share a row length
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float* prow = ws.p(head0 + h) + tri_row_start(min(i0, N - 1)) + j;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int i = i0 + 8 * hf + t;
        pnext[h][t] = (wave_on && i < N && j <= i) ? prow[row_len * (8 * hf + t)] : 0.f;   // nothing outside the triangle is defined
      }
    }
  };
  if (jb < N) fetch(jb);
#pragma unroll 1
  for (int i0 = jb; i0 < N; i0 += ROWS) {
    __syncthreads();   // the previous step's reads of the tile are done
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = threadIdx.x + u * NT;
      if (UNITS % NT == 0 || e < UNITS)
        *reinterpret_cast<u32x4*>(tile + (e / (D / 8)) * TS + 8 * (e % (D / 8))) = dreg[u];   // rows are (head, row) pairs
    }
    u32x4 bop[G];
#pragma unroll
    for (int h = 0; h < G; ++h)
      bop[h] = u32x4{pack_elts(pnext[h][0], pnext[h][1]), pack_elts(pnext[h][2], pnext[h][3]),
                     pack_elts(pnext[h][4], pnext[h][5]), pack_elts(pnext[h][6], pnext[h][7])};
    const bool wave_on = i0 + ROWS - 1 >= jw && jw < N;
    if (i0 + ROWS < N) fetch(i0 + ROWS);
    __syncthreads();
    if (wave_on) {
#pragma unroll
      for (int h = 0; h < G; ++h)
#pragma unroll
        for (int db = 0; db < NDB; ++db)
          acc[db] = mfma32(load_a_trans_natural(tile + h * ROWS * TS, TS, 0, 32 * db), bop[h], acc[db]);
    }
  }
  if (j < N) {
    uint16_t* op = p.dv + ((int64_t)g * N + j) * D;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const u32x2 w = {pack_elts(acc[db][4 * g4], acc[db][4 * g4 + 1]), pack_elts(acc[db][4 * g4 + 2], acc[db][4 * g4 + 3])};
        *reinterpret_cast<u32x2*>(op + db * 32 + 8 * g4 + 4 * hf) = w;
      }
  }
}

// ---------------------------------------------------------------------------------------------------- dk
// dk_j = c sum_i [ R(+delta_ij)(sum_h dS^h_ij q^h_i) + W_ij qL_i ].  One workgroup of 4 waves owns 128 keys of one group
// (32 per wave) and walks the query rows from the block's first key to the end, 8 rows per staged tile.  Per row:
//   u = sum_h dS^h q^h for the wave's 32 keys and all D columns: a (32 keys x heads) x (heads x D) product on the
//       matrix cores - the contraction is only G long, but it takes 2G multiply-adds per (key, pair) off the vector
//       units; the result lands as lane = column (mod 32), registers = 16 of the wave's keys;
//   rotation and accumulation on the vector units: lane (c, half) owns pairs c and c + 32 (D = 128) for the 16 keys of
//       its half: one (sin, cos) and six multiply-adds per (row, key, pair).
// Work per key block falls linearly with the block index, so a workgroup takes blocks b and (last - b) in turn: every
// workgroup sees the same number of rows.  Tiles of DELTA, W, DS^h ([row][matrix][key], fp32) and the rows' queries
// ([row][column][head], bf16, heads padded to 8 with zeros: the B operand is then one 16-byte read) go through LDS,
// fetched into registers one tile ahead.
constexpr int kDkKeys = 128, kDkRows = 8, kDkWaves = 4;

template <int D, int G>
struct CoropeDkCfg {
  static constexpr int kMats = 2 + G;                                       // DELTA, W, DS^h
  static constexpr int kMatBytes = kDkRows * kMats * kDkKeys * 4;
  static constexpr int kQBytes = kDkRows * D * 8 * 2;                       // [row][column][8 heads] bf16
  static constexpr int kLdsBytes = kMatBytes + kQBytes;
};

template <int D, int G>
__global__ __launch_bounds__(kDkWaves* kWave) __attribute__((amdgpu_waves_per_eu(2))) void corope_bwd_dk_kernel(CoropeBwdParams p, CoropeBwdWs ws,
                                                                       CoropeBwdFreqs fr) {
  using Cfg = CoropeDkCfg<D, G>;
  constexpr int HALF = D / 2, NT = kDkWaves * kWave, MATS = Cfg::kMats, NP = D / 64;
  static_assert(D == 64 || D == 128, "pairs per lane are laid out for these head dims");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float* tile = reinterpret_cast<float*>(smem);                                   // [row][matrix][key]
  uint16_t* qT = reinterpret_cast<uint16_t*>(smem + Cfg::kMatBytes);             // [row][column][8 heads]

  const int g = blockIdx.y;
  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int col = lane % 32, hf = lane / 32;
  const int N = p.N, b = g / p.Hkv, kvh = g % p.Hkv;
  const int head0 = b * p.Hq + kvh * G;
  const int n_blocks = (N + kDkKeys - 1) / kDkKeys;
  float w_turn[NP > 0 ? NP : 1];
#pragma unroll
  for (int np = 0; np < (NP > 0 ? NP : 1); ++np) w_turn[np] = fr.turns[min(32 * np + col, HALF - 1)];

  // heads G..7 of the query tile stay zero for the whole kernel
  for (int e = threadIdx.x; e < Cfg::kQBytes / 16; e += NT) reinterpret_cast<u32x4*>(qT)[e] = u32x4{0, 0, 0, 0};

  constexpr int kTileElems = kDkRows * MATS * kDkKeys, TI = kTileElems / NT;      // fp32 values per thread and tile
  constexpr int kRowItems = kDkRows * G * (D / 8), RI = (kRowItems + NT - 1) / NT;  // 16-byte pieces of q rows
  static_assert(kTileElems % (4 * NT) == 0, "tile elements divide evenly over the threads, four keys at a time");

#pragma unroll 1
  for (int phase = 0; phase < 2; ++phase) {
    const int kb = phase == 0 ? (int)blockIdx.x : n_blocks - 1 - (int)blockIdx.x;
    if (phase == 1 && kb <= (int)blockIdx.x) break;   // odd number of blocks: the middle one has been done in phase 0
    const int jb = kb * kDkKeys, jw = jb + 32 * wave;

    f32x4 mv[TI / 4];
    u32x4 qv[RI];
    auto fetch = [&](int i0) __attribute__((always_inline)) {
      // the 8 rows of a tile share a row length; rows past the end repeat the last one (and are zeroed below)
      const int64_t tile0 = tri_row_start(i0);
      const int row_len = 64 * (i0 / 64 + 1);
      static_for<TI / 4>([&](auto k_c) __attribute__((always_inline)) {
        constexpr int k = decltype(k_c)::value;
        const int e = 4 * (threadIdx.x + k * NT);
        const int key = e % kDkKeys, m = (e / kDkKeys) % MATS, r = e / (kDkKeys * MATS);
        const int i = i0 + r, j = jb + key;
        const float* src = m == 0 ? ws.delta(g) : m == 1 ? ws.w(g) : ws.ds(head0 + m - 2);
        // four keys with one load, always inside the padded row (no branch); what lies outside the causal triangle or
        // past N is not defined there and becomes zero
        const f32x4 v = *reinterpret_cast<const f32x4*>(src + tile0 + (int64_t)row_len * min(r, N - 1 - i0) + min(j, row_len - 4));
#pragma unroll
        for (int x = 0; x < 4; ++x) mv[k][x] = (i < N && j + x <= i) ? v[x] : 0.f;
      });
      static_for<RI>([&](auto k_c) __attribute__((always_inline)) {
        constexpr int k = decltype(k_c)::value;
        const int e = threadIdx.x + k * NT;
        if (kRowItems % NT == 0 || e < kRowItems) {
          const int r = e / (G * (D / 8)), h = (e / (D / 8)) % G, v8 = e % (D / 8);
          qv[k] = *reinterpret_cast<const u32x4*>(p.q + ((int64_t)(head0 + h) * N + min(i0 + r, N - 1)) * D + 8 * v8);
        }
      });
    };
    float dk1[NP][16], dk2[NP][16];
#pragma unroll
    for (int np = 0; np < NP; ++np)
#pragma unroll
      for (int e = 0; e < 16; ++e) dk1[np][e] = dk2[np][e] = 0.f;

    fetch(jb);
#pragma unroll 1
    for (int i0 = jb; i0 < N; i0 += kDkRows) {
      __syncthreads();   // the previous tile has been consumed
      static_for<TI / 4>([&](auto k_c) __attribute__((always_inline)) {
        constexpr int k = decltype(k_c)::value;
        *reinterpret_cast<f32x4*>(tile + 4 * (threadIdx.x + k * NT)) = mv[k];
      });
      static_for<RI>([&](auto k_c) __attribute__((always_inline)) {
        constexpr int k = decltype(k_c)::value;
        const int e = threadIdx.x + k * NT;
        if (kRowItems % NT == 0 || e < kRowItems) {
          const int r = e / (G * (D / 8)), h = (e / (D / 8)) % G, v8 = e % (D / 8);
          uint16_t* dst = qT + ((r * D + 8 * v8) * 8 + h);
#pragma unroll
          for (int x = 0; x < 8; ++x) dst[8 * x] = (uint16_t)(x % 2 ? qv[k][x / 2] >> 16 : qv[k][x / 2] & 0xffffu);
        }
      });
      __syncthreads();
      if (i0 + kDkRows < N) fetch(i0 + kDkRows);
      const int n_rows = min(kDkRows, N - i0);
#pragma unroll 1
      for (int r = 0; r < n_rows; ++r) {
        if (i0 + r < jw) continue;   // wave-uniform: all keys of this wave lie above the diagonal of this row
        const float* trow = tile + r * MATS * kDkKeys + 32 * wave;
        // A: (32 keys x 16 contraction slots): lane (key, half 0) holds dS^h for h = 0..7 rounded to bf16, half 1 what the
        // rounding left over (again as bf16); with the queries of heads 0..7 in both halves of B the product carries dS to
        // about 16 bits
        u32x4 aop;
        {
          float dsv[8];
#pragma unroll
          for (int h = 0; h < 8; ++h) {
            const float x = h < G ? trow[(2 + h) * kDkKeys + col] : 0.f;
            dsv[h] = hf == 0 ? x : x - elt_to_f(f_to_elt(x));
          }
          aop = u32x4{pack_elts(dsv[0], dsv[1]), pack_elts(dsv[2], dsv[3]), pack_elts(dsv[4], dsv[5]), pack_elts(dsv[6], dsv[7])};
        }
        // delta and W of this lane's 16 keys: keys 8 n + 4 half + 0..3 for n = 0..3, as the accumulator rows are laid out
        f32x4 dl[4], wg[4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
          dl[n] = *reinterpret_cast<const f32x4*>(trow + 8 * n + 4 * hf);
          wg[n] = *reinterpret_cast<const f32x4*>(trow + kDkKeys + 8 * n + 4 * hf);
        }
        // B: (heads x 32 columns) per column block; the same read also carries the leader's (head 0) value of the column.
        // One rotation pair per pass (columns 32 np + col and the same + D/2), so that only two product blocks are live.
#pragma unroll
        for (int np = 0; np < NP; ++np) {
          const u32x4 bq1 = *reinterpret_cast<const u32x4*>(qT + (r * D + 32 * np + col) * 8);
          const u32x4 bq2 = *reinterpret_cast<const u32x4*>(qT + (r * D + 32 * (NP + np) + col) * 8);
          const float ql1 = elt_lo(bq1[0]), ql2 = elt_lo(bq2[0]);
          const f32x16 u1 = mfma32(aop, bq1, f32x16{0}), u2 = mfma32(aop, bq2, f32x16{0});
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const float delta = dl[e / 4][e % 4], wij = wg[e / 4][e % 4];
            const float x = __builtin_amdgcn_fractf(delta * w_turn[np]);
            const float sn = __builtin_amdgcn_sinf(x), cs = __builtin_amdgcn_cosf(x);
            dk1[np][e] = __builtin_fmaf(cs, u1[e], __builtin_fmaf(-sn, u2[e], __builtin_fmaf(wij, ql1, dk1[np][e])));
            dk2[np][e] = __builtin_fmaf(cs, u2[e], __builtin_fmaf(sn, u1[e], __builtin_fmaf(wij, ql2, dk2[np][e])));
          }
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int j = jw + acc_row(e, hf);
      if (j < N) {
        uint16_t* op = p.dk + ((int64_t)g * N + j) * D;
#pragma unroll
        for (int np = 0; np < NP; ++np) {
          op[32 * np + col] = f_to_elt(dk1[np][e] * p.sm_scale);
          op[32 * np + col + HALF] = f_to_elt(dk2[np][e] * p.sm_scale);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------- host side
int64_t corope_gqa_bwd_workspace_floats(int B, int Hq, int Hkv, int N, int D) {
  return tri_row_start(N) * (2 * (int64_t)B * Hkv + 3 * (int64_t)B * Hq) + (int64_t)B * Hkv * N * D;
}

template <int D, int G>
static hipError_t launch_corope_bwd_cfg(const CoropeBwdParams& p, const CoropeBwdWs& ws, const CoropeBwdFreqs& fr,
                                        hipStream_t stream) {
  const dim3 rows(p.N, p.B * p.Hkv);
  const int nt = (p.N + 127) / 128;
  hipLaunchKernelGGL(corope_bwd_rowdot_kernel<D>, dim3(nt, nt, p.B * p.Hkv), dim3(4 * kWave), 0, stream, p.q, p.k,
                     ws.delta(0), ws.NN, p.N, G, 1);
  hipLaunchKernelGGL(corope_bwd_rowdot_kernel<D>, dim3(nt, nt, p.B * p.Hq), dim3(4 * kWave), 0, stream, p.d_o, p.v,
                     ws.dp(0), ws.NN, p.N, 1, G);
  hipLaunchKernelGGL((corope_bwd_scores_kernel<D, G>), rows, dim3(kWave), 0, stream, p, ws, fr);
  hipLaunchKernelGGL(corope_bwd_dq_leader_kernel<D>, dim3((p.N + 127) / 128, p.B * p.Hkv), dim3(4 * kWave), 0, stream, p, ws);
  using Cfg = CoropeDkCfg<D, G>;
  hipLaunchKernelGGL((corope_bwd_dv_kernel<D, G>), dim3((p.N + 127) / 128, p.B * p.Hkv), dim3(4 * kWave), 0, stream, p, ws);
  auto kern = corope_bwd_dk_kernel<D, G>;
  static std::atomic<uint64_t> lds_ok{0};
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes, lds_ok); e != hipSuccess) return e;
  const int n_key_blocks = (p.N + kDkKeys - 1) / kDkKeys;
  hipLaunchKernelGGL(kern, dim3((n_key_blocks + 1) / 2, p.B * p.Hkv), dim3(kDkWaves * kWave), Cfg::kLdsBytes, stream, p, ws,
                     fr);
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

// One pass of the launch sequence handles `gc` (batch, key/value head) groups with gc * (2 + 3 G) packed matrices; a
// workspace smaller than the whole problem's is walked in passes of as many groups as fit (every group is independent:
// its queries' heads, its key/value head, its slices of dq, dk, dv).
hipError_t launch_corope_gqa_bwd(const CoropeBwdParams& p, int D, float* workspace, int64_t workspace_floats,
                                 hipStream_t stream) {
  CoropeBwdFreqs fr{};
  // theta^(-2d/D) evaluated like the reference's torch expression (fp32 exponent, fp32 power), as in the forward
  for (int d = 0; d < D / 2; ++d) {
    const float e = (float)(2 * d) / (float)D;
    const float inv = 1.0f / powf(p.theta, e);
    fr.rad[d] = inv;
    fr.turns[d] = (float)((double)inv / 6.283185307179586);
  }
  const int G = p.Hq / p.Hkv, n_groups = p.B * p.Hkv;
  const int64_t per_group = corope_gqa_bwd_workspace_floats(1, G, 1, p.N, D);
  // (a launch spreads the groups' heads over the third grid axis, which ends at 65535)
  const int per_pass = (int)std::min<int64_t>(std::min<int64_t>(n_groups, 65535 / G), workspace_floats / per_group);
  if (per_pass < 1) return hipErrorInvalidValue;
  for (int g0 = 0; g0 < n_groups; g0 += per_pass) {
    const int gc = std::min(per_pass, n_groups - g0);
    CoropeBwdParams c = p;
    const int64_t qoff = (int64_t)g0 * G * p.N * D, koff = (int64_t)g0 * p.N * D;
    c.q += qoff;
    c.d_o += qoff;
    c.dq += qoff;
    if (c.o != nullptr) c.o += qoff;
    c.k += koff;
    c.v += koff;
    c.dk += koff;
    c.dv += koff;
    c.B = 1;
    c.Hkv = gc;
    c.Hq = gc * G;
    CoropeBwdWs ws{workspace, tri_row_start(p.N), gc, gc * G};
    const hipError_t e = D == 128 ? launch_corope_bwd_d<128>(c, ws, fr, stream) : launch_corope_bwd_d<64>(c, ws, fr, stream);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace COROPE_NS
