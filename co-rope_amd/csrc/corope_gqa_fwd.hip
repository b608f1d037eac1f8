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
// Three restatements keep the work down.  (1) delta is a suffix sum that starts at the diagonal, so key chunks are
// swept right to left and delta accumulates directly: the reference's extra pass over all keys (:103-135) and the
// cancellation in a[i,i] - a[i,j] disappear (online softmax does not care about chunk order).  (2) The angle is
// shared by the whole group, so the key is rotated once per (i, j, d) - the only place sines and cosines are evaluated.
// (3) With the rotated keys parked in LDS, everything that is a dot product with a key row runs on the matrix cores:
// the leader logits q_leader K^T (bf16 x bf16: exact products), the scores q^h Kt^T (one (G x D) x (D x 64 keys)
// product per chunk, rows beyond G idle), and O^T += V^T P^T.  The rotated keys are rounded to fp16, not bf16, and the
// score product runs in fp16 (the bf16 queries convert exactly): 11 significant bits keep the scores as accurate as the
// bf16 rounding of P afterwards, also at sm_scale = 1 where a bf16 key would cost several percent of a weight.
//
// Mapping: one wave (= one workgroup) per (batch, kv head, query row), longest rows first; lane = key inside a 64-key
// chunk.  Per chunk: the contiguous 64 x D block of K is fetched with whole cache lines per instruction and parked in
// the LDS tile -> logits (16x16x32 MFMA, every lane finds its key's logit in its own registers) -> gate, scan over the lanes,
// delta -> each lane rotates its own key row in place -> scores (32x32x16 MFMA, rows moved back to lane = key with
// v_permlane32_swap) -> online softmax against a wave-uniform
// reference value per head (moved to the running maximum only when a score rises well above it) -> the block of V
// replaces the rotated keys in the tile -> O accumulation (MFMA).  A wave's LDS instructions
// execute in order, so the kernel needs no barriers; global loads for the next step are issued one step ahead.
#include "common.hpp"
#include "kernels.hpp"

namespace COROPE_NS {

struct CoropeFreqs {
  float w[64];  // inverse frequencies divided by 2*pi (revolutions per unit of delta), D/2 entries used
};

template <int D, int G>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(2))) void corope_gqa_fwd_kernel(CoropeParams p,
                                                                                                       CoropeFreqs fr) {
  constexpr int HALF = D / 2, KS = D + 8, WS = kWave + 8, PIECES = D / 8;
  constexpr int NI = 4 * ((G - 1) / 8 + 1);                            // accumulator registers that hold rows < G
  __shared__ __attribute__((aligned(16))) uint16_t tile[kWave * KS];   // [key][d]: K (bf16), then rotated K (fp16), then V (bf16)
  __shared__ __attribute__((aligned(16))) uint16_t ql[D];              // the leader's query row (bf16)
  __shared__ __attribute__((aligned(16))) uint16_t wts[G * WS];        // [head][key] bf16 softmax weights of the chunk
  const int n_groups = p.B * p.Hkv;
  const int grp = blockIdx.x % n_groups;
  const int i = p.N - 1 - blockIdx.x / n_groups;                       // longest rows first
  const int lane = threadIdx.x;
  const int vr = lane % 32, hf = lane / 32;                            // matrix-core identity of this lane
  const int b = grp / p.Hkv, kvh = grp % p.Hkv;
  const int N = p.N;
  const int head0 = b * p.Hq + kvh * G;
  const uint16_t* kbase = p.k + (int64_t)grp * N * D;
  const uint16_t* vbase = p.v + (int64_t)grp * N * D;
  const int n_chunks = i / kWave + 1;
  const float scale2 = p.sm_scale * 1.4426950408889634f;               // scores in the base-2 domain

  // A operand of the score product, constant over the row: lane (vr, hf) holds columns 16 ks + 8 hf .. + 7 of q^vr as fp16
  // for vr < G, zeros otherwise.  The logit product takes the leader's row in the element type from LDS.
  // (This product stays on 32x32x16: with rows m of a 16x16x32 A operand holding head m % 4, which also needs no exchange
  // between lanes, the kernel was 3.7 % slower at G = 4, D = 128 -- unlike the logit product below.)
  u32x4 aop[D / 16];
  {
    const uint16_t* qrow = p.q + ((int64_t)(head0 + (vr < G ? vr : 0)) * N + i) * D + 8 * hf;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + 16 * ks);
      u32x4 h16;
#pragma unroll
      for (int e = 0; e < 4; ++e) h16[e] = pack_f16(elt_lo(raw[e]), elt_hi(raw[e]));
      aop[ks] = vr < G ? h16 : u32x4{0, 0, 0, 0};
    }
    const uint16_t* lrow = p.q + ((int64_t)head0 * N + i) * D;
    for (int d = lane; d < D; d += kWave) ql[d] = lrow[d];
  }

  // one 64 x D block of K or V: consecutive 16-byte pieces per lane, parked as rows of the tile
  u32x4 blk[PIECES];
  // may_run_past_end: only the chunk on the diagonal can; the form without the clamped variant keeps one address per
  // lane (with both forms present the compiler merges them into loads behind sixteen selected 64-bit addresses)
  auto fetch_block = [&](const uint16_t* base, int c, auto may_run_past_end) __attribute__((always_inline)) {
    const uint16_t* block = base + (int64_t)c * kWave * D;   // wave-uniform
    if (!decltype(may_run_past_end)::value || c * kWave + kWave <= N) {
#pragma unroll
      for (int it = 0; it < PIECES; ++it)
        blk[it] = *reinterpret_cast<const u32x4*>(byte_offset(block, 16u * lane + 1024u * it));
    } else {   // the block runs past the last key: clamp the rows (only the chunk on the diagonal can get here)
#pragma unroll
      for (int it = 0; it < PIECES; ++it) {
        const int row = (it * kWave + lane) / PIECES, piece = lane % PIECES;
        blk[it] = *reinterpret_cast<const u32x4*>(base + (int64_t)min(c * kWave + row, N - 1) * D + 8 * piece);
      }
    }
  };
  auto park_block = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int it = 0; it < PIECES; ++it) {
      const int row = (it * kWave + lane) / PIECES, piece = lane % PIECES;
      *reinterpret_cast<u32x4*>(tile + row * KS + 8 * piece) = blk[it];
    }
  };
  // (rows < G of a 64-key product) -> this lane's key: swapping the upper half of the keys-below-32 result with the lower
  // half of the keys-from-32 result puts every key's rows into its own lane
  auto rows_of_key = [&](const f32x16& c0, const f32x16& c1, float (&out)[G]) __attribute__((always_inline)) {
    float lo_rows[NI], hi_rows[NI];   // rows 8 (n / 4) + n % 4 and the same + 4
#pragma unroll
    for (int n = 0; n < NI; ++n) {
      const float x0 = c0[n], x1 = c1[n];   // (a bit_cast applied directly to a vector element reads element 0)
      const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, x0), __builtin_bit_cast(uint32_t, x1),
                                                      false, false);
      lo_rows[n] = __builtin_bit_cast(float, (uint32_t)r[0]);
      hi_rows[n] = __builtin_bit_cast(float, (uint32_t)r[1]);
    }
#pragma unroll
    for (int h = 0; h < G; ++h) out[h] = (h / 4) % 2 ? hi_rows[4 * (h / 8) + h % 4] : lo_rows[4 * (h / 8) + h % 4];
  };
  // Leader logits of the 64 keys (K as parked): a 1 x D by D x 64 product, run as 16x16x32 products with the leader's row in
  // every row of A.  All rows of a result block are then equal, block kb holds keys 16 kb .. 16 kb + 15 in the lanes with
  // that l % 16, so every lane finds its own key's logit in block (lane / 16) of its own registers.
  auto leader_logit = [&]() __attribute__((always_inline)) {
    const int r = lane / 16, c = lane % 16;
    f32x4 acc[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) acc[kb] = f32x4{0, 0, 0, 0};
#pragma unroll
    for (int ks = 0; ks < D / 32; ++ks) {
      const u32x4 a = *reinterpret_cast<const u32x4*>(ql + 32 * ks + 8 * r);   // a broadcast read per 16 lanes
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
        acc[kb] = mfma16(a, *reinterpret_cast<const u32x4*>(tile + (16 * kb + c) * KS + 32 * ks + 8 * r), acc[kb]);
    }
    return r == 0 ? acc[0][0] : r == 1 ? acc[1][0] : r == 2 ? acc[2][0] : acc[3][0];
  };
  // scores of the G heads against the rotated keys (fp16) -> this lane's key: sc[h]
  auto scores_of_key = [&](float (&sc)[G]) __attribute__((always_inline)) {
    f32x16 c0 = f32x16{0}, c1 = f32x16{0};
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      c0 = mfma32_f16(aop[ks], *reinterpret_cast<const u32x4*>(tile + vr * KS + 16 * ks + 8 * hf), c0);
      c1 = mfma32_f16(aop[ks], *reinterpret_cast<const u32x4*>(tile + (32 + vr) * KS + 16 * ks + 8 * hf), c1);
    }
    rows_of_key(c0, c1, sc);
  };

  // O^T += V^T P^T as 16x16x32 products (16 output columns x 16 heads per block, of which G are used: half the matrix-pipe
  // time and half the accumulator registers of the 32x32x16 form).  oacc[db][e]: column 16 db + 4 (lane / 16) + e of head
  // lane % 16's output row (lanes with lane % 16 >= G idle).
  constexpr int NOB = D / 16;
  const int oh = lane % 16, og = lane / 16;
  f32x4 oacc[NOB];
#pragma unroll
  for (int db = 0; db < NOB; ++db) oacc[db] = f32x4{0, 0, 0, 0};
  float m_run[G], l_run[G];   // running maximum (wave-uniform, base-2 domain) and this lane's sum of 2^(s - m)
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m_run[h] = -INFINITY;
    l_run[h] = 0.f;
  }
  float carry = 0.f;          // sum of the gates of the chunks to the right (up to the diagonal)

  // the chunk on the diagonal, the only one that can run past the last key, is fetched here; the loop's own fetches
  // are for chunks inside the sequence
  fetch_block(kbase, n_chunks - 1, std::true_type{});
  park_block();
  fetch_block(vbase, n_chunks - 1, std::true_type{});
#pragma unroll 1
  for (int c = n_chunks - 1; c >= 0; --c) {
    const int j = c * kWave + lane;
    const bool valid = j <= i;
    if (c != n_chunks - 1) {
      park_block();                                  // K of this chunk
      fetch_block(vbase, c, std::false_type{});      // V of this chunk: needed after the scores
    }
    lds_order();                  // (also orders the one-time write of the leader's row before its first read)

    // leader logits (row 0 of the product), gates, delta
    const float lg0 = leader_logit();
    const float z = valid ? 1.f / (1.f + __expf(-lg0 * p.sm_scale)) : 0.f;   // gates beyond the diagonal do not count
    const float zpre = wave_prefix_sum(z), ztot = wave_last(zpre);
    const float delta = carry + (ztot - zpre);   // gates strictly to the right of this key, up to the diagonal
    carry += ztot;

    // each lane rotates its own key row in place: one step of look-ahead in two alternating register sets; the scheduling
    // barriers keep the LDS reads from all moving to the top
    u32x2 wa[2][2];
    wa[0][0] = *reinterpret_cast<const u32x2*>(tile + lane * KS);
    wa[0][1] = *reinterpret_cast<const u32x2*>(tile + lane * KS + HALF);
    static_for<HALF / 4>([&](auto step_c) __attribute__((always_inline)) {
      constexpr int step = decltype(step_c)::value, d0 = step * 4;
      if (d0 + 4 < HALF) {
        wa[(step + 1) % 2][0] = *reinterpret_cast<const u32x2*>(tile + lane * KS + d0 + 4);
        wa[(step + 1) % 2][1] = *reinterpret_cast<const u32x2*>(tile + lane * KS + HALF + d0 + 4);
      }
      const u32x2 w1 = wa[step % 2][0], w2 = wa[step % 2][1];
      float r1v[4], r2v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x = __builtin_amdgcn_fractf(delta * fr.w[d0 + e]);
        const float sn = __builtin_amdgcn_sinf(x), cs = __builtin_amdgcn_cosf(x);
        const float k1 = e % 2 ? elt_hi(w1[e / 2]) : elt_lo(w1[e / 2]);
        const float k2 = e % 2 ? elt_hi(w2[e / 2]) : elt_lo(w2[e / 2]);
        r1v[e] = __builtin_fmaf(cs, k1, sn * k2);
        r2v[e] = __builtin_fmaf(cs, k2, -(sn * k1));
      }
      *reinterpret_cast<u32x2*>(tile + lane * KS + d0) = u32x2{pack_f16(r1v[0], r1v[1]), pack_f16(r1v[2], r1v[3])};
      *reinterpret_cast<u32x2*>(tile + lane * KS + HALF + d0) = u32x2{pack_f16(r2v[0], r2v[1]), pack_f16(r2v[2], r2v[3])};
      __builtin_amdgcn_sched_barrier(0);
    });
    lds_order();

    // scores of every head, online softmax
    float sc[G];
    scores_of_key(sc);
    // The reference value m_run[h] of the exponentials only has to keep them in range, it need not be the running
    // maximum: it moves (to the exact maximum so far, with the usual rescaling) only when some score of the chunk lies
    // more than kLazyMargin above it, which after the first chunks of a row is rare.  The common case then costs one
    // comparison per head instead of a cross-lane maximum.
    constexpr float kLazyMargin = 8.f;   // base-2 units: weights stay below 2^8
    float (&s2)[G] = sc;   // scaled in place
    bool exceeds = false;
#pragma unroll
    for (int h = 0; h < G; ++h) {
      s2[h] = valid ? sc[h] * scale2 : -INFINITY;
      exceeds |= s2[h] > m_run[h] + kLazyMargin;   // m_run starts at -inf: the first chunk always moves it
    }
    if (__builtin_amdgcn_ballot_w64(exceeds) != 0) {   // wave-uniform
      float al = 1.f;          // this lane's head's rescale factor
#pragma unroll
      for (int h = 0; h < G; ++h) {
        const float m_new = fmaxf(m_run[h], wave_max(s2[h]));   // finite: the chunk holds a key <= i
        const float a = fast_exp2(m_run[h] - m_new);
        m_run[h] = m_new;
        l_run[h] *= a;
        al = oh == h ? a : al;
      }
#pragma unroll
      for (int db = 0; db < NOB; ++db)
#pragma unroll
        for (int e = 0; e < 4; ++e) oacc[db][e] *= al;
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float e = fast_exp2(s2[h] - m_run[h]);   // 0 for the keys beyond the diagonal
      l_run[h] += e;
      wts[h * WS + lane] = f_to_elt(e);
    }
    park_block();                          // V replaces the rotated keys
    if (c > 0) fetch_block(kbase, c - 1, std::false_type{});  // K of the next chunk
    lds_order();
#pragma unroll
    for (int ks = 0; ks < kWave / 32; ++ks) {   // 32 keys per product
      u32x4 bop = u32x4{0, 0, 0, 0};
      if (oh < G) bop = *reinterpret_cast<const u32x4*>(wts + oh * WS + 32 * ks + 8 * og);
#pragma unroll
      for (int db = 0; db < NOB; ++db) oacc[db] = mfma16(load_a_trans16(tile, KS, 32 * ks, 16 * db), bop, oacc[db]);
    }
    lds_order();
  }

  float inv_l = 0.f;
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const float l = wave_sum(l_run[h]);
    inv_l = oh == h ? (l > 0.f ? 1.f / l : 0.f) : inv_l;   // same guard as the reference's epilogue (:343-345)
  }
  if (oh < G) {
    uint16_t* op = p.o + ((int64_t)(head0 + oh) * N + i) * D;
#pragma unroll
    for (int db = 0; db < NOB; ++db) {
      const u32x2 w = {pack_elts(oacc[db][0] * inv_l, oacc[db][1] * inv_l), pack_elts(oacc[db][2] * inv_l, oacc[db][3] * inv_l)};
      *reinterpret_cast<u32x2*>(op + db * 16 + 4 * og) = w;
    }
  }
}

template <int D, int G>
static hipError_t launch_corope_cfg(CoropeParams p, const CoropeFreqs& fr, hipStream_t stream) {
  p.num_m_blocks = p.N;   // one query row per workgroup
  hipLaunchKernelGGL((corope_gqa_fwd_kernel<D, G>), dim3(p.N * p.B * p.Hkv), dim3(kWave), 0, stream, p, fr);
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

}  // namespace COROPE_NS
