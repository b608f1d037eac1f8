// Fused half-layout-RoPE flash-attention forward for gfx950, software-pipelined variant for a K that
// rope_rotate_kernel rotated beforehand.
//
// Device counterpart of the reference's _attn_fwd / _attn_fwd_inner
// (fused-rope/fused_rope_attn.py:222-320, :48-138); the work split and the MFMA operand layouts are those of
// rope_attn_fwd.hip (one workgroup = 256 query rows, 8 waves x 32 rows, S^T = K_r Q_r^T, O^T += V^T P^T).
//
// What differs is the order in which a wave issues its work.  Two waves share a SIMD, and they keep the matrix pipe
// busy only if each of them offers it an MFMA every few VALU instructions; a stretch of pure softmax arithmetic in
// both waves leaves the pipe idle, and a stretch of pure MFMAs leaves the VALU idle.  The softmax of a 64-key tile
// (32 exponentials per lane) is therefore spread evenly over the tile's 32 MFMAs by running it half a tile behind
// the MFMAs that produced its scores:
//
//     slot 1:  S0(t)     = K(t)[ 0:32] Q^T      |  softmax of S1(t-1), second half   -> P1(t-1)
//     slot 2:  O^T      += V(t-1)[32:64]^T P1(t-1)  |  softmax of S0(t), first half
//     slot 3:  S1(t)     = K(t)[32:64] Q^T      |  softmax of S0(t), second half     -> P0(t)
//     slot 4:  O^T      += V(t)[ 0:32]^T P0(t)  |  softmax of S1(t), first half
//
// so every slot is D/16 MFMAs with four exponential pairs between them, and V(t-1) is still needed while tile t is
// consumed (three V buffers in LDS, two K buffers; one barrier per tile).
//
// Softmax bookkeeping.  Probabilities are formed against a per-row reference m_ref that is not the running maximum:
// p = exp2((s - m_ref) * c).  Any finite reference gives the same normalised result, so it only has to stay close
// enough to the true maximum for p to remain a comfortable fp32 / bf16 number.  The rotation pass left the largest
// key norm of every tile; with the largest query norm of the wave that bounds every score of the tile
// (Cauchy-Schwarz), so whether a tile could exceed the reference by more than kLazyMargin is one scalar comparison,
// made before the tile is touched.  Only then (and on the first tile) the pipeline is drained, the tile's scores are
// computed once just for their row maxima, the reference moves there and the accumulators are rescaled; the tile is
// then processed like any other.  Inside a tile there is no data-dependent branch.
#include "common.hpp"
#include "kernels.hpp"

#include <type_traits>
#include <utility>

namespace COROPE_NS {

constexpr int kPipeBlockN = 64;
// p stays below 2^kPipeMargin and the fp32 sums below 2^(kPipeMargin + log2 N + log2 max|v|): far from overflow, and
// bf16 has fp32's exponent range, so P loses nothing either.  The reference is lifted at most kPipeLift above the largest
// score seen: the row's largest probability stays above 2^-80 and everything within 2^-46 of it above the smallest normal
// fp32 / bf16 number.  Together the two leave 144 binary orders between the Cauchy-Schwarz bound of a tile and the
// scores actually seen before a tile has to be examined a second time (unit-variance inputs at sm_scale = 0.5 need ~110).
constexpr float kPipeMargin = 64.f;
constexpr float kPipeLift = 80.f;

template <int D, int NW>
struct FwdPipeCfg {
  static constexpr int kThreads = NW * kWave;
  static constexpr int kBlockM = NW * 32;
  static constexpr int kVPad = 32;                                        // V is read only through load_a_trans
  static constexpr int kKBytes = RowTile<D>::bytes(kPipeBlockN);          // K tile, row-major, read row-wise
  static constexpr int kVBytes = RowTile<D, kVPad>::bytes(kPipeBlockN);   // V tile, row-major, read transposed
  static constexpr int kKStages = 2, kVStages = 3;
  static constexpr int kLoopBytes = kKStages * kKBytes + kVStages * kVBytes;
  static constexpr int kEpilogueBytes = NW * 32 * kAccTileStride<D> * 4;   // fp32 O rows of all waves
  static constexpr int kLdsBytes = kLoopBytes > kEpilogueBytes ? kLoopBytes : kEpilogueBytes;
};

// One exponential pair of a 32-key half: scores 2j, 2j+1 of the lane -> one bf16x2 word of the P^T operand.
__device__ __forceinline__ void softmax_pair(int j, const f32x16& sacc, u32x4 (&pb)[2], float& lsum) {
  asm volatile("" : "+v"(lsum));  // the pair starts here, not wherever the optimiser would like to hoist it
  float p0 = fast_exp2(sacc[2 * j]);
  float p1 = fast_exp2(sacc[2 * j + 1]);
  // plain adds: the bf16 dot-product instruction would do this in one op but stalls the MFMA pipe
  lsum += p0 + p1;
  uint32_t w = pack_elts(p0, p1);
  asm volatile("" : "+v"(w), "+v"(lsum));   // ... and ends here, between the two MFMAs it is written between
  pb[j / 4][j % 4] = w;
}

__device__ __forceinline__ float wave_reduce_max(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = fmaxf(x, __shfl_xor(x, m));
  return x;
}

template <int D, bool CAUSAL, int NW>
__global__ __launch_bounds__(NW* kWave) __attribute__((amdgpu_waves_per_eu(2, 2))) void rope_attn_fwd_pipe_kernel(FwdParams p) {
  using Cfg = FwdPipeCfg<D, NW>;
  constexpr int BLOCK_N = kPipeBlockN;
  constexpr int NT = Cfg::kThreads;
  constexpr int M = D / 16;         // MFMAs per slot: contraction chunks of a S^T half = MFMAs of a PV half
  constexpr int NDB = D / 32;       // 32-column blocks of O
  constexpr int RING = 4;           // LDS operands in flight
  constexpr int LSV = RowTile<D, Cfg::kVPad>::kStride;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  // Heaviest query blocks first; consecutive workgroup ids walk over (batch, head) so that all blocks of one
  // head land on the same XCD (ids are dealt round-robin to the 8 XCDs) and share its L2.
  const int bh = blockIdx.x % p.BH;
  const int mb = p.num_m_blocks - 1 - blockIdx.x / p.BH;
  const int m0 = mb * Cfg::kBlockM;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lq = lane % 32, lh = lane / 32;
  const int N = p.N;
  [[maybe_unused]] constexpr int TT = NT - kWave;   // stamping thread: first lane of the last wave (it sees every tile)
  COROPE_STAMP(0, TT);

  const uint16_t* qg = p.q + (int64_t)bh * N * D;
  const int kvs = kv_slab(bh, p.H, p.Hkv);   // key/value slab of this query head
  const uint16_t* kg = p.k_rot + (int64_t)kvs * N * D;
  const uint16_t* vg = p.v + (int64_t)kvs * N * D;

  const int n_k_tiles = (N + BLOCK_N - 1) / BLOCK_N;
  const int n_tiles = CAUSAL ? min((m0 + Cfg::kBlockM + BLOCK_N - 1) / BLOCK_N, n_k_tiles) : n_k_tiles;

  CopyStage<D, BLOCK_N, NT, 8> kst;
  CopyStage<D, BLOCK_N, NT, Cfg::kVPad> vst;
  kst.load(kg, 0, N);
  vst.load(vg, 0, N);
  // Lane i: largest rotated-key norm of tile i (the first 64 tiles; requested here so that it lands under the Q rows)
  const uint32_t* tile_kmax_bits = reinterpret_cast<const uint32_t*>(p.tile_kmax) + (int64_t)kvs * n_k_tiles;
  uint32_t kvec = tile_kmax_bits[min(lane, n_k_tiles - 1)];

  // ---- Q rows of this wave: load, rotate, keep as the B operand (through a wave-private LDS tile: the global loads and
  // the copy of the rotated rows kept for the backward then touch whole row segments) ----------------------------------
  const int q_row = m0 + wave * 32 + lq;           // absolute query index of this lane
  u32x4 qb[M];
  {
    WaveRows<D, true> qrows;
    qrows.load(qg, p.cos, p.sin, p.fstride, m0 + wave * 32, N);
    COROPE_STAMP(8, TT);
#ifdef COROPE_TRACE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    COROPE_STAMP(9, TT);
#endif
    qrows.park(qb, reinterpret_cast<uint16_t*>(smem) + wave * 32 * RowTile<D>::kStride,
               p.q_rot_out != nullptr ? p.q_rot_out + (int64_t)bh * N * D : nullptr, m0 + wave * 32, N, p.qk_scale);
  }
  COROPE_STAMP(10, TT);
  __syncthreads();   // the K and V buffers below overlap the tiles the waves just used
  COROPE_STAMP(11, TT);

  constexpr float scale = 1.f;   // the rotated Q rows carry sm_scale * log2(e): scores come out of the MFMAs in base-2 units
  // Largest |q_r| * scale of the wave's rows (a little generous): times a tile's largest key norm it bounds the
  // tile's scaled scores.
  float q_bound_wave;
  {
    float ss = 0.f;
#pragma unroll
    for (int kc = 0; kc < M; ++kc)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float x0 = elt_lo(qb[kc][w]), x1 = elt_hi(qb[kc][w]);
        ss += x0 * x0 + x1 * x1;
      }
    q_bound_wave = __builtin_sqrtf(wave_reduce_max(half_sum(ss))) * scale * 1.01f;
  }

  f32x16 oacc[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i) oacc[i] = f32x16{0};
  float m_run = -INFINITY;   // reference maximum of the raw scores (this lane's query)
  float m_true = -INFINITY;  // largest raw score seen by the reference moves (at most the row's true running maximum)
  float l_run = 0.f;         // this lane's share of the denominator up to the last move of the reference
  float lsum = 0.f;          // ... and since then
  f32x16 msb = f32x16{0};    // -m_run in every register: the accumulator the score MFMAs start from
  f32x16 s1;                 // scores of the second half of the previous tile (softmax half done)
  u32x4 pb0[2], pb1[2];      // P^T operands of the two halves

  // LDS: K buffers at [0, 2 * kKBytes), V buffers behind them.  The buffers rotate by renaming byte offsets (no
  // modulo in the loop); every LDS address the loop uses is "one per-lane register per buffer and tile + an
  // immediate", which the opaque copies below enforce (left alone, the optimiser folds the buffer offset into each of
  // the ~30 operand addresses separately and keeps them all in registers).
  constexpr int kVBase = Cfg::kKStages * Cfg::kKBytes;
  int koff_cur = 0, koff_next = Cfg::kKBytes;
  int voff_prev = kVBase + 2 * Cfg::kVBytes, voff_cur = kVBase, voff_next = kVBase + Cfg::kVBytes;
  auto rotate_buffers = [&]() __attribute__((always_inline)) {
    int k = koff_cur; koff_cur = koff_next; koff_next = k;
    int v = voff_prev; voff_prev = voff_cur; voff_cur = voff_next; voff_next = v;
  };
  auto lds_at = [&](uint32_t byte_off) { return reinterpret_cast<uint16_t*>(smem + byte_off); };
  // per-lane parts of the operand addresses (bytes): K rows read directly, V through the transposing read
  const uint32_t k_lane_off = RowTile<D>::off(lq, 8 * lh) * 2;
  const uint32_t v_lane_off = a_trans_lane_offset(LSV) * 2;

  // Staging registers hold tile t+1 during iteration t: it is written to its LDS buffers during the iteration and the
  // registers are refilled at once with tile t+2, so a global load has a whole iteration to land.  Row indices
  // are clamped, which makes tiles past the end harmless to load and store.
  kst.store_rows(lds_at(koff_cur));
  vst.store_rows(lds_at(voff_cur));
  // tile 0 has no predecessor: its "previous V" is multiplied by a zero P1, so it only has to be finite
  for (int i = threadIdx.x; i < Cfg::kVBytes / 16; i += NT)
    reinterpret_cast<u32x4*>(smem + voff_prev)[i] = u32x4{0, 0, 0, 0};
  kst.load(kg, BLOCK_N, N);
  vst.load(vg, BLOCK_N, N);
  COROPE_STAMP(12, TT);
  __syncthreads();
  COROPE_STAMP(1, TT);

  const int wave_q_lo = m0 + wave * 32, wave_q_hi = wave_q_lo + 31;
  const int key_limit = CAUSAL ? q_row : N - 1;   // last key this lane's query attends to
  // last tile this wave's rows can see
  const int t_last = __builtin_amdgcn_readfirstlane(CAUSAL ? min(n_tiles - 1, wave_q_hi / BLOCK_N) : n_tiles - 1);

  // Reference value (raw-score units) that puts every tile this wave will see within the margin.
  float lift_target;
  {
    uint32_t kall = lane <= t_last ? kvec : 0u;   // non-negative floats order like their bit patterns
    for (int t0 = kWave; t0 <= t_last; t0 += kWave) {
      const int tt = t0 + lane;
      kall = max(kall, tt <= t_last ? tile_kmax_bits[tt] : 0u);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) kall = max(kall, (uint32_t)__shfl_xor((int)kall, m));
    lift_target = (q_bound_wave * __builtin_bit_cast(float, kall) - kPipeMargin) / scale;
  }

  // Bit patterns of non-negative floats order like the floats: the per-tile test "bound > reference + margin" is
  // kmax_bits > thr_bits with thr = (min over rows of m_run * scale + margin) / q_bound_wave, recomputed when the
  // reference moves.  Lane i of kvec holds the key-norm maximum of tile kvec_base + i.
  uint32_t thr_bits = 0;
  int kvec_base = 0;

  auto stage_next = [&](int t) __attribute__((always_inline)) {
    int ko = koff_next, vo = voff_next;
    asm volatile("" : "+s"(ko), "+s"(vo));
    kst.store_rows(lds_at(ko));
    vst.store_rows(lds_at(vo));
    kst.load(kg, (t + 2) * BLOCK_N, N);
    vst.load(vg, (t + 2) * BLOCK_N, N);
  };
  // v_lane: per-lane address of a V buffer (buffer offset + v_lane_off).  MFMA i of a PV half: block i % NDB, chunk i / NDB
  auto v_operand = [&](uint32_t v_lane, int half, int i) {
    return load_a_trans_at(lds_at(v_lane), LSV, half * 32 + 16 * (i / NDB), (i % NDB) * 32);
  };
  // Takes the second half of the previous tile out of the pipeline: rest of the softmax of its S1, then its PV product.
  auto drain = [&]() __attribute__((always_inline)) {
    uint32_t vp_lane = v_lane_off + voff_prev;
    asm volatile("" : "+v"(vp_lane));
#pragma unroll
    for (int j = 4; j < 8; ++j) softmax_pair(j, s1, pb1, lsum);
#pragma unroll
    for (int i = 0; i < M; ++i) oacc[i % NDB] = mfma32(v_operand(vp_lane, 1, i), pb1[i / NDB], oacc[i % NDB]);
  };

  // (the first 64 key-norm maxima have landed before the loop on every path, for the same reason as in the reload below)
  asm volatile("" ::"v"(kvec));
  COROPE_STAMP(2, TT);
  COROPE_STAMP_ID(TT, n_tiles);
#ifdef COROPE_TRACE
  const uint64_t clk0 = __builtin_readcyclecounter();
  uint64_t exact_passes = 0;   // tiles of this wave that were examined a second time to move the reference
#endif
  // ---- tiles this wave's rows can see ------------------------------------------------------------------------------
  for (int t = 0; t <= t_last; ++t) {
    const int n0 = t * BLOCK_N;
#ifdef COROPE_TRACE
    if (t == 1) COROPE_STAMP(3, TT);
    if (n0 == m0) COROPE_STAMP(4, TT);
#endif
    uint32_t k_lane = k_lane_off + koff_cur, vt = v_lane_off + voff_cur, vprev = v_lane_off + voff_prev;   // K(t), V(t), V(t-1)
    asm volatile("" : "+v"(k_lane), "+v"(vt), "+v"(vprev));
    auto k_operand = [&](int half, int kc) {
      return *reinterpret_cast<const u32x4*>(lds_at(k_lane) + RowTile<D>::off(half * 32, 16 * kc));
    };
    // Register i of a half holds key n0 + 32*half + 8*(i/4) + 4*lh + i%4 (see acc_row).  The lane-dependent part goes
    // into one per-tile value, kept opaque so that the 32 thresholds are compared against immediates here instead of
    // being precomputed outside the loop into 32 registers.
    auto mask_scores = [&](f32x16& sacc, int half) __attribute__((always_inline)) {
      int rel = key_limit - n0 - 4 * lh;
      asm volatile("" : "+v"(rel));
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (half * 32 + 8 * (i / 4) + i % 4 > rel) sacc[i] = -INFINITY;
    };
    const bool need_mask = (CAUSAL && n0 + BLOCK_N - 1 > wave_q_lo) || (!CAUSAL && n0 + BLOCK_N > N);

    // One tile: four slots of M MFMAs, operands fetched RING MFMAs ahead.
    // stream position n -> slot n / M (0: S0, 1: PV1 of the previous tile, 2: S1, 3: PV0), MFMA i = n % M of the slot
    auto run_tile = [&](const bool MASK) __attribute__((always_inline)) {
      auto operand = [&](int n) {
        const int slot = n / M, i = n % M;
        return slot == 0 ? k_operand(0, i) : slot == 1 ? v_operand(vprev, 1, i) : slot == 2 ? k_operand(1, i) : v_operand(vt, 0, i);
      };
      constexpr int TOTAL = 4 * M;
      u32x4 ring[RING];
#pragma unroll
      for (int n = 0; n < RING; ++n) ring[n] = operand(n);
      __builtin_amdgcn_sched_barrier(0);
      f32x16 t0;   // S0(t); S1(t) goes straight into s1, whose previous contents slot 0 has used up by then
      static_for<TOTAL>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int n = decltype(n_c)::value;
        constexpr int slot = n / M, i = n % M;
        // MFMA
        if (slot == 0) t0 = i == 0 ? mfma32_from(ring[n % RING], qb[i], msb) : mfma32(ring[n % RING], qb[i], t0);
        if (slot == 1) oacc[i % NDB] = mfma32(ring[n % RING], pb1[i / NDB], oacc[i % NDB]);
        if (slot == 2) s1 = i == 0 ? mfma32_from(ring[n % RING], qb[i], msb) : mfma32(ring[n % RING], qb[i], s1);
        if (slot == 3) oacc[i % NDB] = mfma32(ring[n % RING], pb0[i / NDB], oacc[i % NDB]);
        if (n + RING < TOTAL) ring[n % RING] = operand(n + RING);
        if (n == 0) stage_next(t);
        // softmax on the side: four exponential pairs per slot
        constexpr int jlo = i * 4 / M, jhi = (i + 1) * 4 / M;
        if (slot == 1 && i == 0 && MASK) mask_scores(t0, 0);
        if (slot == 3 && i == 0 && MASK) mask_scores(s1, 1);
#pragma unroll
        for (int j = jlo; j < jhi; ++j) {
          if (slot == 0) softmax_pair(4 + j, s1, pb1, lsum);   // S1(t-1), second half
          if (slot == 1) softmax_pair(j, t0, pb0, lsum);       // S0(t), first half
          if (slot == 2) softmax_pair(4 + j, t0, pb0, lsum);   // S0(t), second half
          if (slot == 3) softmax_pair(j, s1, pb1, lsum);       // S1(t), first half
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    };

    // ---- does the reference have to move before this tile? ------------------------------------------------------
    if (t - kvec_base == kWave) {
      kvec_base = t;
      kvec = tile_kmax_bits[min(t + lane, n_k_tiles - 1)];
      // waited for here, once in 64 tiles: left to the first use below, the wait would sit on the common path too and
      // there also wait for the next tile's loads, half a tile after they were issued instead of a whole one
      asm volatile("" ::"v"(kvec));
    }
    const uint32_t kmax_bits = __builtin_amdgcn_readlane(kvec, t - kvec_base);
    if (t == 0 || kmax_bits > thr_bits) {
#ifdef COROPE_TRACE
      ++exact_passes;
#endif
      if (t > 0) drain();
      f32x16 r0 = f32x16{0}, r1 = f32x16{0};
#pragma unroll
      for (int kc = 0; kc < M; ++kc) {
        r0 = mfma32(k_operand(0, kc), qb[kc], r0);
        r1 = mfma32(k_operand(1, kc), qb[kc], r1);
      }
      if (need_mask) {
        mask_scores(r0, 0);
        mask_scores(r1, 1);
      }
      float mt = fmaxf(r0[0], r1[0]);
#pragma unroll
      for (int i = 1; i < 16; ++i) mt = fmaxf(fmaxf(mt, r0[i]), r1[i]);
      // Lift the reference towards the largest bound any later tile of this wave can show, so that the test above does
      // not fire again (with the Cauchy-Schwarz bound 2-3x above the scores actually seen, hot logits would otherwise
      // send most tiles through this block).  Never further than kPipeLift above the largest score actually seen in
      // this block so far (m_true, a lower bound of the row's running maximum): the row's largest probability stays
      // above 2^-kPipeLift, far inside fp32 / bf16 range, however often the block runs.
      m_true = fmaxf(m_true, half_max(mt));
      const float m_new = fmaxf(m_run, fmaxf(m_true, fminf(lift_target, m_true + kPipeLift / scale)));
      const float alpha = fast_exp2((m_run - m_new) * scale);   // m_new is finite: every row sees key 0 of tile 0
      l_run = (l_run + lsum) * alpha;
      lsum = 0.f;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
      m_run = m_new;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float x = -m_new;
        asm volatile("" : "+v"(x));   // sixteen values of their own: one value in sixteen places is tied to the first of them
        msb[i] = x;
      }
      const float m_min = -wave_reduce_max(-m_run);
      const float thr = (m_min * scale + kPipeMargin) / q_bound_wave;
      thr_bits = __builtin_amdgcn_readfirstlane(thr > 0.f ? __builtin_bit_cast(uint32_t, thr) : 0u);
      // nothing is pending now: an all-masked S1 and a zero P1 make the pending half of the tile body a no-op
#pragma unroll
      for (int i = 0; i < 16; ++i) s1[i] = -INFINITY;
      pb1[0] = pb1[1] = u32x4{0, 0, 0, 0};
    }
    run_tile(need_mask);
    rotate_buffers();
    __syncthreads();
  }
  drain();
  COROPE_STAMP(5, TT);
#ifdef COROPE_TRACE
  if (p.trace != nullptr && threadIdx.x == TT) {
    p.trace[(int64_t)blockIdx.x * 16 + 7] = __builtin_readcyclecounter() - clk0;
    p.trace[(int64_t)blockIdx.x * 16 + 13] = exact_passes;
  }
#endif
  // ---- tiles entirely above this wave's diagonal: it only stages its share ------------------------------------------
  for (int t = t_last + 1; t < n_tiles; ++t) {
    stage_next(t);
    rotate_buffers();
    __syncthreads();
  }

  // ---- epilogue: normalise, write O (through LDS, whole row segments per store) and the base-2 log-sum-exp ------------
  const float l_tot = half_sum(l_run + lsum);
  const float inv_l = 1.f / l_tot;
  __syncthreads();   // every wave is done with the K and V buffers
  store_rows_via_lds<D, false>(oacc, p.o + (int64_t)bh * N * D, m0 + wave * 32, N, nullptr, nullptr, 0, inv_l,
                               reinterpret_cast<float*>(smem) + wave * 32 * kAccTileStride<D>);
  if (q_row < N && lh == 0) p.lse[(int64_t)bh * N + q_row] = m_run * scale + fast_log2(l_tot);
#ifdef COROPE_TRACE
  __builtin_amdgcn_s_waitcnt(0);
  COROPE_STAMP(6, TT);
#endif
}

// ---- host-side launch -----------------------------------------------------------------------------------------
template <int D, bool CAUSAL, int NW>
static hipError_t launch_pipe_waves(FwdParams p, hipStream_t stream) {
  using Cfg = FwdPipeCfg<D, NW>;
  auto kern = rope_attn_fwd_pipe_kernel<D, CAUSAL, NW>;
  static std::atomic<uint64_t> lds_ok{0};
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes, lds_ok); e != hipSuccess) return e;
  p.num_m_blocks = (p.N + Cfg::kBlockM - 1) / Cfg::kBlockM;
#ifdef COROPE_TRACE
  p.trace = g_trace_buf;
#endif
  dim3 grid(p.num_m_blocks * p.BH);
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, p);
  return hipGetLastError();
}

template <int D, bool CAUSAL>
static hipError_t launch_pipe_cfg(const FwdParams& p, hipStream_t stream) {
  return use_small_tiles(p.N, p.BH) ? launch_pipe_waves<D, CAUSAL, 4>(p, stream) : launch_pipe_waves<D, CAUSAL, 8>(p, stream);
}

hipError_t launch_rope_attn_fwd_prerotated(const FwdParams& p, int D, bool causal, hipStream_t stream) {
  if (D == 128) return causal ? launch_pipe_cfg<128, true>(p, stream) : launch_pipe_cfg<128, false>(p, stream);
  return causal ? launch_pipe_cfg<64, true>(p, stream) : launch_pipe_cfg<64, false>(p, stream);
}

}  // namespace COROPE_NS
