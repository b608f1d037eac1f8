// Fused half-layout-RoPE flash-attention forward for gfx950 on a K that rope_rotate_kernel rotated beforehand:
// the forms that keep the Q operand and the O accumulators in the accumulation half of the register file and issue
// their score products as asm statements -- 64 query rows per wave, one wave per SIMD, at head dim 128 (first part of the
// file: a measured alternative), and 32 query rows per wave on 32-key tiles (second part: the forward of head dim 256, one
// wave per SIMD; at head dim 128, two workgroups per compute unit, another measured alternative).
//
// Device counterpart of the reference's _attn_fwd / _attn_fwd_inner (fused-rope/fused_rope_attn.py:222-320, :48-138).
// Same mathematics, MFMA operand layouts, softmax bookkeeping (lazy reference value against per-tile key-norm bounds)
// and persistent item walk as rope_attn_fwd_pipe.hip; what differs is who owns which rows.  There a workgroup is 8 waves
// of 32 query rows, two per SIMD, and every K / V^T fragment a wave reads from LDS feeds one MFMA.  Here a workgroup is
// 4 waves, one per SIMD with up to 512 registers, and a wave owns TWO 32-row blocks of the item: every fragment it reads
// feeds two MFMAs (half the LDS reads per MFMA), and the blocks are paired (0,7), (1,6), (2,5), (3,4) inside a wave, so
// on the causal diagonal a wave drops its lower block first and carries on with the upper one alone -- every SIMD then
// has the same number of block-tiles on the diagonal and none of them idles while another finishes.
//
// With one wave per SIMD nothing but the wave's own instruction order overlaps vector work with the matrix pipe, so the
// softmax is cut into half pairs (one exponential, one add, every second time one pack) and one of them follows every
// MFMA:
//
//     slot 1:  S0(t)     = K(t)[ 0:32] Q^T          |  softmax of S1(t-1), second half   -> P1(t-1)
//     slot 2:  O^T      += V(t-1)[32:64]^T P1(t-1)  |  softmax of S0(t), first half
//     slot 3:  S1(t)     = K(t)[32:64] Q^T          |  softmax of S0(t), second half     -> P0(t)
//     slot 4:  O^T      += V(t)[ 0:32]^T P0(t)      |  softmax of S1(t), first half
//
// each slot being D/16 fragments x (MFMA of block A, half pair of A, MFMA of block B, half pair of B).
#include "common.hpp"
#include "kernels.hpp"

#include <type_traits>
#include <utility>

namespace COROPE_NS {

namespace pipe64 {

constexpr int kBlockN = 64;
// As in rope_attn_fwd_pipe.hip: p stays below 2^kMargin; the reference value is lifted at most kLift above the largest
// score seen.
constexpr float kMargin = 64.f;
constexpr float kLift = 80.f;

template <int D>
struct Cfg {
  static constexpr int kWaves = 4;
  static constexpr int kThreads = kWaves * kWave;
  static constexpr int kBlockM = 256;                                     // 4 waves x 2 blocks x 32 rows
  static constexpr int kVPad = 32;                                        // V is read only through load_a_trans
  static constexpr int kKBytes = RowTile<D>::bytes(kBlockN);              // K tile, row-major, read row-wise
  static constexpr int kVBytes = RowTile<D, kVPad>::bytes(kBlockN);       // V tile, row-major, read transposed
  static constexpr int kKStages = 2, kVStages = 3;
  static constexpr int kRingBytes = kKStages * kKBytes + kVStages * kVBytes;
  // behind the ring: two private tiles per wave (one per 32-row block), for Q rows on their way in and O rows on their way out
  static constexpr int kLdsBytes = kRingBytes + 2 * kWaves * WaveTile<D>::kBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS of a compute unit");
};

// Half of an exponential pair of a 32-key half: score 2j + e of the lane (already relative to the reference value, base-2
// units); the second half packs the pair into one word of the P^T operand.
__device__ __forceinline__ void softmax_half(int j, int e, const f32x16& sacc, u32x4 (&pb)[2], float& lsum, float& keep) {
  asm volatile("" : "+v"(lsum));   // the piece starts here, not wherever the optimiser would like to hoist it
  const float pr = fast_exp2(sacc[2 * j + e]);
  lsum += pr;
  if (e == 0) {
    keep = pr;
    asm volatile("" : "+v"(keep), "+v"(lsum));
  } else {
    uint32_t w = pack_elts(keep, pr);
    asm volatile("" : "+v"(w), "+v"(lsum));   // ... and ends here, behind the MFMA it is written behind
    pb[j / 4][j % 4] = w;
  }
}

// A 16-byte operand moved into / out of the accumulation half of the register file, explicitly: values that only ever meet
// "a" constraints afterwards stay there.
__device__ __forceinline__ u32x4 to_acc_half(const u32x4& x) {
  u32x4 y;
  asm volatile("" : "=a"(y) : "0"(x));   // the compiler makes the copy, into four consecutive registers of that half
  return y;
}
__device__ __forceinline__ u32x4 from_acc_half(const u32x4& x) {
  u32x4 y;
  asm volatile("" : "=v"(y) : "0"(x));
  return y;
}

}  // namespace pipe64

template <int D, bool CAUSAL>
__global__ __launch_bounds__(pipe64::Cfg<D>::kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void rope_attn_fwd_pipe64_kernel(FwdParams p) {
  using namespace pipe64;
  using C = Cfg<D>;
  constexpr int BLOCK_N = kBlockN;
  constexpr int NT = C::kThreads;
  constexpr int M = D / 16;         // fragments per slot: contraction chunks of a S^T half = steps of a PV half
  constexpr int NDB = D / 32;       // 32-column blocks of O
  constexpr int RING = 4;           // LDS fragments in flight (2 and 6 measured the same)
  static_assert(M == 8, "the softmax schedule below places 8 half pairs behind 7 of a slot's 8 MFMAs");
  constexpr int LSV = RowTile<D, C::kVPad>::kStride;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lq = lane % 32, lh = lane / 32;
  // the wave's two 32-row blocks of the item: block A = rb[0] (lower rows), block B = rb[1]
  const int rb[2] = {wave, 7 - wave};
  const int N = p.N;
  [[maybe_unused]] constexpr int TT = 0;   // stamping thread: first lane of the wave with the item's last rows
  uint8_t* const wave_tile[2] = {smem + C::kRingBytes + (2 * wave) * WaveTile<D>::kBytes,
                                 smem + C::kRingBytes + (2 * wave + 1) * WaveTile<D>::kBytes};

  // ---- the workgroup's list of items --------------------------------------------------------------------------------
  const ItemList items;
  const int total = p.num_m_blocks * p.BH;
  auto item_at = [&](int r) { return items.at(r); };   // position in the heaviest-first order; >= total: none
  const int n_k_tiles = (N + BLOCK_N - 1) / BLOCK_N;
  auto tiles_of = [&](int mb) {
    return CAUSAL ? min((mb * C::kBlockM + C::kBlockM + BLOCK_N - 1) / BLOCK_N, n_k_tiles) : n_k_tiles;
  };

  // ---- the stream of K/V tiles: a cursor two tiles ahead of the tile being consumed -----------------------------------
  CopyStage<D, BLOCK_N, NT, 8> kst;
  CopyStage<D, BLOCK_N, NT, C::kVPad> vst;
  int l_round = 0, l_tile = 0, l_tiles;
  const uint16_t *l_kg, *l_vg;
  auto load_item = [&](int r) {    // false: no such item
    const int i = item_at(r);
    if (i >= total) return false;
    const int kvs = kv_slab(i % p.BH, p.H, p.Hkv);
    l_kg = p.k_rot + (int64_t)kvs * N * D;
    l_vg = p.v_slab(kvs);
    l_tiles = tiles_of(p.num_m_blocks - 1 - i / p.BH);
    return true;
  };
  auto load_next_tile = [&]() __attribute__((always_inline)) {   // moves the cursor on and requests that tile
    if (l_tile + 1 < l_tiles) {
      ++l_tile;
    } else if (load_item(l_round + 1)) {
      ++l_round;
      l_tile = 0;
    }   // else: past the last tile of the last item; the same tile is requested again and never used
    kst.load(l_kg, l_tile * BLOCK_N, N);
    vst.load(l_vg, l_tile * BLOCK_N, N, (uint32_t)p.v_sn * 2);
  };

  // LDS ring: K buffers at [0, 2 * kKBytes), V buffers behind them; the buffers rotate by renaming byte offsets.
  constexpr int kVBase = C::kKStages * C::kKBytes;
  int koff_cur = 0, koff_next = C::kKBytes;
  int voff_prev = kVBase + 2 * C::kVBytes, voff_cur = kVBase, voff_next = kVBase + C::kVBytes;
  auto rotate_buffers = [&]() __attribute__((always_inline)) {
    int k = koff_cur; koff_cur = koff_next; koff_next = k;
    int v = voff_prev; voff_prev = voff_cur; voff_cur = voff_next; voff_next = v;
    koff_cur = __builtin_amdgcn_readfirstlane(koff_cur); koff_next = __builtin_amdgcn_readfirstlane(koff_next);
    voff_prev = __builtin_amdgcn_readfirstlane(voff_prev); voff_cur = __builtin_amdgcn_readfirstlane(voff_cur);
    voff_next = __builtin_amdgcn_readfirstlane(voff_next);
  };
  auto lds_at = [&](uint32_t byte_off) { return reinterpret_cast<uint16_t*>(smem + byte_off); };
  const uint32_t k_lane_off = RowTile<D>::off(lq, 8 * lh) * 2;
  const uint32_t v_lane_off = a_trans_lane_offset(LSV) * 2;
  auto stage_next = [&]() __attribute__((always_inline)) {
    int ko = koff_next, vo = voff_next;
    asm volatile("" : "+s"(ko), "+s"(vo));
    kst.store_rows(lds_at(ko));
    vst.store_rows(lds_at(vo));
    load_next_tile();
  };

  // ---- Q rows of an item: load, rotate, scale, keep as the B operands; the largest key norms of the item's first 64 tiles
  WaveRows<D, true> qrows[2];
  u32x4 qb[2][M];   // as loaded (vector half of the register file): for the norm bound, then moved over into ...
  u32x4 qa[2][M];   // ... the accumulation half, where the score products read them
  uint32_t kvec;   // lane i: bit pattern of the largest rotated-key norm of tile kvec_base + i
  auto opaque_lane = [&]() __attribute__((always_inline)) {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  auto request_q = [&](int i, auto b_c) __attribute__((always_inline)) {
    constexpr int b = decltype(b_c)::value;
    const int bh = i % p.BH, m0 = (p.num_m_blocks - 1 - i / p.BH) * C::kBlockM;
    qrows[b].load(p.q_slab(bh), p.cos, p.sin, p.fstride, m0 + rb[b] * 32, N, opaque_lane(), (uint32_t)p.q_sn * 2);
  };
  auto request_kvec = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH;
    kvec = reinterpret_cast<const uint32_t*>(p.tile_kmax)[(int64_t)kv_slab(bh, p.H, p.Hkv) * n_k_tiles + min(opaque_lane(), n_k_tiles - 1)];
  };
  auto take_q = [&](int i, auto b_c) __attribute__((always_inline)) {
    constexpr int b = decltype(b_c)::value;
    const int bh = i % p.BH, m0 = (p.num_m_blocks - 1 - i / p.BH) * C::kBlockM;
    park_rotated_rows<D>(qrows[b], qb[b], wave_tile[b], p.q_rot_out != nullptr ? p.q_rot_out + (int64_t)bh * N * D : nullptr,
                         m0 + rb[b] * 32, N, p.qk_scale, opaque_lane());
  };
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;

  // ---- first item: nothing to hide its prologue behind ----------------------------------------------------------------
  int item = item_at(0);
  COROPE_ISTAMP(0);
  load_item(0);
  kst.load(l_kg, 0, N);
  vst.load(l_vg, 0, N, (uint32_t)p.v_sn * 2);
  request_q(item, B0{});
  request_q(item, B1{});
  request_kvec(item);
  take_q(item, B0{});
  take_q(item, B1{});
  kst.store_rows(lds_at(koff_cur));
  vst.store_rows(lds_at(voff_cur));
  load_next_tile();
  __syncthreads();

  for (int round = 0;; ++round) {
    const int bh = item % p.BH, mb = p.num_m_blocks - 1 - item / p.BH;
    const int m0 = mb * C::kBlockM;
    const int n_tiles = tiles_of(mb);
    const uint32_t* tile_kmax_bits = reinterpret_cast<const uint32_t*>(p.tile_kmax) + (int64_t)kv_slab(bh, p.H, p.Hkv) * n_k_tiles;
    COROPE_ISTAMP(1);

    // Largest |q_r| (scaled: base-2 units) of the wave's rows, a little generous: times a tile's largest key norm it
    // bounds the tile's scores.
    float q_bound_wave;
    {
      float ss[2] = {0.f, 0.f};
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int kc = 0; kc < M; ++kc)
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            float x0 = elt_lo(qb[b][kc][w]), x1 = elt_hi(qb[b][kc][w]);
            ss[b] += x0 * x0 + x1 * x1;
          }
      q_bound_wave = __builtin_sqrtf(wave_max(fmaxf(half_sum(ss[0]), half_sum(ss[1])))) * 1.01f;
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int kc = 0; kc < M; ++kc) qa[b][kc] = to_acc_half(qb[b][kc]);
    }

    f32x16 oacc[2][NDB];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < NDB; ++i) oacc[b][i] = f32x16{0};
    float m_run[2] = {-INFINITY, -INFINITY};    // reference value of the exponentials (this lane's queries), base-2 units
    float m_true[2] = {-INFINITY, -INFINITY};   // largest score seen by the reference moves
    float l_run[2] = {0.f, 0.f};                // this lane's share of the denominators up to the last move of the reference
    float lsum[2] = {0.f, 0.f};                 // ... and since then
    float keep[2] = {0.f, 0.f};                 // first probability of the pair in flight
    f32x16 msb[2] = {f32x16{0}, f32x16{0}};     // -m_run in every register: the accumulator the score MFMAs start from
    f32x16 s1[2];                               // scores of the second half of the previous tile (softmax half done)
    f32x16 t0[2];                               // scores of the first half of the tile
    u32x4 pb0[2][2], pb1[2][2];                 // P^T operands of the two halves

    int wave_q_lo[2], key_limit[2], t_last[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      wave_q_lo[b] = m0 + rb[b] * 32;
      key_limit[b] = CAUSAL ? wave_q_lo[b] + lq : N - 1;   // last key this lane's query attends to
      t_last[b] = __builtin_amdgcn_readfirstlane(CAUSAL ? min(n_tiles - 1, (wave_q_lo[b] + 31) / BLOCK_N) : n_tiles - 1);
    }

    // Reference value that puts every tile this wave will see within the margin.
    float lift_target;
    {
      uint32_t kall = lane <= t_last[1] ? kvec : 0u;   // non-negative floats order like their bit patterns
      for (int tb = kWave; tb <= t_last[1]; tb += kWave) {
        const int tt = tb + lane;
        kall = max(kall, tt <= t_last[1] ? tile_kmax_bits[tt] : 0u);
      }
      lift_target = q_bound_wave * wave_max(__builtin_bit_cast(float, kall)) - kMargin;
    }
    uint32_t thr_bits = 0;
    int kvec_base = 0;

    auto v_operand = [&](uint32_t v_lane, int half, int i) {
      return load_a_trans_at(lds_at(v_lane), LSV, half * 32 + 16 * (i / NDB), (i % NDB) * 32);
    };
    // Takes the second half of the previous tile of block b out of the pipeline: rest of the softmax of its S1, then its PV product.
    auto drain = [&](auto b_c) __attribute__((always_inline)) {
      constexpr int b = decltype(b_c)::value;
      uint32_t vp_lane = v_lane_off + voff_prev;
      asm volatile("" : "+v"(vp_lane));
#pragma unroll
      for (int j = 4; j < 8; ++j) {
        softmax_half(j, 0, s1[b], pb1[b], lsum[b], keep[b]);
        softmax_half(j, 1, s1[b], pb1[b], lsum[b], keep[b]);
      }
#pragma unroll
      for (int i = 0; i < M; ++i) oacc[b][i % NDB] = mfma32(v_operand(vp_lane, 1, i), pb1[b][i / NDB], oacc[b][i % NDB]);
    };

#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int kc = 0; kc < M; ++kc) asm volatile("" ::"a"(qa[b][kc]));
    asm volatile("" ::"v"(kvec));
    COROPE_ISTAMP(2);
#ifdef COROPE_TRACE
    COROPE_ISTAMP_ID(n_tiles);
    const uint64_t clk0 = __builtin_readcyclecounter();
    uint64_t exact_passes = 0;
#endif

    // One tile for the blocks FIRST..1 (FIRST = 0: both, FIRST = 1: block B alone).  MASK: the scores of block FIRST (causal:
    // the only block whose diagonal can cross the tile while it is the first active one) or of every active block (not
    // causal: keys past the end of the sequence) are masked.
    auto tile_step = [&](int t, auto first_c, bool need_mask) __attribute__((always_inline)) {
      constexpr int FIRST = decltype(first_c)::value;
      const int n0 = t * BLOCK_N;
#ifdef COROPE_TRACE
      if (t == 1) COROPE_ISTAMP(3);
      if (n0 == m0) COROPE_ISTAMP(4);
#endif
      uint32_t k_lane = k_lane_off + koff_cur, vt = v_lane_off + voff_cur, vprev = v_lane_off + (t == 0 ? voff_cur : voff_prev);
      asm volatile("" : "+v"(k_lane), "+v"(vt), "+v"(vprev));
      auto k_operand = [&](int half, int kc) {
        return *reinterpret_cast<const u32x4*>(lds_at(k_lane) + RowTile<D>::off(half * 32, 16 * kc));
      };
      auto mask_scores = [&](f32x16& sacc, int half, int b) __attribute__((always_inline)) {
        int rel = key_limit[b] - n0 - 4 * lh;
        asm volatile("" : "+v"(rel));
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (half * 32 + 8 * (i / 4) + i % 4 > rel) sacc[i] = -INFINITY;
      };
      auto masked_block = [&](int b) { return CAUSAL ? b == FIRST : true; };

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
        static_for<TOTAL>([&](auto n_c) __attribute__((always_inline)) {
          constexpr int n = decltype(n_c)::value;
          constexpr int slot = n / M, i = n % M;
          static_for<2>([&](auto b_c) __attribute__((always_inline)) {
            constexpr int b = decltype(b_c)::value;
            if constexpr (b >= FIRST) {
              const u32x4 frag = ring[n % RING];
              if (slot == 0) { if (i == 0) t0[b] = mfma32_from_aq(frag, qa[b][i], msb[b]); else mfma32_acc_aq(t0[b], frag, qa[b][i]); }
              if (slot == 1) oacc[b][i % NDB] = mfma32(frag, pb1[b][i / NDB], oacc[b][i % NDB]);
              if (slot == 2) { if (i == 0) s1[b] = mfma32_from_aq(frag, qa[b][i], msb[b]); else mfma32_acc_aq(s1[b], frag, qa[b][i]); }
              if (slot == 3) oacc[b][i % NDB] = mfma32(frag, pb0[b][i / NDB], oacc[b][i % NDB]);
              if (b == 1) {
                if (n + RING < TOTAL) ring[n % RING] = operand(n + RING);
                if (n == 0) stage_next();
              }
              // The slot's eight half pairs follow its MFMAs 1..7 (two behind the last): the scores a slot starts on were
              // completed by the last MFMA of the slot before, an asm statement behind which the compiler inserts no wait
              // states, so nothing reads them behind MFMA 0, which waits a little instead.
              if (i == 0) {
                if (FIRST == 0) asm volatile("s_nop 1"); else asm volatile("s_nop 7");
              }
              if (slot == 1 && i == 1 && MASK && masked_block(b)) mask_scores(t0[b], 0, b);
              if (slot == 3 && i == 1 && MASK && masked_block(b)) mask_scores(s1[b], 1, b);
#pragma unroll
              for (int hh = (i == 0 ? 0 : i - 1); hh < (i == 0 ? 0 : i == M - 1 ? 8 : i); ++hh) {
                const int j = hh / 2, e = hh % 2;
                if (slot == 0) softmax_half(4 + j, e, s1[b], pb1[b], lsum[b], keep[b]);   // S1(t-1), second half
                if (slot == 1) softmax_half(j, e, t0[b], pb0[b], lsum[b], keep[b]);       // S0(t), first half
                if (slot == 2) softmax_half(4 + j, e, t0[b], pb0[b], lsum[b], keep[b]);   // S0(t), second half
                if (slot == 3) softmax_half(j, e, s1[b], pb1[b], lsum[b], keep[b]);       // S1(t), first half
              }
              __builtin_amdgcn_sched_barrier(0);
            }
          });
        });
      };

      // ---- does the reference have to move before this tile? ------------------------------------------------------
      if (t - kvec_base == kWave) {
        kvec_base = t;
        kvec = tile_kmax_bits[min(t + lane, n_k_tiles - 1)];
        asm volatile("" ::"v"(kvec));
      }
      const uint32_t kmax_bits = __builtin_amdgcn_readlane(kvec, t - kvec_base);
      if (t == 0 || kmax_bits > thr_bits) {
#ifdef COROPE_TRACE
        ++exact_passes;
#endif
        static_for<2>([&](auto b_c) __attribute__((always_inline)) {
          constexpr int b = decltype(b_c)::value;
          if constexpr (b >= FIRST) {
            if (t > 0) drain(b_c);
            f32x16 r0 = f32x16{0}, r1 = f32x16{0};
#pragma unroll
            for (int kc = 0; kc < M; ++kc) {
              const u32x4 qv = from_acc_half(qa[b][kc]);
              r0 = mfma32(k_operand(0, kc), qv, r0);
              r1 = mfma32(k_operand(1, kc), qv, r1);
            }
            if (need_mask && masked_block(b)) {
              mask_scores(r0, 0, b);
              mask_scores(r1, 1, b);
            }
            float mt = fmaxf(r0[0], r1[0]);
#pragma unroll
            for (int i = 1; i < 16; ++i) mt = fmaxf(fmaxf(mt, r0[i]), r1[i]);
            m_true[b] = fmaxf(m_true[b], half_max(mt));
            const float m_new = fmaxf(m_run[b], fmaxf(m_true[b], fminf(lift_target, m_true[b] + kLift)));
            const float alpha = fast_exp2(m_run[b] - m_new);   // m_new is finite: every row sees key 0 of tile 0
            l_run[b] = (l_run[b] + lsum[b]) * alpha;
            lsum[b] = 0.f;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
              for (int i = 0; i < 16; ++i) oacc[b][db][i] *= alpha;
            m_run[b] = m_new;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              float x = -m_new;
              asm volatile("" : "+v"(x));   // sixteen values of their own
              msb[b][i] = x;
            }
            // nothing is pending now: an all-masked S1 and a zero P1 make the pending half of the tile body a no-op
#pragma unroll
            for (int i = 0; i < 16; ++i) s1[b][i] = -INFINITY;
            pb1[b][0] = pb1[b][1] = u32x4{0, 0, 0, 0};
          }
        });
        const float m_min = -wave_max(FIRST == 0 ? fmaxf(-m_run[0], -m_run[1]) : -m_run[1]);
        const float thr = (m_min + kMargin) / q_bound_wave;
        thr_bits = __builtin_amdgcn_readfirstlane(thr > 0.f ? __builtin_bit_cast(uint32_t, thr) : 0u);
      }
      run_tile(need_mask);
      rotate_buffers();
      __syncthreads();
    };

    // ---- tiles both blocks see; then block A leaves; then the tiles only block B sees ------------------------------------
    for (int t = 0; t <= t_last[0]; ++t)
      tile_step(t, B0{}, (CAUSAL && t * BLOCK_N + BLOCK_N - 1 > wave_q_lo[0]) || (!CAUSAL && t * BLOCK_N + BLOCK_N > N));
    drain(B0{});
    {
      const float l_tot = half_sum(l_run[0] + lsum[0]);
      store_rows_via_wave_tile<D>(oacc[0], p.o + (int64_t)bh * N * D, wave_q_lo[0], N, 1.f / l_tot, wave_tile[0], opaque_lane());
      if (wave_q_lo[0] + lq < N && lh == 0) p.lse[(int64_t)bh * N + wave_q_lo[0] + lq] = m_run[0] + fast_log2(l_tot);
    }
    for (int t = t_last[0] + 1; t <= t_last[1]; ++t)
      tile_step(t, B1{}, (CAUSAL && t * BLOCK_N + BLOCK_N - 1 > wave_q_lo[1]) || (!CAUSAL && t * BLOCK_N + BLOCK_N > N));

    // The next item's Q rows are requested as soon as the registers of this item's Q rows are free.  (After the last item
    // its own rows are requested once more and never used.)
    const int next_item = item_at(round + 1);
    const bool has_next = next_item < total;
    request_q(has_next ? next_item : item, B0{});
    request_q(has_next ? next_item : item, B1{});
    request_kvec(has_next ? next_item : item);
    drain(B1{});
    COROPE_ISTAMP(5);
#ifdef COROPE_TRACE
    if (p.trace != nullptr && threadIdx.x == TT) {
      p.trace[(int64_t)item * 16 + 7] = __builtin_readcyclecounter() - clk0;
      p.trace[(int64_t)item * 16 + 13] = exact_passes;
    }
#endif
    // of the tiles entirely above this wave's diagonal it only stages its share
    for (int t = t_last[1] + 1; t < n_tiles; ++t) {
      stage_next();
      rotate_buffers();
      __syncthreads();
    }
    {
      const float l_tot = half_sum(l_run[1] + lsum[1]);
      store_rows_via_wave_tile<D>(oacc[1], p.o + (int64_t)bh * N * D, wave_q_lo[1], N, 1.f / l_tot, wave_tile[1], opaque_lane());
      if (wave_q_lo[1] + lq < N && lh == 0) p.lse[(int64_t)bh * N + wave_q_lo[1] + lq] = m_run[1] + fast_log2(l_tot);
    }
    COROPE_ISTAMP(6);
    if (!has_next) break;
    item = next_item;
    COROPE_ISTAMP(0);
    take_q(item, B0{});
    take_q(item, B1{});
  }
}

// ================================================================================ head dim 256
// The same one-wave-per-SIMD form for head dim 256: a workgroup is 4 waves of 32 query rows (128-row items); a wave's Q
// operand (64 registers) and O accumulators (128) live in the accumulation half of its 512 registers.  K and V tiles are 32
// keys, so that a ring of 2 K + 3 V buffers and the waves' private tiles fit the LDS (151 KB), and a tile is what a 32-key
// half is above: with 16 MFMAs per product a wave spends two slots on every tile,
//
//     slot A:  S(t)  = K(t) Q^T              |  softmax of S(t-1), second half   -> P(t-1)
//     slot B:  O^T  += V(t-1)^T P(t-1)       |  softmax of S(t), first half
//
// the eight exponential half pairs of a slot spread over its MFMAs.  At the end of a tile the eight scores per lane that its softmax
// still needs and the finished half of its P^T operand are moved to registers of their own (12 vector moves).
namespace pipe64 {
template <int D_>
struct Cfg32 {
  static constexpr int kD = D_;
  // head dim 256: one wave per SIMD (512 registers each); 128: two, i.e. two workgroups per compute unit
  static constexpr int kWavesPerSimd = D_ > 128 ? 1 : 2;
  static constexpr int kWaves = 4;
  static constexpr int kThreads = kWaves * kWave;
  static constexpr int kBlockM = kWaves * 32;
  static constexpr int kBlockN = 32;
  static constexpr int kVPad = 32;
  static constexpr int kKBytes = RowTile<kD>::bytes(kBlockN);
  static constexpr int kVBytes = RowTile<kD, kVPad>::bytes(kBlockN);
  static constexpr int kKStages = 2, kVStages = 3;
  static constexpr int kRingBytes = kKStages * kKBytes + kVStages * kVBytes;
  static constexpr int kLdsBytes = kRingBytes + kWaves * WaveTile<kD>::kBytes;
  static_assert(kWavesPerSimd * kLdsBytes <= 160 * 1024, "LDS of a compute unit");
};
using Cfg256 = Cfg32<256>;
}  // namespace pipe64

template <int D_, bool CAUSAL>
__global__ __launch_bounds__(pipe64::Cfg32<D_>::kThreads)
    __attribute__((amdgpu_waves_per_eu(pipe64::Cfg32<D_>::kWavesPerSimd, pipe64::Cfg32<D_>::kWavesPerSimd))) void rope_attn_fwd_pipe32_kernel(FwdParams p) {
  using namespace pipe64;
  using C = Cfg32<D_>;
  constexpr int D = C::kD;
  constexpr int BLOCK_N = C::kBlockN;
  constexpr int NT = C::kThreads;
  constexpr int M = D / 16;         // MFMAs per slot: contraction chunks of S^T = (16-key steps) x (32-column blocks) of PV
  constexpr int NDB = D / 32;       // 32-column blocks of O
  constexpr int RING = 4;           // LDS fragments in flight
  constexpr int LSV = RowTile<D, C::kVPad>::kStride;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lq = lane % 32, lh = lane / 32;
  const int N = p.N;
  [[maybe_unused]] constexpr int TT = (C::kWaves - 1) * kWave;   // stamping thread: first lane of the wave with the item's last rows
  uint8_t* const wave_tile = smem + C::kRingBytes + wave * WaveTile<D>::kBytes;

  // ---- the workgroup's list of items --------------------------------------------------------------------------------
  const ItemList items;
  const int total = p.num_m_blocks * p.BH;
  auto item_at = [&](int r) { return items.at(r); };   // position in the heaviest-first order; >= total: none
  const int n_k_tiles = (N + BLOCK_N - 1) / BLOCK_N;
  const int n_norm_tiles = (N + 63) / 64;              // the rotation pass leaves one key-norm maximum per 64 keys
  auto tiles_of = [&](int mb) {
    return CAUSAL ? min((mb * C::kBlockM + C::kBlockM + BLOCK_N - 1) / BLOCK_N, n_k_tiles) : n_k_tiles;
  };

  // ---- the stream of K/V tiles: a cursor two tiles ahead of the tile being consumed -----------------------------------
  CopyStage<D, BLOCK_N, NT, 8> kst;
  CopyStage<D, BLOCK_N, NT, C::kVPad> vst;
  int l_round = 0, l_tile = 0, l_tiles;
  const uint16_t *l_kg, *l_vg;
  auto load_item = [&](int r) {    // false: no such item
    const int i = item_at(r);
    if (i >= total) return false;
    const int kvs = kv_slab(i % p.BH, p.H, p.Hkv);
    l_kg = p.k_rot + (int64_t)kvs * N * D;
    l_vg = p.v_slab(kvs);
    l_tiles = tiles_of(p.num_m_blocks - 1 - i / p.BH);
    return true;
  };
  auto load_next_tile = [&]() __attribute__((always_inline)) {   // moves the cursor on and requests that tile
    if (l_tile + 1 < l_tiles) {
      ++l_tile;
    } else if (load_item(l_round + 1)) {
      ++l_round;
      l_tile = 0;
    }   // else: past the last tile of the last item; the same tile is requested again and never used
    kst.load(l_kg, l_tile * BLOCK_N, N);
    vst.load(l_vg, l_tile * BLOCK_N, N, (uint32_t)p.v_sn * 2);
  };

  // LDS ring: K buffers at [0, 2 * kKBytes), V buffers behind them; the buffers rotate by renaming byte offsets.
  constexpr int kVBase = C::kKStages * C::kKBytes;
  int koff_cur = 0, koff_next = C::kKBytes;
  int voff_prev = kVBase + 2 * C::kVBytes, voff_cur = kVBase, voff_next = kVBase + C::kVBytes;
  auto rotate_buffers = [&]() __attribute__((always_inline)) {
    int k = koff_cur; koff_cur = koff_next; koff_next = k;
    int v = voff_prev; voff_prev = voff_cur; voff_cur = voff_next; voff_next = v;
    koff_cur = __builtin_amdgcn_readfirstlane(koff_cur); koff_next = __builtin_amdgcn_readfirstlane(koff_next);
    voff_prev = __builtin_amdgcn_readfirstlane(voff_prev); voff_cur = __builtin_amdgcn_readfirstlane(voff_cur);
    voff_next = __builtin_amdgcn_readfirstlane(voff_next);
  };
  auto lds_at = [&](uint32_t byte_off) { return reinterpret_cast<uint16_t*>(smem + byte_off); };
  const uint32_t k_lane_off = RowTile<D>::off(lq, 8 * lh) * 2;
  const uint32_t v_lane_off = a_trans_lane_offset(LSV) * 2;
  auto stage_next = [&]() __attribute__((always_inline)) {
    int ko = koff_next, vo = voff_next;
    asm volatile("" : "+s"(ko), "+s"(vo));
    kst.store_rows(lds_at(ko));
    vst.store_rows(lds_at(vo));
    load_next_tile();
  };

  // ---- Q rows of an item: load, rotate, scale, keep as the B operand; the largest key norms of the item's first tiles
  WaveRows<D, true> qrows;
  u32x4 qb[M];   // as loaded (vector half of the register file): for the norm bound, then moved over into ...
  u32x4 qa[M];   // ... the accumulation half, where the score products read them
  uint32_t kvec;   // lane i: bit pattern of the largest rotated-key norm of keys [64 (kvec_base + i), + 64)
  auto opaque_lane = [&]() __attribute__((always_inline)) {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  auto request_q = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH, m0 = (p.num_m_blocks - 1 - i / p.BH) * C::kBlockM;
    qrows.load(p.q_slab(bh), p.cos, p.sin, p.fstride, m0 + wave * 32, N, opaque_lane(), (uint32_t)p.q_sn * 2);
  };
  auto request_kvec = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH;
    kvec = reinterpret_cast<const uint32_t*>(p.tile_kmax)[(int64_t)kv_slab(bh, p.H, p.Hkv) * n_norm_tiles + min(opaque_lane(), n_norm_tiles - 1)];
  };
  auto take_q = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH, m0 = (p.num_m_blocks - 1 - i / p.BH) * C::kBlockM;
    park_rotated_rows<D>(qrows, qb, wave_tile, p.q_rot_out != nullptr ? p.q_rot_out + (int64_t)bh * N * D : nullptr,
                         m0 + wave * 32, N, p.qk_scale, opaque_lane());
  };

  // ---- first item: nothing to hide its prologue behind ----------------------------------------------------------------
  int item = item_at(0);
  COROPE_ISTAMP(0);
  load_item(0);
  kst.load(l_kg, 0, N);
  vst.load(l_vg, 0, N, (uint32_t)p.v_sn * 2);
  request_q(item);
  request_kvec(item);
  take_q(item);
  kst.store_rows(lds_at(koff_cur));
  vst.store_rows(lds_at(voff_cur));
  load_next_tile();
  __syncthreads();

  for (int round = 0;; ++round) {
    const int bh = item % p.BH, mb = p.num_m_blocks - 1 - item / p.BH;
    const int m0 = mb * C::kBlockM;
    const int n_tiles = tiles_of(mb);
    const uint32_t* tile_kmax_bits = reinterpret_cast<const uint32_t*>(p.tile_kmax) + (int64_t)kv_slab(bh, p.H, p.Hkv) * n_norm_tiles;
    COROPE_ISTAMP(1);

    // Largest |q_r| (scaled: base-2 units) of the wave's rows, a little generous: times the largest key norm of a tile it
    // bounds the tile's scores.
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
      q_bound_wave = __builtin_sqrtf(wave_max(half_sum(ss))) * 1.01f;
#pragma unroll
      for (int kc = 0; kc < M; ++kc) qa[kc] = to_acc_half(qb[kc]);
    }

    f32x16 oacc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i) oacc[i] = f32x16{0};
    float m_run = -INFINITY;    // reference value of the exponentials (this lane's query), base-2 units
    float m_true = -INFINITY;   // largest score seen by the reference moves
    float l_run = 0.f;          // this lane's share of the denominator up to the last move of the reference
    float lsum = 0.f;           // ... and since then
    float keep = 0.f;           // first probability of the pair in flight
    f32x16 msb = f32x16{0};     // -m_run in every register: the accumulator the score MFMAs start from
    f32x16 s;                   // scores of the tile
    float s_prev[8];            // scores 8..15 of the lane in the tile before it (the half whose softmax is still to come)
    u32x4 pb[2];                // P^T operand of the tile: the first half of its softmax fills pb[0]
    u32x4 pb_prev[2];           // ... of the tile before it: pb_prev[0] taken over from pb[0], pb_prev[1] from s_prev

    const int wave_q_lo = m0 + wave * 32;
    const int key_limit = CAUSAL ? wave_q_lo + lq : N - 1;   // last key this lane's query attends to
    const int t_last = __builtin_amdgcn_readfirstlane(CAUSAL ? min(n_tiles - 1, (wave_q_lo + 31) / BLOCK_N) : n_tiles - 1);
    const int norm_last = (t_last * BLOCK_N) / 64;

    // Reference value that puts every tile this wave will see within the margin.
    float lift_target;
    {
      uint32_t kall = lane <= norm_last ? kvec : 0u;   // non-negative floats order like their bit patterns
      for (int tb = kWave; tb <= norm_last; tb += kWave) {
        const int tt = tb + lane;
        kall = max(kall, tt <= norm_last ? tile_kmax_bits[tt] : 0u);
      }
      lift_target = q_bound_wave * wave_max(__builtin_bit_cast(float, kall)) - kMargin;
    }
    uint32_t thr_bits = 0;
    int kvec_base = 0;

    auto v_operand = [&](uint32_t v_lane, int i) {   // MFMA i of a PV slot: output block i % NDB, 16-key step i / NDB
      return load_a_trans_at(lds_at(v_lane), LSV, 16 * (i / NDB), (i % NDB) * 32);
    };
    // Second half of the softmax of the previous tile, pair j (0..3), element e: from s_prev into pb_prev[1].
    auto softmax_prev = [&](int j, int e) __attribute__((always_inline)) {
      asm volatile("" : "+v"(lsum));
      const float pr = fast_exp2(s_prev[2 * j + e]);
      lsum += pr;
      if (e == 0) {
        keep = pr;
        asm volatile("" : "+v"(keep), "+v"(lsum));
      } else {
        uint32_t w = pack_elts(keep, pr);
        asm volatile("" : "+v"(w), "+v"(lsum));
        pb_prev[1][j] = w;
      }
    };
    // Takes the previous tile (first half of its softmax done) out of the pipeline: rest of its softmax, then its PV product
    // (its V tile is the previous one of the ring).
    auto drain = [&]() __attribute__((always_inline)) {
      uint32_t vp_lane = v_lane_off + voff_prev;
      asm volatile("" : "+v"(vp_lane));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        softmax_prev(j, 0);
        softmax_prev(j, 1);
      }
#pragma unroll
      for (int i = 0; i < M; ++i) oacc[i % NDB] = mfma32(v_operand(vp_lane, i), pb_prev[i / NDB], oacc[i % NDB]);
    };

#pragma unroll
    for (int kc = 0; kc < M; ++kc) asm volatile("" ::"a"(qa[kc]));
    asm volatile("" ::"v"(kvec));
    COROPE_ISTAMP(2);
#ifdef COROPE_TRACE
    COROPE_ISTAMP_ID(n_tiles);
    const uint64_t clk0 = __builtin_readcyclecounter();
    uint64_t exact_passes = 0;
#endif

    auto tile_step = [&](int t, bool need_mask) __attribute__((always_inline)) {
      const int n0 = t * BLOCK_N;
#ifdef COROPE_TRACE
      if (t == 1) COROPE_ISTAMP(3);
      if (n0 == m0) COROPE_ISTAMP(4);
#endif
      uint32_t k_lane = k_lane_off + koff_cur, vprev = v_lane_off + (t == 0 ? voff_cur : voff_prev);
      asm volatile("" : "+v"(k_lane), "+v"(vprev));
      auto k_operand = [&](int kc) { return *reinterpret_cast<const u32x4*>(lds_at(k_lane) + RowTile<D>::off(0, 16 * kc)); };
      auto mask_scores = [&](f32x16& sacc) __attribute__((always_inline)) {
        int rel = key_limit - n0 - 4 * lh;
        asm volatile("" : "+v"(rel));
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (8 * (i / 4) + i % 4 > rel) sacc[i] = -INFINITY;
      };

      auto run_tile = [&](const bool MASK) __attribute__((always_inline)) {
        auto operand = [&](int n) { return n < M ? k_operand(n) : v_operand(vprev, n - M); };
        constexpr int TOTAL = 2 * M;
        u32x4 ring[RING];
#pragma unroll
        for (int n = 0; n < RING; ++n) ring[n] = operand(n);
        __builtin_amdgcn_sched_barrier(0);
        static_for<TOTAL>([&](auto n_c) __attribute__((always_inline)) {
          constexpr int n = decltype(n_c)::value;
          constexpr int slot = n / M, i = n % M;
          const u32x4 frag = ring[n % RING];
          if (slot == 0) { if (i == 0) s = mfma32_from_aq(frag, qa[i], msb); else mfma32_acc_aq(s, frag, qa[i]); }
          if (slot == 1) oacc[i % NDB] = mfma32(frag, pb_prev[i / NDB], oacc[i % NDB]);
          if (n + RING < TOTAL) ring[n % RING] = operand(n + RING);
          if (n == 0) stage_next();
          // The scores a slot's softmax reads were completed by an asm statement, behind which the compiler inserts no wait
          // states: nothing reads them behind MFMA 0 of the next slot, which waits a little instead.
          if (i == 0) asm volatile("s_nop 7");
          if (slot == 1 && i == 1 && MASK) mask_scores(s);
          // the slot's eight half pairs, spread over its MFMAs 1 .. M-1
#pragma unroll
          for (int hh = (i == 0 ? 0 : (i - 1) * 8 / (M - 1)); hh < (i == 0 ? 0 : i * 8 / (M - 1)); ++hh) {
            const int j = hh / 2, e = hh % 2;
            if (slot == 0) softmax_prev(j, e);                          // S(t-1), second half
            if (slot == 1) softmax_half(j, e, s, pb, lsum, keep);       // S(t), first half
          }
          __builtin_amdgcn_sched_barrier(0);
        });
        // the tile becomes the previous one: the scores its softmax still needs and the half of its P^T that exists move over
        // (vector moves of matrix-core results: the last score MFMA lies a whole slot back)
#pragma unroll
        for (int i = 0; i < 8; ++i) s_prev[i] = s[8 + i];
        pb_prev[0] = pb[0];
      };

      // ---- does the reference have to move before this tile? ------------------------------------------------------
      const int nt = n0 / 64;   // the 64-key block whose norm maximum bounds this tile
      if (nt - kvec_base == kWave) {
        kvec_base = nt;
        kvec = tile_kmax_bits[min(nt + lane, n_norm_tiles - 1)];
        asm volatile("" ::"v"(kvec));
      }
      const uint32_t kmax_bits = __builtin_amdgcn_readlane(kvec, nt - kvec_base);
      if (t == 0 || kmax_bits > thr_bits) {
#ifdef COROPE_TRACE
        ++exact_passes;
#endif
        if (t > 0) drain();
        f32x16 r = f32x16{0};
#pragma unroll
        for (int kc = 0; kc < M; ++kc) r = mfma32(k_operand(kc), from_acc_half(qa[kc]), r);
        if (need_mask) mask_scores(r);
        float mt = r[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mt = fmaxf(mt, r[i]);
        m_true = fmaxf(m_true, half_max(mt));
        const float m_new = fmaxf(m_run, fmaxf(m_true, fminf(lift_target, m_true + kLift)));
        const float alpha = fast_exp2(m_run - m_new);   // m_new is finite: every row sees key 0 of tile 0
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
          asm volatile("" : "+v"(x));   // sixteen values of their own
          msb[i] = x;
        }
        // nothing is pending now: all-masked previous scores and a zero P make the pending half of the tile body a no-op
#pragma unroll
        for (int i = 0; i < 8; ++i) s_prev[i] = -INFINITY;
        pb_prev[0] = pb_prev[1] = u32x4{0, 0, 0, 0};
        const float m_min = -wave_max(-m_run);
        const float thr = (m_min + kMargin) / q_bound_wave;
        thr_bits = __builtin_amdgcn_readfirstlane(thr > 0.f ? __builtin_bit_cast(uint32_t, thr) : 0u);
      }
      run_tile(need_mask);
      rotate_buffers();
      __syncthreads();
    };

    for (int t = 0; t <= t_last; ++t) {
      const bool need_mask = (CAUSAL && t * BLOCK_N + BLOCK_N - 1 > wave_q_lo) || (!CAUSAL && t * BLOCK_N + BLOCK_N > N);
      tile_step(t, need_mask);
    }

    // The next item's Q rows are requested as soon as the registers of this item's Q rows are free.  (After the last item
    // its own rows are requested once more and never used.)
    const int next_item = item_at(round + 1);
    const bool has_next = next_item < total;
    request_q(has_next ? next_item : item);
    request_kvec(has_next ? next_item : item);
    drain();
    COROPE_ISTAMP(5);
#ifdef COROPE_TRACE
    if (p.trace != nullptr && threadIdx.x == TT) {
      p.trace[(int64_t)item * 16 + 7] = __builtin_readcyclecounter() - clk0;
      p.trace[(int64_t)item * 16 + 13] = exact_passes;
    }
#endif
    // of the tiles entirely above this wave's diagonal it only stages its share
    for (int t = t_last + 1; t < n_tiles; ++t) {
      stage_next();
      rotate_buffers();
      __syncthreads();
    }
    {
      const float l_tot = half_sum(l_run + lsum);
      store_rows_via_wave_tile<D>(oacc, p.o + (int64_t)bh * N * D, wave_q_lo, N, 1.f / l_tot, wave_tile, opaque_lane());
      if (wave_q_lo + lq < N && lh == 0) p.lse[(int64_t)bh * N + wave_q_lo + lq] = m_run + fast_log2(l_tot);
    }
    COROPE_ISTAMP(6);
    if (!has_next) break;
    item = next_item;
    COROPE_ISTAMP(0);
    take_q(item);
  }
}

// ---- host-side launch -----------------------------------------------------------------------------------------
template <int D, bool CAUSAL>
static hipError_t launch_pipe64(FwdParams p, hipStream_t stream) {
  using C = pipe64::Cfg<D>;
  auto kern = rope_attn_fwd_pipe64_kernel<D, CAUSAL>;
  static std::atomic<uint64_t> lds_ok{0};
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), C::kLdsBytes, lds_ok); e != hipSuccess) return e;
  p.num_m_blocks = (p.N + C::kBlockM - 1) / C::kBlockM;
#ifdef COROPE_TRACE
  p.trace = g_trace_buf;
#endif
  const int64_t n_items = (int64_t)p.num_m_blocks * p.BH;
  const int64_t cus = device_cu_count();
  dim3 grid((unsigned)(n_items < cus ? n_items : cus));
  hipLaunchKernelGGL(kern, grid, dim3(C::kThreads), C::kLdsBytes, stream, p);
  return hipGetLastError();
}

hipError_t launch_rope_attn_fwd_prerotated_rows64(const FwdParams& p, int D, bool causal, hipStream_t stream) {
  if (D != 128) return hipErrorInvalidValue;
  return causal ? launch_pipe64<128, true>(p, stream) : launch_pipe64<128, false>(p, stream);
}

template <int D, bool CAUSAL>
static hipError_t launch_pipe32(FwdParams p, hipStream_t stream) {
  using C = pipe64::Cfg32<D>;
  auto kern = rope_attn_fwd_pipe32_kernel<D, CAUSAL>;
  static std::atomic<uint64_t> lds_ok{0};
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), C::kLdsBytes, lds_ok); e != hipSuccess) return e;
  p.num_m_blocks = (p.N + C::kBlockM - 1) / C::kBlockM;
#ifdef COROPE_TRACE
  p.trace = g_trace_buf;
#endif
  const int64_t n_items = (int64_t)p.num_m_blocks * p.BH;
  const int64_t slots = (int64_t)device_cu_count() * C::kWavesPerSimd;   // workgroups resident at once
  dim3 grid((unsigned)(n_items < slots ? n_items : slots));
  hipLaunchKernelGGL(kern, grid, dim3(C::kThreads), C::kLdsBytes, stream, p);
  return hipGetLastError();
}

hipError_t launch_rope_attn_fwd_prerotated_pipe256(const FwdParams& p, bool causal, hipStream_t stream) {
  return causal ? launch_pipe32<256, true>(p, stream) : launch_pipe32<256, false>(p, stream);
}

// Head dim 128 in the same form, two workgroups of four waves per compute unit.
hipError_t launch_rope_attn_fwd_prerotated_pipe32x2(const FwdParams& p, bool causal, hipStream_t stream) {
  return causal ? launch_pipe32<128, true>(p, stream) : launch_pipe32<128, false>(p, stream);
}

}  // namespace COROPE_NS
