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
  static constexpr int kRingBytes = kKStages * kKBytes + kVStages * kVBytes;
  // behind the ring: one private tile per wave, for its Q rows on their way in and its O rows on their way out.  The ring
  // is never reused for anything else, so the stream of K/V tiles runs on from one (head, query block) to the next.
  static constexpr int kLdsBytes = kRingBytes + NW * WaveTile<D>::kBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS of a compute unit");
};

// P^T is a bf16 operand in both builds (its unnormalised values span up to 2^kPipeMargin, more binary orders than fp16
// has), so the product O^T += V^T P^T is a bf16 product in both: in the fp16 build the V tile is converted to bf16 while
// it is staged (fp16's 11 significant bits become 8: the same rounding P itself carries).
#ifdef COROPE_F16
__device__ __forceinline__ u32x4 v_operand_format(u32x4 x) {
#pragma unroll
  for (int w = 0; w < 4; ++w) x[w] = pack_bf16(elt_lo(x[w]), elt_hi(x[w]));
  return x;
}
#else
__device__ __forceinline__ u32x4 v_operand_format(u32x4 x) { return x; }
#endif
template <class Stage, class Tile>
__device__ __forceinline__ void store_v_rows(const Stage& st, uint16_t* lds, Tile) {
#pragma unroll
  for (int it = 0; it < Stage::kIters; ++it) {
    const int u = threadIdx.x + it * (Stage::kUnits / Stage::kIters);
    *reinterpret_cast<u32x4*>(lds + Tile::off(u / Stage::kChunks, (u % Stage::kChunks) * 8)) = v_operand_format(st.x[it]);
  }
}

// One exponential pair of a 32-key half: scores 2j, 2j+1 of the lane (already relative to the reference value, base-2
// units) -> one bf16x2 word of the P^T operand.
__device__ __forceinline__ void softmax_pair(int j, const f32x16& sacc, u32x4 (&pb)[2], float& lsum) {
  asm volatile("" : "+v"(lsum));  // the pair starts here, not wherever the optimiser would like to hoist it
  float p0 = fast_exp2(sacc[2 * j]);
  float p1 = fast_exp2(sacc[2 * j + 1]);
  // plain adds: the bf16 dot-product instruction would do this in one op but stalls the MFMA pipe
  lsum += p0 + p1;
  uint32_t w = pack_bf16(p0, p1);
  asm volatile("" : "+v"(w), "+v"(lsum));   // ... and ends here, between the two MFMAs it is written between
  pb[j / 4][j % 4] = w;
}

__device__ __forceinline__ float wave_reduce_max(float x) { return wave_max(x); }   // data-parallel-primitive moves, no LDS round trips

// Persistent: the launch has one workgroup per compute unit (or per item, if those are fewer) and every workgroup walks
// its own list of items, an item being 32*NW query rows of one (batch, head).  The lists are fixed by arithmetic: items
// are ordered heaviest first (causal: last query block first; within a block over the heads), dealt to the workgroups in
// rounds, forwards in even rounds and backwards in odd ones, so that every workgroup ends up with the same number of
// key tiles when the rounds are full.  Workgroup ids are dealt round-robin to the 8 XCDs and both directions keep
// id % 8, so all items of a head stay on one XCD and share its L2.
//
// Across items the stream of K/V tiles does not stop: while the last tiles of an item are consumed, the staging
// registers and the ring already hold the first tiles of the next one.  Each wave keeps a private LDS tile behind the
// ring for its Q rows and O rows, so nothing at the change of items needs a workgroup barrier: a wave that is past its
// causal diagonal normalises and stores its O rows and requests the next item's Q rows while the other waves still work
// on the diagonal tiles, and only keeps staging its share of those tiles.
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

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lq = lane % 32, lh = lane / 32;
  // 32-row block of the item this wave owns.  Waves w and w + 4 share a SIMD: pairing blocks (0,7), (1,6), (2,5), (3,4)
  // gives every SIMD the same number of diagonal tiles.
  const int rb = NW == 8 ? (wave < 4 ? wave : 11 - wave) : wave;
  const int N = p.N;
  [[maybe_unused]] constexpr int TT = NW == 8 ? 4 * kWave : (NW - 1) * kWave;   // stamping thread: first lane of the wave with the last rows
  uint8_t* const wave_tile = smem + Cfg::kRingBytes + wave * WaveTile<D>::kBytes;

  // ---- the workgroup's list of items --------------------------------------------------------------------------------
  const ItemList items;
  const int total = p.num_m_blocks * p.BH;
  auto item_at = [&](int r) { return items.at(r); };   // position in the heaviest-first order; >= total: none
  const int n_k_tiles = (N + BLOCK_N - 1) / BLOCK_N;
  auto tiles_of = [&](int mb) {
    return CAUSAL ? min((mb * Cfg::kBlockM + Cfg::kBlockM + BLOCK_N - 1) / BLOCK_N, n_k_tiles) : n_k_tiles;
  };

  // ---- the stream of K/V tiles: a cursor two tiles ahead of the tile being consumed -----------------------------------
  CopyStage<D, BLOCK_N, NT, 8> kst;
  CopyStage<D, BLOCK_N, NT, Cfg::kVPad> vst;
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

  // LDS ring: K buffers at [0, 2 * kKBytes), V buffers behind them.  The buffers rotate by renaming byte offsets (no
  // modulo in the loop); every LDS address the loop uses is "one per-lane register per buffer and tile + an
  // immediate", which the opaque copies below enforce (left alone, the optimiser folds the buffer offset into each of
  // the ~30 operand addresses separately and keeps them all in registers).
  constexpr int kVBase = Cfg::kKStages * Cfg::kKBytes;
  int koff_cur = 0, koff_next = Cfg::kKBytes;
  int voff_prev = kVBase + 2 * Cfg::kVBytes, voff_cur = kVBase, voff_next = kVBase + Cfg::kVBytes;
  auto rotate_buffers = [&]() __attribute__((always_inline)) {
    int k = koff_cur; koff_cur = koff_next; koff_next = k;
    int v = voff_prev; voff_prev = voff_cur; voff_cur = voff_next; voff_next = v;
    // wave-uniform by construction; said explicitly, they stay in scalar registers
    koff_cur = __builtin_amdgcn_readfirstlane(koff_cur); koff_next = __builtin_amdgcn_readfirstlane(koff_next);
    voff_prev = __builtin_amdgcn_readfirstlane(voff_prev); voff_cur = __builtin_amdgcn_readfirstlane(voff_cur);
    voff_next = __builtin_amdgcn_readfirstlane(voff_next);
  };
  auto lds_at = [&](uint32_t byte_off) { return reinterpret_cast<uint16_t*>(smem + byte_off); };
  // per-lane parts of the operand addresses (bytes): K rows read directly, V through the transposing read
  const uint32_t k_lane_off = RowTile<D>::off(lq, 8 * lh) * 2;
  const uint32_t v_lane_off = a_trans_lane_offset(LSV) * 2;
  // Staging registers hold the tile after the one being consumed: it is written to its LDS buffers during the iteration
  // and the registers are refilled at once with the tile after that, so a global load has a whole iteration to land.
  // Row indices are clamped, which makes tiles past the end of a sequence harmless to load and store.
  auto stage_next = [&]() __attribute__((always_inline)) {
    int ko = koff_next, vo = voff_next;
    asm volatile("" : "+s"(ko), "+s"(vo));
    kst.store_rows(lds_at(ko));
    store_v_rows(vst, lds_at(vo), RowTile<D, Cfg::kVPad>{});
    load_next_tile();
  };

  // ---- Q rows of an item: load, rotate, scale, keep as the B operand; the largest key norms of the item's first 64 tiles --
  WaveRows<D, true> qrows;
  u32x4 qb[M];
  uint32_t kvec;   // lane i: bit pattern of the largest rotated-key norm of tile kvec_base + i
  // (the lane index goes in as a value the optimiser cannot see through: the two dozen per-lane address parts of these
  // steps are then recomputed per item; kept across the loop they do not fit the registers and come back one by one from
  // scratch memory, each with its full latency)
  auto opaque_lane = [&]() __attribute__((always_inline)) {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  auto request_q = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH, m0 = (p.num_m_blocks - 1 - i / p.BH) * Cfg::kBlockM;
    const int l = opaque_lane();
    qrows.load(p.q_slab(bh), p.cos, p.sin, p.fstride, m0 + rb * 32, N, l, (uint32_t)p.q_sn * 2);
    kvec = reinterpret_cast<const uint32_t*>(p.tile_kmax)[(int64_t)kv_slab(bh, p.H, p.Hkv) * n_k_tiles + min(l, n_k_tiles - 1)];
  };
  auto take_q = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH, m0 = (p.num_m_blocks - 1 - i / p.BH) * Cfg::kBlockM;
    park_rotated_rows<D>(qrows, qb, wave_tile, p.q_rot_out != nullptr ? p.q_rot_out + (int64_t)bh * N * D : nullptr,
                         m0 + rb * 32, N, p.qk_scale, opaque_lane());
  };

  // ---- first item: nothing to hide its prologue behind ----------------------------------------------------------------
  int item = item_at(0);
  COROPE_ISTAMP(0);
  load_item(0);
  kst.load(l_kg, 0, N);
  vst.load(l_vg, 0, N, (uint32_t)p.v_sn * 2);
  request_q(item);
  take_q(item);
  kst.store_rows(lds_at(koff_cur));
  store_v_rows(vst, lds_at(voff_cur), RowTile<D, Cfg::kVPad>{});
  load_next_tile();
  __syncthreads();

  for (int round = 0;; ++round) {
    const int bh = item % p.BH, mb = p.num_m_blocks - 1 - item / p.BH;
    const int m0 = mb * Cfg::kBlockM;
    const int n_tiles = tiles_of(mb);
    const int q_row = m0 + rb * 32 + lq;           // absolute query index of this lane
    const uint32_t* tile_kmax_bits = reinterpret_cast<const uint32_t*>(p.tile_kmax) + (int64_t)kv_slab(bh, p.H, p.Hkv) * n_k_tiles;
    COROPE_ISTAMP(1);

    // Largest |q_r| (scaled: base-2 units) of the wave's rows, a little generous: times a tile's largest key norm it
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
      q_bound_wave = __builtin_sqrtf(wave_reduce_max(half_sum(ss))) * 1.01f;
    }

    f32x16 oacc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i) oacc[i] = f32x16{0};
    float m_run = -INFINITY;   // reference value of the exponentials (this lane's query), base-2 units
    float m_true = -INFINITY;  // largest score seen by the reference moves (at most the row's true running maximum)
    float l_run = 0.f;         // this lane's share of the denominator up to the last move of the reference
    float lsum = 0.f;          // ... and since then
    f32x16 msb = f32x16{0};    // -m_run in every register: the accumulator the score MFMAs start from
    f32x16 s1;                 // scores of the second half of the previous tile (softmax half done)
    u32x4 pb0[2], pb1[2];      // P^T operands of the two halves

    const int wave_q_lo = m0 + rb * 32, wave_q_hi = wave_q_lo + 31;
    const int key_limit = CAUSAL ? q_row : N - 1;   // last key this lane's query attends to
    // last tile this wave's rows can see
    const int t_last = __builtin_amdgcn_readfirstlane(CAUSAL ? min(n_tiles - 1, wave_q_hi / BLOCK_N) : n_tiles - 1);

    // Reference value that puts every tile this wave will see within the margin.
    float lift_target;
    {
      uint32_t kall = lane <= t_last ? kvec : 0u;   // non-negative floats order like their bit patterns
      for (int t0 = kWave; t0 <= t_last; t0 += kWave) {
        const int tt = t0 + lane;
        kall = max(kall, tt <= t_last ? tile_kmax_bits[tt] : 0u);
      }
      // (bit patterns of non-negative floats: the float maximum is their maximum)
      lift_target = q_bound_wave * wave_max(__builtin_bit_cast(float, kall)) - kPipeMargin;
    }

    // Bit patterns of non-negative floats order like the floats: the per-tile test "bound > reference + margin" is
    // kmax_bits > thr_bits with thr = (min over rows of m_run + margin) / q_bound_wave, recomputed when the
    // reference moves.  Lane i of kvec holds the key-norm maximum of tile kvec_base + i.
    uint32_t thr_bits = 0;
    int kvec_base = 0;

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
      for (int i = 0; i < M; ++i) oacc[i % NDB] = mfma32_bf16(v_operand(vp_lane, 1, i), pb1[i / NDB], oacc[i % NDB]);
    };

    // the Q operands and the first 64 key-norm maxima have landed before the loop on every path: left to their first use,
    // the wait would sit inside the loop and there also wait for the next tile's loads
#pragma unroll
    for (int kc = 0; kc < M; ++kc) asm volatile("" ::"v"(qb[kc]));
    asm volatile("" ::"v"(kvec));
    COROPE_ISTAMP(2);
#ifdef COROPE_TRACE
    COROPE_ISTAMP_ID(n_tiles);
    const uint64_t clk0 = __builtin_readcyclecounter();
    uint64_t exact_passes = 0;   // tiles of this wave that were examined a second time to move the reference
#endif
    // ---- tiles this wave's rows can see ------------------------------------------------------------------------------
    for (int t = 0; t <= t_last; ++t) {
      const int n0 = t * BLOCK_N;
#ifdef COROPE_TRACE
      if (t == 1) COROPE_ISTAMP(3);
      if (n0 == m0) COROPE_ISTAMP(4);
#endif
      // K(t), V(t), V(t-1); the first tile of an item has no predecessor: its "previous V" is multiplied by a zero P1 and
      // only has to be finite wherever V(0) is, so it is V(0) itself
      uint32_t k_lane = k_lane_off + koff_cur, vt = v_lane_off + voff_cur, vprev = v_lane_off + (t == 0 ? voff_cur : voff_prev);
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
          if (slot == 1) oacc[i % NDB] = mfma32_bf16(ring[n % RING], pb1[i / NDB], oacc[i % NDB]);
          if (slot == 2) s1 = i == 0 ? mfma32_from(ring[n % RING], qb[i], msb) : mfma32(ring[n % RING], qb[i], s1);
          if (slot == 3) oacc[i % NDB] = mfma32_bf16(ring[n % RING], pb0[i / NDB], oacc[i % NDB]);
          if (n + RING < TOTAL) ring[n % RING] = operand(n + RING);
          if (n == 0) stage_next();
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
        const float m_new = fmaxf(m_run, fmaxf(m_true, fminf(lift_target, m_true + kPipeLift)));
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
          asm volatile("" : "+v"(x));   // sixteen values of their own: one value in sixteen places is tied to the first of them
          msb[i] = x;
        }
        const float m_min = -wave_reduce_max(-m_run);
        const float thr = (m_min + kPipeMargin) / q_bound_wave;
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
    // The next item's Q rows are requested as soon as the registers of this item's Q rows are free: for the waves that see
    // the item's last tile nothing but the rest of this block hides that latency.  (After the last item its own rows are
    // requested once more and never used: the request is then unconditional, and the registers it fills are free during
    // the tile loop on every path.)
    const int next_item = item_at(round + 1);
    const bool has_next = next_item < total;
    request_q(has_next ? next_item : item);
    drain();
    COROPE_ISTAMP(5);
#ifdef COROPE_TRACE
    if (p.trace != nullptr && threadIdx.x == TT) {
      p.trace[(int64_t)item * 16 + 7] = __builtin_readcyclecounter() - clk0;
      p.trace[(int64_t)item * 16 + 13] = exact_passes;
    }
#endif

    // ---- of the tiles entirely above this wave's diagonal it only stages its share; then the item's O rows and statistic
    // leave, all waves at once, and the next item's Q rows are taken in -----------------------------------------------------
    for (int t = t_last + 1; t < n_tiles; ++t) {
      stage_next();
      rotate_buffers();
      __syncthreads();
    }
    {
      const float l_tot = half_sum(l_run + lsum);
      store_rows_via_wave_tile<D>(oacc, p.o + (int64_t)bh * N * D, m0 + rb * 32, N, 1.f / l_tot, wave_tile, opaque_lane());
      if (q_row < N && lh == 0) p.lse[(int64_t)bh * N + q_row] = m_run + fast_log2(l_tot);
    }
    COROPE_ISTAMP(6);
    if (!has_next) break;
    item = next_item;
    COROPE_ISTAMP(0);
    take_q(item);
  }
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
  dim3 grid(persistent_grid((int64_t)p.num_m_blocks * p.BH, NW, Cfg::kLdsBytes));
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, p);
  return hipGetLastError();
}

template <int D, bool CAUSAL>
static hipError_t launch_pipe_cfg(const FwdParams& p, hipStream_t stream) {
  return use_small_tiles(p.N, p.BH, FwdPipeCfg<D, 4>::kLdsBytes) ? launch_pipe_waves<D, CAUSAL, 4>(p, stream)
                                                                  : launch_pipe_waves<D, CAUSAL, 8>(p, stream);
}

hipError_t launch_rope_attn_fwd_prerotated(const FwdParams& p, int D, bool causal, hipStream_t stream) {
  // without key-norm maxima: the kernel that needs none
  if (p.tile_kmax == nullptr) return launch_rope_attn_fwd_single_prerotated(p, D, causal, stream);
#ifndef COROPE_F16
  if (D == 256 && g_fwd_wave_rows.load(std::memory_order_relaxed) != 32)
    return launch_rope_attn_fwd_prerotated_pipe256(p, causal, stream);
#endif
  if (D == 256) return launch_rope_attn_fwd_single_prerotated(p, D, causal, stream);
  if (D != 64 && D != 128) return hipErrorInvalidValue;
#ifndef COROPE_F16
  if (D == 128 && g_fwd_wave_rows.load(std::memory_order_relaxed) == 128)
    return launch_rope_attn_fwd_prerotated_pipe32x2(p, causal, stream);
  if (D == 128 && !use_small_tiles(p.N, p.BH) && g_fwd_wave_rows.load(std::memory_order_relaxed) == 64)
    return launch_rope_attn_fwd_prerotated_rows64(p, D, causal, stream);
#endif
  if (D == 128) return causal ? launch_pipe_cfg<128, true>(p, stream) : launch_pipe_cfg<128, false>(p, stream);
  return causal ? launch_pipe_cfg<64, true>(p, stream) : launch_pipe_cfg<64, false>(p, stream);
}

}  // namespace COROPE_NS
