// Fused half-layout-RoPE flash-attention backward for gfx950: the dK/dV kernel and the dQ kernel.
//
// Device counterparts of the reference's _attn_bwd_dkdv / _attn_bwd_dq
// (fused-rope/fused_rope_attn.py:342-404, :409-470, driver :474-649).  The reference runs both halves in one
// program and re-rotates Q (resp. K) in registers on every inner iteration; here each half is its own kernel
// and the streamed operand is rotated once per workgroup per tile while it is staged into LDS.  No atomics:
// dK/dV are owned by the key block's workgroup, dQ by the query block's.
//
// Scaling contract (same as the reference's, :385, :457, :574-575, :643-644, with the host-side K pre-scale
// :746-748 folded in): P = exp2(s * sm_scale * log2e - M) with M the forward's base-2 statistic;
// dS = P o (dP - delta); dK_r = sm_scale * dS^T Q_r; dQ_r = sm_scale * dS K_r; both un-rotated in fp32
// before the single rounding to bf16.
//
// Operands that must be read "transposed" (contraction along the sequence axis of a row-major tile) use the
// gfx950 transposing LDS read, so every tile is staged row-major exactly once.
#include "common.hpp"
#include "kernels.hpp"

namespace COROPE_NS {

// Layout of LDS tiles that are read both row-wise (16 bytes per lane, lane = row) and through the transposing read
// (8 bytes per lane, 4 rows x 32 bytes per 16 lanes).  With plain row padding, 16 bytes keep the row-wise reads free of
// bank conflicts and leave the transposing ones four-way conflicted, 64 bytes do the opposite; measured on the fused
// dK+dV kernel at B2 H32 N4096 D128, paddings of 16 / 32 / 48 / 64 / 80 bytes gave 0.551 / 0.524 / 0.512 / 0.561 /
// 0.523 ms.  The staggered layout (free of conflicts both ways, 68 bytes a row) gains another 1.4 % there, side by side
// on one device; in the dQ kernel it loses 2.8 % to the 48-byte padding (more registers spilled for its addresses).
constexpr int kBothWaysPad = 24;
constexpr int kDkdvBothWaysPad = kStaggerPad;

// ===================================================================================== dK / dV
// Workgroup = NWAVES waves x 32 keys.  K_r and V rows of the wave stay in registers as B operands.
// Per query tile (BLOCK_M rows, staged: rotated Q and dO, plus M and delta):
//   S  = Q_r K_r^T            (A = Q_r rows from LDS,      B = K_r regs)   lane = key, registers = queries
//   dP = dO V^T               (A = dO rows from LDS,       B = V regs)
//   P  = exp2(S*c - M), dS = P o (dP - delta)                               (bf16, already B-operand shaped)
//   dV^T   += dO^T  P         (A = dO tile read transposed, B = P)
//   dK_r^T += Q_r^T dS        (A = Q_r tile read transposed, B = dS)
// DO_PAD: row padding of the dO tile.  The dV-only kernel reads dO through the transposing load alone and takes the
// padding that is conflict-free for it (32); the dK kernel reads dO row-wise (8).
// V_LDS: the waves' V rows live in LDS instead of registers -- the fused dK+dV kernel, whose two sets of accumulators
// leave no room for them.
//
// Persistent, like the other attention kernels: one workgroup per compute unit walks a balanced list of (key/value slab,
// key block) items and the stream of query tiles runs on from item to item.  Behind the two tile stages every wave has an
// LDS slot of its own (32 padded rows): its V rows during an item (V_LDS), and at the change of items the tile through
// which its dV and dK rows leave and its next K_r rows come in -- nothing there needs a workgroup barrier.
template <int D, int NWAVES, int BLOCK_M, int DO_PAD, int Q_PAD>
struct DkdvCfg {
  static constexpr int kThreads = NWAVES * kWave;
  static constexpr int kBlockN = NWAVES * 32;
  static constexpr int kTileBytes = RowTile<D, Q_PAD>::bytes(BLOCK_M);
  static constexpr int kDoTileBytes = RowTile<D, DO_PAD>::bytes(BLOCK_M);
  static constexpr int kStatBytes = BLOCK_M * 4;
  static constexpr int kStageBytes = kTileBytes + kDoTileBytes + 2 * kStatBytes;
  static constexpr int kRingBytes = 2 * kStageBytes;
  static constexpr int kWaveBytes = RowTile<D>::bytes(32);
  static_assert(kWaveBytes >= WaveTile<D>::kBytes, "a wave's slot holds its unpadded tile too");
  static constexpr int kLdsBytes = kRingBytes + NWAVES * kWaveBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS of a compute unit");
};

// PREROT: Q and K come from copies that rope_rotate_kernel rotated beforehand (no table reads in the loop).
template <int D, int NWAVES, int BLOCK_M, bool CAUSAL, bool DO_DV, bool DO_DK, bool PREROT>
__global__ __launch_bounds__(NWAVES* kWave) __attribute__((amdgpu_waves_per_eu(kWavesPerSimd<D>, kWavesPerSimd<D>))) void rope_attn_bwd_dkdv_kernel(BwdParams p) {
  constexpr int DO_PAD = DO_DK ? (DO_DV ? kDkdvBothWaysPad : 8) : 32;
  constexpr int Q_PAD = DO_DK ? kDkdvBothWaysPad : 8;
  constexpr bool V_LDS = DO_DV && DO_DK;
  using Cfg = DkdvCfg<D, NWAVES, BLOCK_M, DO_PAD, Q_PAD>;
  constexpr int NT = Cfg::kThreads;
  constexpr int KC = D / 16, NDB = D / 32, NQB = BLOCK_M / 32;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lq = lane % 32, lh = lane / 32;
  // 32-key block of the item this wave owns; waves w and w + 4 share a SIMD, blocks (0,7), (1,6), (2,5), (3,4) give
  // every SIMD the same number of diagonal tiles
  const int rb = NWAVES == 8 ? (wave < 4 ? wave : 11 - wave) : wave;
  [[maybe_unused]] constexpr int TT = 0;   // stamping thread: first lane of the wave with the first keys (it sees every tile)
  const int N = p.N;
  uint8_t* const wave_slot = smem + Cfg::kRingBytes + wave * Cfg::kWaveBytes;
  uint16_t* const vrows = reinterpret_cast<uint16_t*>(wave_slot);   // V_LDS: the wave's V rows, row-major, padded

  // An item: a key block of one key/value slab; its workgroup sweeps the query tiles of every query head of the group
  // (one head without grouped-query attention), accumulating dK and dV over all of them.  Heaviest first: causal key
  // blocks see fewer query tiles the later they lie.
  const ItemList items;
  const int BHkv = p.BH / p.H * p.Hkv, GQ = p.H / p.Hkv;
  const int total = p.num_blocks * BHkv;   // item i: key block i / BHkv of slab i % BHkv
  const int m_tiles = (N + BLOCK_M - 1) / BLOCK_M;
  const uint16_t* q_all = PREROT ? p.q_rot : p.q;

  // ---- the stream of query tiles: a cursor one tile ahead of the tile being consumed -----------------------------------
  RopeStage<D, BLOCK_M, NT, PREROT, true, Q_PAD> qst;   // Q_r tiles carry qk_scale: S leaves the matrix cores in base-2 units
  qst.out_scale = p.qk_scale;
  CopyStage<D, BLOCK_M, NT, DO_PAD> dst;
  float st_lse = 0.f, st_delta = 0.f;
  int l_round = 0, l_it = 0, l_iters, l_slab0, l_mt0, l_tph;
  auto load_item = [&](int r) {    // false: no such item
    const int i = items.at(r);
    if (i >= total) return false;
    const int bkv = i % BHkv, n0 = (i / BHkv) * Cfg::kBlockN;
    l_slab0 = (bkv / p.Hkv) * p.H + (bkv % p.Hkv) * GQ;   // first query head of the group
    l_mt0 = CAUSAL ? n0 / BLOCK_M : 0;
    l_tph = max(m_tiles - l_mt0, 0);
    l_iters = GQ * l_tph;
    return true;
  };
  // iteration it of an item -> query head slab0 + it / tph, query tile mt0 + it % tph
  auto load_next_tile = [&](bool advance) __attribute__((always_inline)) {
    if (advance) {
      if (l_it + 1 < l_iters) {
        ++l_it;
      } else if (load_item(l_round + 1)) {
        ++l_round;
        l_it = 0;
      }   // else: past the last tile of the last item; the same tile is requested again and never used
    }
    const int qs = l_slab0 + l_it / l_tph, m0 = (l_mt0 + l_it % l_tph) * BLOCK_M;
    qst.load(q_all + (int64_t)qs * N * D, p.cos, p.sin, p.fstride, m0, N);
    dst.load(p.d_o + (int64_t)qs * N * D, m0, N);
    if (threadIdx.x < BLOCK_M) {
      int qi = m0 + threadIdx.x;
      // -M and -delta: what the S and dP products start from.  Rows past the end: M = +inf makes P = 0, so they
      // contribute nothing
      st_lse = qi < N ? -p.lse[(int64_t)qs * N + qi] : -INFINITY;
      if constexpr (DO_DK) st_delta = qi < N ? -p.delta[(int64_t)qs * N + qi] : 0.f;
    }
  };
  auto q_tile = [&](int buf) { return reinterpret_cast<uint16_t*>(smem + buf * Cfg::kStageBytes); };
  auto do_tile = [&](int buf) { return reinterpret_cast<uint16_t*>(smem + buf * Cfg::kStageBytes + Cfg::kTileBytes); };
  auto lse_tile = [&](int buf) {
    return reinterpret_cast<float*>(smem + buf * Cfg::kStageBytes + Cfg::kTileBytes + Cfg::kDoTileBytes);
  };
  auto delta_tile = [&](int buf) {
    return reinterpret_cast<float*>(smem + buf * Cfg::kStageBytes + Cfg::kTileBytes + Cfg::kDoTileBytes + Cfg::kStatBytes);
  };
  auto store_tile = [&](int buf) __attribute__((always_inline)) {
    qst.store_rows(q_tile(buf));
    dst.store_rows(do_tile(buf));
    if (threadIdx.x < BLOCK_M) {
      lse_tile(buf)[threadIdx.x] = st_lse;
      if constexpr (DO_DK) delta_tile(buf)[threadIdx.x] = st_delta;
    }
  };
  int cur = 0;   // ring stage of the tile being consumed

  // ---- the wave's K_r (and V) rows of an item ----------------------------------------------------------------------
  // (the lane index goes in as a value the optimiser cannot see through: the per-lane address parts of these steps are
  // then recomputed per item instead of being kept in registers, or in scratch memory, across the whole loop)
  auto opaque_lane = [&]() __attribute__((always_inline)) {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  WaveRows<D, !PREROT> krows;
  WaveRows<D, false> vrows_regs;
  u32x4 kb[KC], vb[(DO_DK && !V_LDS) ? KC : 1];
  auto request_rows = [&](int i) __attribute__((always_inline)) {
    const int64_t base = (int64_t)(i % BHkv) * N * D;
    const int row0 = (i / BHkv) * Cfg::kBlockN + rb * 32, l = opaque_lane();
    krows.load((PREROT ? p.k_rot : p.k) + base, p.cos, p.sin, p.fstride, row0, N, l);
    if constexpr (DO_DK) vrows_regs.load(p.v + base, nullptr, nullptr, 0, row0, N, l);
  };
  auto take_rows = [&]() __attribute__((always_inline)) {
    const int l = opaque_lane();
    park_rows<D>(krows, kb, wave_slot, 1.f, l);
    if constexpr (DO_DK && !V_LDS) park_plain_rows<D>(vrows_regs, vb, wave_slot, l);
    if constexpr (V_LDS) {
      using WR = WaveRows<D, false>;
      lds_order();
#pragma unroll
      for (int i = 0; i < WR::IT; ++i)
        *reinterpret_cast<u32x4*>(vrows + RowTile<D>::off(WR::RPI * i + l / WR::CPR, (l % WR::CPR) * 8)) = vrows_regs.x[i];
      lds_order();
    }
  };

  // ---- first item: nothing to hide its prologue behind ----------------------------------------------------------------
  int item = items.at(0);
  COROPE_ISTAMP(0);
  load_item(0);
  load_next_tile(false);
  request_rows(item);
  take_rows();
  store_tile(0);
  __syncthreads();

  for (int round = 0;; ++round) {
    const int bkv = item % BHkv, n0 = (item / BHkv) * Cfg::kBlockN;
    const int64_t base = (int64_t)bkv * N * D;                           // k, v, dk, dv
    const int mt0 = CAUSAL ? n0 / BLOCK_M : 0;
    const int tiles_per_head = max(m_tiles - mt0, 0), n_iter = GQ * tiles_per_head;
    const int wk_lo = n0 + rb * 32, wk_hi = wk_lo + 31;
    const int key = wk_lo + lq;
    COROPE_ISTAMP(1);
    COROPE_ISTAMP_ID(n_iter);
#ifdef COROPE_TRACE
    const uint64_t clk0 = __builtin_readcyclecounter();
#endif

    f32x16 dvacc[DO_DV ? NDB : 1], dkacc[DO_DK ? NDB : 1];
#pragma unroll
    for (int i = 0; i < NDB; ++i) {
      if constexpr (DO_DV) dvacc[i] = f32x16{0};
      if constexpr (DO_DK) dkacc[i] = f32x16{0};
    }
    // The wave's K_r (and V) rows must have landed on EVERY path into the loop: left to the first product that reads
    // them, the wait for them is placed inside the loop, where each time round it also waits for the next tile's loads
    // issued a few instructions earlier, and the prefetch hides less.
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) {
      asm volatile("" ::"v"(kb[kc]));
      if constexpr (DO_DK && !V_LDS) asm volatile("" ::"v"(vb[kc]));
    }

    for (int it = 0; it < n_iter; ++it) {
      const int m0 = (mt0 + it % tiles_per_head) * BLOCK_M;
#ifdef COROPE_TRACE
      if (it == 1) COROPE_ISTAMP(3);
      if (it == Cfg::kBlockN / BLOCK_M) COROPE_ISTAMP(4);   // first tile past the diagonal block
#endif
      load_next_tile(true);

      const uint16_t* qs = q_tile(cur);
      const uint16_t* dos = do_tile(cur);
      const float* lses = lse_tile(cur);
      const float* deltas = delta_tile(cur);
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb) {
        const int mq0 = m0 + qb * 32;
        // queries of this 32-row block that lie above every key of the wave see none of them
        if (CAUSAL && mq0 + 31 < wk_lo) continue;
        // The products start from -M and -delta of their rows (register i holds query 8*(i/4) + 4*lh + i%4 of the block):
        // S - M and dP - delta leave the matrix cores, no vector instruction applies them.
        f32x16 sacc, dpacc = f32x16{0};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 m4 = *reinterpret_cast<const f32x4*>(lses + qb * 32 + 8 * g + 4 * lh);
#pragma unroll
          for (int e = 0; e < 4; ++e) sacc[4 * g + e] = m4[e];
          if constexpr (DO_DK) {
            const f32x4 d4 = *reinterpret_cast<const f32x4*>(deltas + qb * 32 + 8 * g + 4 * lh);
#pragma unroll
            for (int e = 0; e < 4; ++e) dpacc[4 * g + e] = d4[e];
          }
        }
        const uint16_t* qrow = qs + RowTile<D, Q_PAD>::off(qb * 32 + lq, 8 * lh);
        const uint16_t* dorow = dos + RowTile<D, DO_PAD>::off(qb * 32 + lq, 8 * lh);
        constexpr bool V_FORM = kWavesPerSimd<D> == 1;   // see mfma32_acc_v
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
          const u32x4 a = *reinterpret_cast<const u32x4*>(qrow + 16 * kc);
          if constexpr (V_FORM) mfma32_acc_v(sacc, a, kb[kc]); else sacc = mfma32(a, kb[kc], sacc);
        }
        if constexpr (DO_DK) {
#pragma unroll
          for (int kc = 0; kc < KC; ++kc) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(dorow + 16 * kc);
            const u32x4 b = V_LDS ? *reinterpret_cast<const u32x4*>(vrows + RowTile<D>::off(lq, 8 * lh + 16 * kc)) : vb[V_LDS ? 0 : kc];
            if constexpr (V_FORM) mfma32_acc_v(dpacc, a, b); else dpacc = mfma32(a, b, dpacc);
          }
        }
        if constexpr (V_FORM) mfma32_settle(DO_DK ? dpacc : sacc);

        // Causal mask on the raw scores, under a wave-uniform branch of its own (written into the exponential loop it
        // is turned into compare + select on every tile).  Register i holds query mq0 + 8*(i/4) + 4*lh + i%4; the
        // lane-dependent part of the threshold goes into one opaque value so that the 16 thresholds stay immediates.
        if (CAUSAL && mq0 < wk_hi) {
          int rel = key - mq0 - 4 * lh;
          asm volatile("" : "+v"(rel));
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (8 * (i / 4) + i % 4 < rel) sacc[i] = -INFINITY;
        }
        u32x4 pb[2], dsb[2];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float pv[4], ds[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            pv[e] = fast_exp2(sacc[4 * g + e]);
            ds[e] = pv[e] * dpacc[4 * g + e];
          }
          if constexpr (DO_DV) {
            pb[g / 2][2 * (g % 2)] = pack_elts(pv[0], pv[1]);
            pb[g / 2][2 * (g % 2) + 1] = pack_elts(pv[2], pv[3]);
          }
          if constexpr (DO_DK) {
            dsb[g / 2][2 * (g % 2)] = pack_elts(ds[0], ds[1]);
            dsb[g / 2][2 * (g % 2) + 1] = pack_elts(ds[2], ds[3]);
          }
        }
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
          const int kbase = qb * 32 + 16 * cc;
#pragma unroll
          for (int db = 0; db < NDB; ++db) {
            if constexpr (DO_DV) dvacc[db] = mfma32(load_a_trans_of<RowTile<D, DO_PAD>>(dos, kbase, db * 32), pb[cc], dvacc[db]);
            if constexpr (DO_DK) dkacc[db] = mfma32(load_a_trans_of<RowTile<D, Q_PAD>>(qs, kbase, db * 32), dsb[cc], dkacc[db]);
          }
        }
        // without the causal branches the two blocks of a tile are one stretch of code: kept apart, or the scheduler
        // interleaves them and needs both blocks' score registers at once
        if constexpr (!CAUSAL) __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (kWavesPerSimd<D> == 1) {
        // one wave per SIMD: the accumulators' home is the accumulation half of the register file, where the MFMAs the
        // compiler selects update them; said here, or it carries them round the loop in the other half and copies all of
        // them over and back on every tile
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          if constexpr (DO_DV) asm volatile("" : "+a"(dvacc[db]));
          if constexpr (DO_DK) asm volatile("" : "+a"(dkacc[db]));
        }
      }
      store_tile(cur ^ 1);
      cur ^= 1;
      __syncthreads();
    }

    COROPE_ISTAMP(5);
#ifdef COROPE_TRACE
    if (p.trace != nullptr && threadIdx.x == TT) p.trace[(int64_t)item * 16 + 7] = __builtin_readcyclecounter() - clk0;
#endif
    // ---- change of items, all within the wave's own LDS slot.  The table values dK needs on its way out are requested
    // first and land while dV leaves (which waits for nothing); behind them (loads return in the order they were issued)
    // the next item's rows, which land while dK leaves.  After the last item its own rows are requested once more and
    // never used: the request is then unconditional, and the registers it fills are free during the tile loop on every path.
    UnrotateTables<D> tb;
    if constexpr (DO_DK && PREROT) tb.load(p.cos, p.sin, p.fstride, wk_lo, N, opaque_lane());
    if constexpr (DO_DV) store_rows_via_wave_tile<D>(dvacc, p.dv + base, wk_lo, N, 1.f, wave_slot, opaque_lane());
    const int next_item = items.at(round + 1);
    const bool has_next = next_item < total;
    request_rows(has_next ? next_item : item);
    if constexpr (DO_DK) {
      if constexpr (!PREROT) tb.load(p.cos, p.sin, p.fstride, wk_lo, N, opaque_lane());
      // the Q_r operand carried sm_scale * log2(e): ln 2 is what is left of sm_scale
      store_unrotated_rows_via_wave_tile<D>(dkacc, tb, p.dk + base, wk_lo, N, 0.6931471805599453f, wave_slot, opaque_lane());
    }
    COROPE_ISTAMP(6);
    if (!has_next) break;
    item = next_item;
    COROPE_ISTAMP(0);
    take_rows();
  }
}

// ===================================================================================== dQ
// Workgroup = NWAVES waves x 32 queries.  Rotated Q rows and dO rows of the wave stay in registers.
// Per key tile (BLOCK_N rows, staged: rotated K and V):
//   S^T  = K_r Q_r^T          (A = K_r rows from LDS, B = Q_r regs)    lane = query, registers = keys
//   dP^T = V dO^T             (A = V rows from LDS,   B = dO regs)
//   dS^T = P^T o (dP^T - delta)                                        (bf16, B-operand shaped)
//   dQ_r^T += K_r^T dS^T      (A = K_r tile read transposed, B = dS^T)
template <int D, int NWAVES, int BLOCK_N>
struct DqCfg {
  static constexpr int kThreads = NWAVES * kWave;
  static constexpr int kBlockM = NWAVES * 32;
  static constexpr int kKTileBytes = RowTile<D, kBothWaysPad>::bytes(BLOCK_N);   // K_r: read row-wise and transposed
  static constexpr int kVTileBytes = RowTile<D>::bytes(BLOCK_N);                 // V: read row-wise
  static constexpr int kStageBytes = kKTileBytes + kVTileBytes;
  static constexpr int kRingBytes = 2 * kStageBytes;
  // behind the ring, per wave: a private tile for its operand rows on their way in and its dQ rows on their way out, and
  // the 32 delta values of its rows
  static constexpr int kWaveBytes = WaveTile<D>::kBytes + 32 * 4;
  static constexpr int kLdsBytes = kRingBytes + NWAVES * kWaveBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS of a compute unit");
};

// Persistent, like the forward on a pre-rotated K: one workgroup per compute unit walks a balanced list of (head, query
// block) items, the stream of K/V tiles runs on from item to item, and nothing at the change of items needs a workgroup
// barrier (a wave's operand rows and its dQ rows go through an LDS tile of its own).
template <int D, int NWAVES, int BLOCK_N, bool CAUSAL, bool PREROT>
__global__ __launch_bounds__(NWAVES* kWave) __attribute__((amdgpu_waves_per_eu(kWavesPerSimd<D>, kWavesPerSimd<D>))) void rope_attn_bwd_dq_kernel(BwdParams p) {
  using Cfg = DqCfg<D, NWAVES, BLOCK_N>;
  constexpr int NT = Cfg::kThreads;
  constexpr int KC = D / 16, NDB = D / 32, NKB = BLOCK_N / 32;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lq = lane % 32, lh = lane / 32;
  // 32-row block of the item this wave owns; waves w and w + 4 share a SIMD, blocks (0,7), (1,6), (2,5), (3,4) give
  // every SIMD the same number of diagonal tiles
  const int rb = NWAVES == 8 ? (wave < 4 ? wave : 11 - wave) : wave;
  [[maybe_unused]] constexpr int TT = NWAVES == 8 ? 4 * kWave : (NWAVES - 1) * kWave;   // stamping thread: first lane of the wave with the last rows
  const int N = p.N;
  uint8_t* const wave_tile = smem + Cfg::kRingBytes + wave * Cfg::kWaveBytes;
  float* const wave_delta = reinterpret_cast<float*>(wave_tile + WaveTile<D>::kBytes);

  const ItemList items;
  const int total = p.num_blocks * p.BH;   // item i (heaviest first): query block num_blocks - 1 - i / BH of head i % BH
  const int n_k_tiles = (N + BLOCK_N - 1) / BLOCK_N;
  auto tiles_of = [&](int mb) {
    return CAUSAL ? min((mb * Cfg::kBlockM + Cfg::kBlockM + BLOCK_N - 1) / BLOCK_N, n_k_tiles) : n_k_tiles;
  };

  // ---- the stream of K/V tiles: a cursor one tile ahead of the tile being consumed -------------------------------------
  RopeStage<D, BLOCK_N, NT, PREROT, false, kBothWaysPad> kst;
  CopyStage<D, BLOCK_N, NT> vst;
  int l_round = 0, l_tile = 0, l_tiles;
  const uint16_t *l_kg, *l_vg;
  auto load_item = [&](int r) {    // false: no such item
    const int i = items.at(r);
    if (i >= total) return false;
    const int64_t kv_base = (int64_t)kv_slab(i % p.BH, p.H, p.Hkv) * N * D;
    l_kg = (PREROT ? p.k_rot : p.k) + kv_base;
    l_vg = p.v + kv_base;
    l_tiles = tiles_of(p.num_blocks - 1 - i / p.BH);
    return true;
  };
  auto load_next_tile = [&]() __attribute__((always_inline)) {   // moves the cursor on and requests that tile
    if (l_tile + 1 < l_tiles) {
      ++l_tile;
    } else if (load_item(l_round + 1)) {
      ++l_round;
      l_tile = 0;
    }   // else: past the last tile of the last item; the same tile is requested again and never used
    kst.load(l_kg, p.cos, p.sin, p.fstride, l_tile * BLOCK_N, N);
    vst.load(l_vg, l_tile * BLOCK_N, N);
  };
  auto k_tile = [&](int buf) { return reinterpret_cast<uint16_t*>(smem + buf * Cfg::kStageBytes); };
  auto v_tile = [&](int buf) { return reinterpret_cast<uint16_t*>(smem + buf * Cfg::kStageBytes + Cfg::kKTileBytes); };
  int cur = 0;   // ring stage of the tile being consumed

  // ---- operand rows of an item: Q_r (rotated and scaled here unless a pre-rotated copy is given), dO, O for delta ------
  // (the lane index goes in as a value the optimiser cannot see through: the per-lane address parts of these steps are
  // then recomputed per item instead of being kept in registers, or in scratch memory, across the whole loop)
  auto opaque_lane = [&]() __attribute__((always_inline)) {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  WaveRows<D, !PREROT> qrows;
  WaveRows<D, false> dorows, orows;
  float lse_q, delta_in;
  u32x4 qb[KC], dob[KC];
  float delta_q;
  auto request_rows = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH, row0 = (p.num_blocks - 1 - i / p.BH) * Cfg::kBlockM + rb * 32;
    const int64_t base = (int64_t)bh * N * D;
    const int l = opaque_lane();
    qrows.load((PREROT ? p.q_rot : p.q) + base, p.cos, p.sin, p.fstride, row0, N, l);
    dorows.load(p.d_o + base, nullptr, nullptr, 0, row0, N, l);
    // (without O the dO rows are requested twice: the request is then unconditional and the registers it fills are free
    // during the tile loop on every path)
    orows.load((p.o != nullptr ? p.o : p.d_o) + base, nullptr, nullptr, 0, row0, N, l);
    const int q_c = min(row0 + l % 32, N - 1);
    lse_q = p.lse[(int64_t)bh * N + q_c];
    // delta_i = sum_d o_id * do_id (reference _attn_bwd_preprocess, :324-337): read from the preprocess pass, or -- when the
    // caller hands over O instead -- computed here for the rows this workgroup owns and written out for the dK kernel,
    // which then has to run after this one.
    delta_in = 0.f;
    if (p.o == nullptr) delta_in = p.delta[(int64_t)bh * N + q_c];
  };
  auto take_rows = [&](int i) __attribute__((always_inline)) {
    const int bh = i % p.BH, row0 = (p.num_blocks - 1 - i / p.BH) * Cfg::kBlockM + rb * 32;
    const int l = opaque_lane();
    park_rows<D>(qrows, qb, wave_tile, p.qk_scale, l);   // Q_r carries qk_scale (a pre-rotated copy already does)
    park_plain_rows<D>(dorows, dob, wave_tile, l);
    delta_q = delta_in;
    if (p.o != nullptr) {
      // 16 lanes per row: O and dO in registers, same chunk order
      constexpr int CPR = D / 8, RPI = kWave / CPR;
#pragma unroll
      for (int i2 = 0; i2 < 32 / RPI; ++i2) {
        const int r = RPI * i2 + l / CPR, ch = l % CPR;
        const u32x4 ow = orows.x[i2], dw = dorows.x[i2];
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) acc += elt_lo(ow[w]) * elt_lo(dw[w]) + elt_hi(ow[w]) * elt_hi(dw[w]);
        if constexpr (CPR == 16) {
          acc = row16_sum(acc);
        } else {
#pragma unroll
          for (int m = CPR / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m);
        }
        if (ch == 0) wave_delta[r] = acc;
      }
      lds_order();
      delta_q = wave_delta[l % 32];
      lds_order();
      if (l / 32 == 0 && row0 + l % 32 < N) p.delta[(int64_t)bh * N + row0 + l % 32] = delta_q;
    }
  };

  // ---- first item: nothing to hide its prologue behind ----------------------------------------------------------------
  int item = items.at(0);
  COROPE_ISTAMP(0);
  load_item(0);
  kst.load(l_kg, p.cos, p.sin, p.fstride, 0, N);
  vst.load(l_vg, 0, N);
  request_rows(item);
  take_rows(item);
  kst.store_rows(k_tile(0));
  vst.store_rows(v_tile(0));
  __syncthreads();

  for (int round = 0;; ++round) {
    const int bh = item % p.BH, mb = p.num_blocks - 1 - item / p.BH;
    const int m0 = mb * Cfg::kBlockM;
    const int n_tiles = tiles_of(mb);
    const int q_row = m0 + rb * 32 + lq;
    const int wq_lo = m0 + rb * 32, wq_hi = wq_lo + 31;
    const int key_limit = CAUSAL ? q_row : N - 1;   // last key this lane's query attends to
    // last tile this wave's rows can see
    const int t_last = __builtin_amdgcn_readfirstlane(CAUSAL ? min(n_tiles - 1, wq_hi / BLOCK_N) : n_tiles - 1);
    COROPE_ISTAMP(1);
    COROPE_ISTAMP_ID(n_tiles);
#ifdef COROPE_TRACE
    const uint64_t clk0 = __builtin_readcyclecounter();
#endif

    f32x16 dqacc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i) dqacc[i] = f32x16{0};
    // S - M leaves the matrix cores: the score products start from -M of the lane's query in every register
    f32x16 msb;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float x = -lse_q;
      asm volatile("" : "+v"(x));   // sixteen values of their own: one value in sixteen places is tied to the first of them
      msb[i] = x;
    }
    // the wave's operands have landed on every path into the loop (left to their first use, the wait would sit inside
    // the loop and there also wait for the next tile's loads)
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) asm volatile("" ::"v"(qb[kc]), "v"(dob[kc]));
    asm volatile("" ::"v"(delta_q));

    auto stage_next = [&]() __attribute__((always_inline)) {
      kst.store_rows(k_tile(cur ^ 1));
      vst.store_rows(v_tile(cur ^ 1));
    };

    for (int t = 0; t <= t_last; ++t) {
      const int n0 = t * BLOCK_N;
#ifdef COROPE_TRACE
      if (t == 1) COROPE_ISTAMP(3);
      if (n0 == m0) COROPE_ISTAMP(4);
#endif
      load_next_tile();
      const uint16_t* ks = k_tile(cur);
      const uint16_t* vs = v_tile(cur);
      const bool need_mask = (CAUSAL && n0 + BLOCK_N - 1 > wq_lo) || (!CAUSAL && n0 + BLOCK_N > N);
      u32x4 dsb[BLOCK_N / 16];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        f32x16 sacc, dpacc;   // dP starts from a literal zero, S from -M
        const uint16_t* krow = ks + RowTile<D, kBothWaysPad>::off(kb * 32 + lq, 8 * lh);
        const uint16_t* vrow = vs + RowTile<D>::off(kb * 32 + lq, 8 * lh);
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
          // (mfma32_from is for builds whose accumulators stay in the registers it names: with one wave per SIMD the
          // compiler keeps them in the other half of the register file and would copy the result there at once)
          sacc = kc > 0 ? mfma32(*reinterpret_cast<const u32x4*>(krow + 16 * kc), qb[kc], sacc)
                 : kWavesPerSimd<D> == 2 ? mfma32_from(*reinterpret_cast<const u32x4*>(krow), qb[0], msb)
                                         : mfma32(*reinterpret_cast<const u32x4*>(krow), qb[0], msb);
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
          dpacc = mfma32(*reinterpret_cast<const u32x4*>(vrow + 16 * kc), dob[kc], kc == 0 ? f32x16{0} : dpacc);
        // mask on the raw scores under a wave-uniform branch of its own; register i holds key
        // n0 + 32*kb + 8*(i/4) + 4*lh + i%4, the lane-dependent part of the threshold goes into one opaque value
        if (need_mask) {
          int rel = key_limit - n0 - 4 * lh;
          asm volatile("" : "+v"(rel));
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (kb * 32 + 8 * (i / 4) + i % 4 > rel) sacc[i] = -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          float ds[2];
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            float pv = fast_exp2(sacc[i + e]);
            ds[e] = pv * (dpacc[i + e] - delta_q);
          }
          dsb[2 * kb + i / 8][(i % 8) / 2] = pack_elts(ds[0], ds[1]);
        }
      }
#pragma unroll
      for (int c = 0; c < BLOCK_N / 16; ++c)
#pragma unroll
        for (int db = 0; db < NDB; ++db)
          dqacc[db] = mfma32(load_a_trans_of<RowTile<D, kBothWaysPad>>(ks, 16 * c, db * 32), dsb[c], dqacc[db]);
      stage_next();
      cur ^= 1;
      __syncthreads();
    }
    COROPE_ISTAMP(5);
#ifdef COROPE_TRACE
    if (p.trace != nullptr && threadIdx.x == TT) p.trace[(int64_t)item * 16 + 7] = __builtin_readcyclecounter() - clk0;
#endif
    // The next item's rows are requested as soon as the registers of this item's rows are free.  (After the last item its
    // own rows are requested once more and never used: the request is then unconditional, and the registers it fills are
    // free during the tile loop on every path.)
    // Ahead of them go the table values that the item's dQ rows need on their way out: loads return in the order they
    // were issued, and those must not wait for the next item's rows.
    // (Only on pre-rotated operands: rows that are rotated here travel with their own table values, and both sets do not
    // fit the registers.)
    UnrotateTables<D> tb;
    if constexpr (PREROT) tb.load(p.cos, p.sin, p.fstride, wq_lo, N, opaque_lane());
    const int next_item = items.at(round + 1);
    const bool has_next = next_item < total;
    request_rows(has_next ? next_item : item);
    // of the tiles entirely above this wave's diagonal it only stages its share
    for (int t = t_last + 1; t < n_tiles; ++t) {
      load_next_tile();
      stage_next();
      cur ^= 1;
      __syncthreads();
    }
    // dQ_r -> dQ: scaled, un-rotated in fp32, rounded once, whole rows per store
    if constexpr (!PREROT) tb.load(p.cos, p.sin, p.fstride, wq_lo, N, opaque_lane());
    store_unrotated_rows_via_wave_tile<D>(dqacc, tb, p.dq + (int64_t)bh * N * D, wq_lo, N, p.sm_scale, wave_tile, opaque_lane());
    COROPE_ISTAMP(6);
    if (!has_next) break;
    item = next_item;
    COROPE_ISTAMP(0);
    take_rows(item);
  }
}

// ===================================================================================== launchers
template <int D, bool CAUSAL, bool DO_DV, bool DO_DK, bool PREROT, int NWAVES>
static hipError_t launch_dkdv_waves(BwdParams p, hipStream_t stream) {
  constexpr int BLOCK_M = D > 128 ? 32 : 64;   // what fits the LDS beside the waves' own slots
  using Cfg = DkdvCfg<D, NWAVES, BLOCK_M, DO_DK ? (DO_DV ? kDkdvBothWaysPad : 8) : 32, DO_DK ? kDkdvBothWaysPad : 8>;
  auto kern = rope_attn_bwd_dkdv_kernel<D, NWAVES, BLOCK_M, CAUSAL, DO_DV, DO_DK, PREROT>;
  static std::atomic<uint64_t> lds_ok{0};
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes, lds_ok); e != hipSuccess) return e;
  p.num_blocks = (p.N + Cfg::kBlockN - 1) / Cfg::kBlockN;
#ifdef COROPE_TRACE
  p.trace = g_trace_buf;
#endif
  const unsigned grid = persistent_grid((int64_t)p.num_blocks * (p.BH / p.H * p.Hkv), NWAVES, Cfg::kLdsBytes);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, p);
  return hipGetLastError();
}

template <int D, bool CAUSAL, bool DO_DV, bool DO_DK, bool PREROT>
static hipError_t launch_dkdv_cfg(const BwdParams& p, hipStream_t stream) {
  if constexpr (D > 128) {
    return launch_dkdv_waves<D, CAUSAL, DO_DV, DO_DK, PREROT, 4>(p, stream);   // 4 waves x 512 registers
  } else {
    using Small = DkdvCfg<D, 4, 64, DO_DK ? (DO_DV ? kDkdvBothWaysPad : 8) : 32, DO_DK ? kDkdvBothWaysPad : 8>;
    return use_small_tiles(p.N, p.BH / p.H * p.Hkv, Small::kLdsBytes) ? launch_dkdv_waves<D, CAUSAL, DO_DV, DO_DK, PREROT, 4>(p, stream)
                                                     : launch_dkdv_waves<D, CAUSAL, DO_DV, DO_DK, PREROT, 8>(p, stream);
  }
}

template <int D, bool CAUSAL, bool PREROT, int NWAVES>
static hipError_t launch_dq_waves(BwdParams p, hipStream_t stream) {
  constexpr int BLOCK_N = D > 128 ? 32 : 64;   // what fits the LDS beside the waves' own tiles
  using Cfg = DqCfg<D, NWAVES, BLOCK_N>;
  auto kern = rope_attn_bwd_dq_kernel<D, NWAVES, BLOCK_N, CAUSAL, PREROT>;
  static std::atomic<uint64_t> lds_ok{0};
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes, lds_ok); e != hipSuccess) return e;
  p.num_blocks = (p.N + Cfg::kBlockM - 1) / Cfg::kBlockM;
#ifdef COROPE_TRACE
  p.trace = g_trace_buf;
#endif
  const unsigned grid = persistent_grid((int64_t)p.num_blocks * p.BH, NWAVES, Cfg::kLdsBytes);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, p);
  return hipGetLastError();
}

template <int D, bool CAUSAL, bool PREROT>
static hipError_t launch_dq_cfg(const BwdParams& p, hipStream_t stream) {
  if constexpr (D > 128) {
    return launch_dq_waves<D, CAUSAL, PREROT, 4>(p, stream);   // 4 waves x 512 registers
  } else {
    return use_small_tiles(p.N, p.BH, DqCfg<D, 4, 64>::kLdsBytes) ? launch_dq_waves<D, CAUSAL, PREROT, 4>(p, stream)
                                      : launch_dq_waves<D, CAUSAL, PREROT, 8>(p, stream);
  }
}

// Dispatch on the run-time switches (head dim, causal, pre-rotated operands present).
template <bool DO_DV, bool DO_DK>
static hipError_t launch_dkdv(const BwdParams& p, int D, bool causal, hipStream_t stream) {
  const bool pre = p.q_rot != nullptr && p.k_rot != nullptr;
#define COROPE_DKDV(DD, CC, PP) launch_dkdv_cfg<DD, CC, DO_DV, DO_DK, PP>(p, stream)
  if (D == 256) {   // separate dV and dK only: the accumulators of both do not fit one wave
    if (DO_DV && DO_DK) return hipErrorInvalidValue;
    if constexpr (!(DO_DV && DO_DK)) {
      if (pre) return causal ? COROPE_DKDV(256, true, true) : COROPE_DKDV(256, false, true);
      return causal ? COROPE_DKDV(256, true, false) : COROPE_DKDV(256, false, false);
    }
  }
  if (D == 128) {
    if (pre) return causal ? COROPE_DKDV(128, true, true) : COROPE_DKDV(128, false, true);
    return causal ? COROPE_DKDV(128, true, false) : COROPE_DKDV(128, false, false);
  }
  if (D != 64) return hipErrorInvalidValue;
  if (pre) return causal ? COROPE_DKDV(64, true, true) : COROPE_DKDV(64, false, true);
  return causal ? COROPE_DKDV(64, true, false) : COROPE_DKDV(64, false, false);
#undef COROPE_DKDV
}

hipError_t launch_bwd_dkdv_fused(const BwdParams& p, int D, bool causal, hipStream_t stream) {
  if (D == 256) {
    if (p.q_rot != nullptr && p.k_rot != nullptr)   // on rotated copies: fused, both sets of accumulators in the accumulation registers
      return causal ? launch_dkdv_cfg<256, true, true, true, true>(p, stream) : launch_dkdv_cfg<256, false, true, true, true>(p, stream);
    if (hipError_t e = launch_dkdv<true, false>(p, D, causal, stream); e != hipSuccess) return e;
    return launch_dkdv<false, true>(p, D, causal, stream);
  }
  return launch_dkdv<true, true>(p, D, causal, stream);
}

hipError_t launch_bwd_dv(const BwdParams& p, int D, bool causal, hipStream_t stream) {
  return launch_dkdv<true, false>(p, D, causal, stream);
}

hipError_t launch_bwd_dk(const BwdParams& p, int D, bool causal, hipStream_t stream) {
  return launch_dkdv<false, true>(p, D, causal, stream);
}

hipError_t launch_bwd_dq(const BwdParams& p, int D, bool causal, hipStream_t stream) {
  const bool pre = p.q_rot != nullptr && p.k_rot != nullptr;
  if (D == 256) {
    if (pre) return causal ? launch_dq_cfg<256, true, true>(p, stream) : launch_dq_cfg<256, false, true>(p, stream);
    return causal ? launch_dq_cfg<256, true, false>(p, stream) : launch_dq_cfg<256, false, false>(p, stream);
  }
  if (D == 128) {
    if (pre) return causal ? launch_dq_cfg<128, true, true>(p, stream) : launch_dq_cfg<128, false, true>(p, stream);
    return causal ? launch_dq_cfg<128, true, false>(p, stream) : launch_dq_cfg<128, false, false>(p, stream);
  }
  if (D != 64) return hipErrorInvalidValue;
  if (pre) return causal ? launch_dq_cfg<64, true, true>(p, stream) : launch_dq_cfg<64, false, true>(p, stream);
  return causal ? launch_dq_cfg<64, true, false>(p, stream) : launch_dq_cfg<64, false, false>(p, stream);
}

}  // namespace COROPE_NS
