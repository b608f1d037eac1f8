// Fused half-layout-RoPE flash-attention forward for gfx950.
//
// Device counterpart of the reference's _attn_fwd / _attn_fwd_inner
// (fused-rope/fused_rope_attn.py:222-320, :48-138).
//
// One workgroup owns 256 query rows of one (batch, head); each of its 8 waves owns 32 of them.
// Scores are produced transposed, S^T = K_r Q_r^T, with 32x32x16 bf16 MFMAs: the rotated K tile is the A
// operand (read from LDS), the rotated Q rows are the B operand (registers, loaded and rotated once).  In
// the 32x32 accumulator every lane then holds 16 keys of ONE query, so the online-softmax row statistics
// are a per-lane reduction plus one exchange between the two halves of the wave, and the bf16 P^T values
// are already laid out as the B operand of O^T += V^T P^T (V tile staged row-major, read with the transposing
// LDS load).
//
// K tiles are rotated while they are staged global -> registers -> LDS, once per workgroup per tile
// (the reference re-rotates per program: :82-99); the next tile's global loads are issued before the
// current tile's MFMAs and written to the next LDS buffer afterwards (one barrier per tile).
#include "common.hpp"
#include "kernels.hpp"

#include <type_traits>

namespace COROPE_NS {

// Workgroup = 8 waves x 32 query rows = 256 rows, two waves per SIMD.
//
// Issue schedule.  VALU work only overlaps an MFMA that is already in flight, so a wave that mixes independent VALU
// instructions into its MFMA stream keeps the matrix pipe busier than one that runs an MFMA phase followed by a
// VALU phase.  A 64-key tile is therefore consumed as two 32-key halves in four slots of 8 MFMAs each, and every
// slot carries the VALU work of another stage in the same basic block for the instruction scheduler to mix in:
//     slot A:  S^T(half 0)          +  rotate K / copy V of tile t+1 into LDS, refill the staging registers (tile t+2)
//     slot B:  S^T(half 1)          +  online softmax of half 0
//     slot C:  O^T += V^T P^T(h0)   +  online softmax of half 1
//     slot D:  O^T += V^T P^T(h1)
// Scheduling barriers separate the slots and pin the operand prefetches ahead of the MFMAs that use them.
constexpr int kFwdStages = 2;

template <int D, int BLOCK_N, int NW>
struct FwdCfg {
  static constexpr int kThreads = NW * kWave;
  static constexpr int kBlockM = NW * 32;
  static constexpr int kVPad = 32;                                       // V is read only through load_a_trans
  static constexpr int kKBytes = RowTile<D>::bytes(BLOCK_N);             // K tile, row-major, read row-wise
  static constexpr int kVBytes = RowTile<D, kVPad>::bytes(BLOCK_N);      // V tile, row-major, read transposed
  static constexpr int kStageBytes = kKBytes + kVBytes;
  static constexpr int kLoopBytes = kFwdStages * kStageBytes;
  static constexpr int kEpilogueBytes = NW * 32 * kAccTileStride<D> * 4;   // fp32 O rows of all waves on their way out
  static constexpr int kLdsBytes = kLoopBytes > kEpilogueBytes ? kLoopBytes : kEpilogueBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS of a compute unit");
};

// ---- online softmax with a lazily updated reference maximum -------------------------------------------------------
// Probabilities are formed against a per-row reference m_ref that is NOT the running maximum: p = exp2(s*c - m_ref*c).
// Any finite reference gives the same normalised result (numerator and denominator carry the same factor), so the
// reference only has to stay close enough to the true maximum for p to remain a comfortable fp32 / bf16 number.  The
// fast path therefore skips the maximum altogether (no reduction, no cross-lane exchange, no accumulator rescale, no
// dependency between the scores and the first exponential); it only watches the half's partial denominator, and when
// that grows past kLsumLimit -- some score is ~2^20 above the reference, or the reference is still -inf on the first
// tile, which shows up as inf/NaN -- the half is redone on the slow path, which moves the reference to the true maximum
// and rescales the accumulators like a classic online softmax.
#ifdef COROPE_F16
constexpr float kLsumLimit = 16384.f;     // fp16 probabilities: everything the matrix cores see stays below 65504
#else
constexpr float kLsumLimit = 1048576.f;
#endif

// Fast-path piece `step` of `n_steps`: exponentiates 8 / n_steps score pairs of a half.
__device__ __forceinline__ void softmax_fast_piece(int step, int n_steps, const f32x16& sacc, u32x4 (&pb)[2], float& lsum,
                                                   float scale, float ms) {
  const int lo = step * 8 / n_steps, hi = (step + 1) * 8 / n_steps;
  asm volatile("" : "+v"(ms));  // the piece starts here, not wherever the scheduler would like to hoist it
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if (j < lo || j >= hi) continue;
    float p0 = fast_exp2(sacc[2 * j] * scale - ms);
    float p1 = fast_exp2(sacc[2 * j + 1] * scale - ms);
    // plain adds: the bf16 dot-product instruction would do this in one op but stalls the MFMA pipe
    lsum += p0 + p1;
    uint32_t w = pack_elts(p0, p1);
    asm volatile("" : "+v"(w));  // keeps the piece between the two MFMAs it is written between
    pb[j / 4][j % 4] = w;
  }
}

// Slow path of one half: classic online-softmax step.  Returns the factor the accumulators must be multiplied by.
__device__ __forceinline__ float softmax_slow_half(const f32x16& sacc, u32x4 (&pb)[2], float& m_ref, float& l_run,
                                                   float scale) {
  float mt = fmaxf(sacc[0], sacc[1]);
#pragma unroll
  for (int i = 2; i < 16; i += 2) mt = fmaxf(fmaxf(mt, sacc[i]), sacc[i + 1]);
  const float m_new = fmaxf(m_ref, half_max(mt));
  const float ms = m_new * scale;
  const float alpha = fast_exp2(m_ref * scale - ms);
  float lsum = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float p0 = fast_exp2(sacc[2 * j] * scale - ms);
    float p1 = fast_exp2(sacc[2 * j + 1] * scale - ms);
    lsum += p0 + p1;
    pb[j / 4][j % 4] = pack_elts(p0, p1);
  }
  l_run = l_run * alpha + lsum;
  m_ref = m_new;
  return alpha;
}

// This kernel knows nothing about the keys in advance, so every half runs the fast pieces and is verified afterwards
// (two data-dependent branches per tile); the two-launch forward in rope_attn_fwd_pipe.hip gets the same guarantee
// from key norms computed beforehand and has no such branch.
// PREROT: the keys come from a copy that rope_rotate_kernel rotated beforehand (p.k_rot; no table reads and no rotation in
// the loop), and the rotated, scaled query rows are also written to p.q_rot_out when that is given.
template <int D, int BLOCK_N, bool CAUSAL, int NW, bool PREROT = false>
__global__ __launch_bounds__(NW* kWave) __attribute__((amdgpu_waves_per_eu(kWavesPerSimd<D>, kWavesPerSimd<D>))) void rope_attn_fwd_kernel(FwdParams p) {
  using Cfg = FwdCfg<D, BLOCK_N, NW>;
  static_assert(BLOCK_N == 64, "the slot schedule is written for two 32-key halves");
  constexpr int NT = Cfg::kThreads;
  constexpr int KC = D / 16;        // contraction chunks of QK^T = MFMAs per S^T half
  constexpr int NDB = D / 32;       // 32-column blocks of O
  constexpr int NPV = 2 * NDB;      // MFMAs per PV half
  constexpr int KA = D > 128 ? 2 : 4;       // K operands in flight
  constexpr int NAV = D > 128 ? 4 : NDB;    // transposed V operands in flight
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

  const uint16_t* qg = p.q_slab(bh);
  const uint32_t q_rb = (uint32_t)p.q_sn * 2, k_rb = PREROT ? D * 2 : (uint32_t)p.k_sn * 2, v_rb = (uint32_t)p.v_sn * 2;   // bytes between rows
  const int kvs = kv_slab(bh, p.H, p.Hkv);   // key/value slab of this query head
  const uint16_t* kg = PREROT ? p.k_rot + (int64_t)kvs * N * D : p.k_slab(kvs);
  const uint16_t* vg = p.v_slab(kvs);

  const int n_k_tiles = (N + BLOCK_N - 1) / BLOCK_N;
  const int n_tiles = CAUSAL ? min((m0 + Cfg::kBlockM + BLOCK_N - 1) / BLOCK_N, n_k_tiles) : n_k_tiles;

  // SPLIT (D = 256, where registers are short): the staging registers hold half a tile (32 rows) at a time, and each
  // half has half an iteration to land.
  constexpr bool SPLIT = D > 128;
  constexpr int SROWS = SPLIT ? BLOCK_N / 2 : BLOCK_N;
  RopeStage<D, SROWS, NT, PREROT> kst;
  CopyStage<D, SROWS, NT, Cfg::kVPad> vst;
  kst.load(kg, p.cos, p.sin, p.fstride, 0, N, k_rb);
  vst.load(vg, 0, N, v_rb);

  // ---- Q rows of this wave: load, rotate, keep as the B operand (through a wave-private LDS tile, so that the
  // global loads touch whole row segments) ---------------------------------------------------------------------
  const int q_row = m0 + wave * 32 + lq;           // absolute query index of this lane
  u32x4 qb[KC];
  {
    WaveRows<D, true> qrows;
    qrows.load(qg, p.cos, p.sin, p.fstride, m0 + wave * 32, N, threadIdx.x % kWave, q_rb);
    // the rotated Q rows carry sm_scale * log2(e), as in every other kernel of the operator: forward and backward then
    // see the same rounded operands, and the same scores
    qrows.park(qb, reinterpret_cast<uint16_t*>(smem) + wave * 32 * RowTile<D>::kStride,
               PREROT && p.q_rot_out != nullptr ? p.q_rot_out + (int64_t)bh * N * D : nullptr, m0 + wave * 32, N, p.qk_scale);
  }
  __syncthreads();   // the K and V buffers below overlap the tiles the waves just used
  if constexpr (D > 128) {
    // one wave per SIMD: the Q operand's home is the accumulator half of the register file (the matrix cores read their
    // B operand from there as well); left to itself the register allocator keeps it in scratch memory and reloads a piece
    // in front of every score product
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) asm volatile("" : "+a"(qb[kc]));
  }

  constexpr float scale = 1.f;   // scores come out of the matrix cores in base-2 units
  f32x16 oacc[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i) oacc[i] = f32x16{0};
  float m_run = -INFINITY;   // reference maximum of the raw scores (this lane's query); see the softmax notes above
  float l_run = 0.f;         // this lane's share of the running denominator

  auto ks = [&](int t) { return reinterpret_cast<uint16_t*>(smem + (t % kFwdStages) * Cfg::kStageBytes); };
  auto vs = [&](int t) {
    return reinterpret_cast<uint16_t*>(smem + (t % kFwdStages) * Cfg::kStageBytes + Cfg::kKBytes);
  };
  // Staging registers hold tile t+1 during iteration t: it is written to its LDS buffer during the iteration and the
  // registers are refilled at once with tile t+2, so a global load has a whole iteration to land.  Row indices
  // are clamped, which makes tiles past the end harmless to load and store.
  kst.store_rows(ks(0));
  vst.store_rows(vs(0));
  if constexpr (SPLIT) {
    kst.load(kg, p.cos, p.sin, p.fstride, SROWS, N, k_rb);
    vst.load(vg, SROWS, N, v_rb);
    kst.store_rows(ks(0) + RowTile<D>::off(SROWS, 0));
    vst.store_rows(vs(0) + RowTile<D, Cfg::kVPad>::off(SROWS, 0));
  }
  kst.load(kg, p.cos, p.sin, p.fstride, BLOCK_N, N, k_rb);
  vst.load(vg, BLOCK_N, N, v_rb);
  __syncthreads();

  const int wave_q_lo = m0 + wave * 32, wave_q_hi = wave_q_lo + 31;
  for (int t = 0; t < n_tiles; ++t) {
    const int n0 = t * BLOCK_N;
    const uint16_t* kt = ks(t) + RowTile<D>::off(lq, 8 * lh);
    const uint16_t* vt = vs(t);
    // All of the staging happens at one point of the iteration: tile t+1 goes from the staging registers to its LDS
    // buffer and the registers are refilled with tile t+2 straight away.
    auto stage_next = [&]() {
      kst.store_rows(ks(t + 1));
      vst.store_rows(vs(t + 1));
      const int next_rows = SPLIT ? n0 + BLOCK_N + SROWS : n0 + 2 * BLOCK_N;   // SPLIT: the other half of tile t+1
      kst.load(kg, p.cos, p.sin, p.fstride, next_rows, N, k_rb);
      vst.load(vg, next_rows, N, v_rb);
    };
    auto stage_second_half = [&]() {   // SPLIT only: second half of tile t+1 to LDS, first half of tile t+2 requested
      if constexpr (SPLIT) {
        kst.store_rows(ks(t + 1) + RowTile<D>::off(SROWS, 0));
        vst.store_rows(vs(t + 1) + RowTile<D, Cfg::kVPad>::off(SROWS, 0));
        kst.load(kg, p.cos, p.sin, p.fstride, n0 + 2 * BLOCK_N, N, k_rb);
        vst.load(vg, n0 + 2 * BLOCK_N, N, v_rb);
      }
    };
    auto k_operand = [&](int half, int kc) {
      return *reinterpret_cast<const u32x4*>(kt + RowTile<D>::off(half * 32, 16 * kc));
    };
    auto v_operand = [&](int half, int i) {  // MFMA i of a PV half: output block i % NDB, 16-key chunk i / NDB
      return load_a_trans(vt, LSV, half * 32 + 16 * (i / NDB), (i % NDB) * 32);
    };
    auto mask_scores = [&](f32x16& sacc, int half) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        int key = n0 + half * 32 + acc_row(i, lh);
        if (CAUSAL ? key > q_row : key >= N) sacc[i] = -INFINITY;
      }
    };
    auto rescale = [&](float alpha) {
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
    };

    // One tile in four slots of 8 MFMAs (see the schedule at the top of the file).
    auto run_tile = [&](const bool MASK) {
      f32x16 s0 = f32x16{0}, s1 = f32x16{0};
      u32x4 pb0[2], pb1[2];
      float lsum0 = 0.f, lsum1 = 0.f;
      float ms_ref = m_run * scale;
      u32x4 a[KA];  // ring of A operands, fetched KA MFMAs ahead of their use
#pragma unroll
      for (int kc = 0; kc < KA; ++kc) a[kc] = k_operand(0, kc);
      __builtin_amdgcn_sched_barrier(0);
      // ---- slot A: S^T(half 0), staging on the side --------------------------------------------------------------
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) {
        s0 = mfma32(a[kc % KA], qb[kc], s0);
        a[kc % KA] = kc + KA < KC ? k_operand(0, kc + KA) : k_operand(1, kc + KA - KC);
        if (kc == 0) stage_next();
      }
      __builtin_amdgcn_sched_barrier(0);
      if (MASK) mask_scores(s0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // ---- slot B: S^T(half 1), softmax of half 0 between the MFMAs ---------------------------------------------
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) {
        s1 = mfma32(a[kc % KA], qb[kc], s1);
        if (kc + KA < KC) a[kc % KA] = k_operand(1, kc + KA);
        softmax_fast_piece(kc, KC, s0, pb0, lsum0, scale, ms_ref);
        __builtin_amdgcn_sched_barrier(0);
      }
      {
        if (__builtin_amdgcn_ballot_w64(!(lsum0 <= kLsumLimit))) {
          rescale(softmax_slow_half(s0, pb0, m_run, l_run, scale));
        } else {
          l_run += lsum0;
        }
        ms_ref = m_run * scale;
      }
      if (MASK) mask_scores(s1, 1);
      u32x4 av[NAV];  // transposed V operands, NAV MFMAs ahead (one 16-key chunk up to D = 128)
#pragma unroll
      for (int db = 0; db < NAV; ++db) av[db] = v_operand(0, db);
      __builtin_amdgcn_sched_barrier(0);
      // ---- slot C: O^T += V^T P^T(half 0), softmax of half 1 between the MFMAs -----------------------------------
#pragma unroll
      for (int i = 0; i < NPV; ++i) {
        oacc[i % NDB] = mfma32(av[i % NAV], pb0[i / NDB], oacc[i % NDB]);
        av[i % NAV] = i + NAV < NPV ? v_operand(0, i + NAV) : v_operand(1, i + NAV - NPV);
        if (i == 0) stage_second_half();
        softmax_fast_piece(i, NPV, s1, pb1, lsum1, scale, ms_ref);
        __builtin_amdgcn_sched_barrier(0);
      }
      {
        if (__builtin_amdgcn_ballot_w64(!(lsum1 <= kLsumLimit))) {
          rescale(softmax_slow_half(s1, pb1, m_run, l_run, scale));
        } else {
          l_run += lsum1;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      // ---- slot D: O^T += V^T P^T(half 1) ------------------------------------------------------------------------
#pragma unroll
      for (int i = 0; i < NPV; ++i) {
        oacc[i % NDB] = mfma32(av[i % NAV], pb1[i / NDB], oacc[i % NDB]);
        if (i + NAV < NPV) av[i % NAV] = v_operand(1, i + NAV);
      }
    };
    // Tiles entirely above this wave's diagonal contribute nothing to it; the wave still stages its share.
    const bool active = !CAUSAL || n0 <= wave_q_hi;
    const bool need_mask = (CAUSAL && n0 + BLOCK_N - 1 > wave_q_lo) || (!CAUSAL && n0 + BLOCK_N > N);
    if (active) {
      run_tile(need_mask);
    } else {
      stage_next();
      stage_second_half();
    }
    __syncthreads();
  }

  // ---- epilogue: normalise, write O (through LDS, whole row segments per store) and the base-2 log-sum-exp ------------
  // (the loop ends with a barrier: every wave is done with the K and V buffers)
  const float l_tot = half_sum(l_run);
  const float inv_l = 1.f / l_tot;
  store_rows_via_lds<D, false>(oacc, p.o + (int64_t)bh * N * D, m0 + wave * 32, N, nullptr, nullptr, 0, inv_l,
                               reinterpret_cast<float*>(smem) + wave * 32 * kAccTileStride<D>);
  if (q_row < N && lh == 0) p.lse[(int64_t)bh * N + q_row] = m_run * scale + fast_log2(l_tot);
}

// ---- host-side launch -----------------------------------------------------------------------------------------
template <int D, int BLOCK_N, bool CAUSAL, int NW, bool PREROT = false>
static hipError_t launch_fwd_waves(FwdParams p, hipStream_t stream) {
  using Cfg = FwdCfg<D, BLOCK_N, NW>;
  auto kern = rope_attn_fwd_kernel<D, BLOCK_N, CAUSAL, NW, PREROT>;
  static std::atomic<uint64_t> lds_ok{0};
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes, lds_ok); e != hipSuccess) return e;
  p.num_m_blocks = (p.N + Cfg::kBlockM - 1) / Cfg::kBlockM;
  dim3 grid(p.num_m_blocks * p.BH);
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, p);
  return hipGetLastError();
}

template <int D, int BLOCK_N, bool CAUSAL, bool PREROT = false>
static hipError_t launch_fwd_cfg(const FwdParams& p, hipStream_t stream) {
  return use_small_tiles(p.N, p.BH) ? launch_fwd_waves<D, BLOCK_N, CAUSAL, 4, PREROT>(p, stream)
                                    : launch_fwd_waves<D, BLOCK_N, CAUSAL, 8, PREROT>(p, stream);
}

hipError_t launch_rope_attn_fwd(const FwdParams& p, int D, bool causal, hipStream_t stream) {
  // D = 256: four waves of 512 registers each, whatever the shape
  if (D == 256) return causal ? launch_fwd_waves<256, 64, true, 4>(p, stream) : launch_fwd_waves<256, 64, false, 4>(p, stream);
  if (D == 128) return causal ? launch_fwd_cfg<128, 64, true>(p, stream) : launch_fwd_cfg<128, 64, false>(p, stream);
  if (D != 64) return hipErrorInvalidValue;
  return causal ? launch_fwd_cfg<64, 64, true>(p, stream) : launch_fwd_cfg<64, 64, false>(p, stream);
}

// The same kernel on a key copy rotated beforehand (p.k_rot): no rotation and no table reads in its loop; it needs no key
// norms, and keeps the softmax bookkeeping of the single launch (probabilities in the tensors' own 16-bit type).
hipError_t launch_rope_attn_fwd_single_prerotated(const FwdParams& p, int D, bool causal, hipStream_t stream) {
  if (D == 256) return causal ? launch_fwd_waves<256, 64, true, 4, true>(p, stream) : launch_fwd_waves<256, 64, false, 4, true>(p, stream);
  if (D == 128) return causal ? launch_fwd_cfg<128, 64, true, true>(p, stream) : launch_fwd_cfg<128, 64, false, true>(p, stream);
  if (D != 64) return hipErrorInvalidValue;
  return causal ? launch_fwd_cfg<64, 64, true, true>(p, stream) : launch_fwd_cfg<64, 64, false, true>(p, stream);
}

}  // namespace COROPE_NS
