// Half-layout rotation of a whole (B*H, N, D) bf16 tensor, written back as bf16, plus the largest row norm of
// every 64-row tile.
//
// The rotation is the reference's apply_rotary_emb (fused-rope/rope_attn_pytorch.py:71-84, rotate_half :52-68; in-kernel form
// fused-rope/fused_rope_attn.py:82-99): y1 = x1 cos - x2 sin, y2 = x2 cos + x1 sin on the two halves of a row,
// evaluated in fp32 and rounded to bf16 once -- bit for bit what the attention kernels produce when they rotate a
// tile themselves.  A K tile is needed by every query block of its head, so for long sequences rotating K once
// here costs one extra pass over K (HBM-bound) and removes N / 256 repeated rotations -- and their fp32 table
// reads -- from the attention kernel's inner loop.
//
// out_scale != 1: y = out_scale * rotated x, still one rounding -- the form in which the backward kernels and the
// two-launch forward take a pre-rotated Q (out_scale = sm_scale * log2(e)).
//
// tile_max[bh][t] = max over the rows of tile t of |y| (norm of the ROUNDED row).  With the norm of a query this
// bounds every score of the tile, which lets the forward kernel pick its softmax mode per tile up front.
#include "common.hpp"
#include "kernels.hpp"

namespace COROPE_NS {

constexpr int kRotRows = 64;
constexpr int kRotThreads = 256;

template <int D, bool SCALED>
__global__ __launch_bounds__(kRotThreads) void rope_rotate_kernel(const uint16_t* __restrict__ x,
                                                                  const float* __restrict__ cosp,
                                                                  const float* __restrict__ sinp, int64_t fstride,
                                                                  uint16_t* __restrict__ y, float* __restrict__ tile_max,
                                                                  int N, int n_tiles, float out_scale, int H, int64_t x_sb,
                                                                  int64_t x_sh, int x_sn) {
  using Stage = RotStage<D, kRotRows, kRotThreads, SCALED>;
  constexpr int kChunks = Stage::kChunks;
  __shared__ float wave_max[kRotThreads / kWave];
  const int tile = blockIdx.x % n_tiles, bh = blockIdx.x / n_tiles;
  const int row0 = tile * kRotRows;
  const uint16_t* xg = x + (bh / H) * x_sb + (bh % H) * x_sh;   // the source may be a strided view; y is contiguous
  uint16_t* yg = y + (int64_t)bh * N * D;

  Stage st;
  st.out_scale = out_scale;
  st.load(xg, cosp, sinp, fstride, row0, N, (uint32_t)x_sn * 2);
  float best = 0.f;
#pragma unroll
  for (int it = 0; it < Stage::kIters; ++it) {
    const int u = threadIdx.x + it * kRotThreads;
    const int r = u / kChunks, ch = u % kChunks;
    u32x4 y1, y2;
    st.rotate(it, y1, y2);
    float ss = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float a0 = elt_lo(y1[w]), a1 = elt_hi(y1[w]), b0 = elt_lo(y2[w]), b1 = elt_hi(y2[w]);
      ss += (a0 * a0 + a1 * a1) + (b0 * b0 + b1 * b1);
    }
    // the kChunks lanes of a row are consecutive
#pragma unroll
    for (int m = 1; m < kChunks; m *= 2) ss += __shfl_xor(ss, m);
    if (row0 + r < N) {
      uint16_t* dst = yg + (int64_t)(row0 + r) * D + ch * 8;
      *reinterpret_cast<u32x4*>(dst) = y1;
      *reinterpret_cast<u32x4*>(dst + D / 2) = y2;
      best = fmaxf(best, ss);
    }
  }
  if (tile_max == nullptr) return;
#pragma unroll
  for (int m = kChunks; m < kWave; m *= 2) best = fmaxf(best, __shfl_xor(best, m));
  if (threadIdx.x % kWave == 0) wave_max[threadIdx.x / kWave] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = wave_max[0];
#pragma unroll
    for (int w = 1; w < kRotThreads / kWave; ++w) m = fmaxf(m, wave_max[w]);
    tile_max[(int64_t)bh * n_tiles + tile] = __builtin_sqrtf(m);
  }
}

hipError_t launch_rope_rotate(const uint16_t* x, const float* cosp, const float* sinp, int64_t fstride, uint16_t* y,
                              float* tile_max, int BH, int N, int D, hipStream_t stream, float out_scale, int H, int64_t x_sb,
                              int64_t x_sh, int x_sn) {
  if (D != 64 && D != 128 && D != 256) return hipErrorInvalidValue;
  if (x_sn == 0) {   // contiguous (BH, N, D)
    H = 1;
    x_sb = (int64_t)N * D;
    x_sh = 0;
    x_sn = D;
  }
  const int n_tiles = (N + kRotRows - 1) / kRotRows;
  dim3 grid((unsigned)n_tiles * BH);   // one axis: the second grid axis stops at 65535 slabs
#define COROPE_ROT(DD, SS)                                                                                             \
  hipLaunchKernelGGL((rope_rotate_kernel<DD, SS>), grid, dim3(kRotThreads), 0, stream, x, cosp, sinp, fstride, y, tile_max, \
                     N, n_tiles, out_scale, H, x_sb, x_sh, x_sn)
  if (D == 256) {
    if (out_scale == 1.f) COROPE_ROT(256, false); else COROPE_ROT(256, true);
  } else if (D == 128) {
    if (out_scale == 1.f) COROPE_ROT(128, false); else COROPE_ROT(128, true);
  } else {
    if (out_scale == 1.f) COROPE_ROT(64, false); else COROPE_ROT(64, true);
  }
#undef COROPE_ROT
  return hipGetLastError();
}

}  // namespace COROPE_NS
