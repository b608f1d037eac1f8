// delta[row] = sum_d O[row, d] * dO[row, d]  (fp32), the backward's preprocessing pass.
//
// Device counterpart of the reference's _attn_bwd_preprocess (fused-rope/fused_rope_attn.py:324-337).
// HBM-bound: reads 2 * rows * D bf16, writes rows fp32.  D/8 lanes share one row (16-byte loads), reduce with
// lane shuffles; every thread keeps kRowsPerThread independent row loads in flight.
#include "common.hpp"
#include "kernels.hpp"

namespace COROPE_NS {

template <int D>
__global__ __launch_bounds__(256) void bwd_preprocess_kernel(const uint16_t* __restrict__ o,
                                                             const uint16_t* __restrict__ d_o,
                                                             float* __restrict__ delta, int64_t rows) {
  constexpr int kLanesPerRow = D / 8;
  constexpr int kRowsPerPass = 256 / kLanesPerRow;
  constexpr int kRowsPerThread = 4;
  const int sub = threadIdx.x % kLanesPerRow;
  const int64_t base = (int64_t)blockIdx.x * (kRowsPerPass * kRowsPerThread) + threadIdx.x / kLanesPerRow;
  u32x4 a[kRowsPerThread], b[kRowsPerThread];
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    int64_t row = min(base + (int64_t)r * kRowsPerPass, rows - 1);
    a[r] = *reinterpret_cast<const u32x4*>(o + row * D + sub * 8);
    b[r] = *reinterpret_cast<const u32x4*>(d_o + row * D + sub * 8);
  }
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) acc += elt_lo(a[r][w]) * elt_lo(b[r][w]) + elt_hi(a[r][w]) * elt_hi(b[r][w]);
#pragma unroll
    for (int off = kLanesPerRow / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    int64_t row = base + (int64_t)r * kRowsPerPass;
    if (sub == 0 && row < rows) delta[row] = acc;
  }
}

hipError_t launch_bwd_preprocess(const BwdParams& p, int D, hipStream_t stream) {
  const int64_t rows = (int64_t)p.BH * p.N;
  if (D == 256) {
    constexpr int per_block = (256 / 32) * 4;
    hipLaunchKernelGGL(bwd_preprocess_kernel<256>, dim3((unsigned)((rows + per_block - 1) / per_block)), dim3(256), 0,
                       stream, p.o, p.d_o, p.delta, rows);
  } else if (D == 128) {
    constexpr int per_block = (256 / 16) * 4;
    hipLaunchKernelGGL(bwd_preprocess_kernel<128>, dim3((unsigned)((rows + per_block - 1) / per_block)), dim3(256), 0,
                       stream, p.o, p.d_o, p.delta, rows);
  } else {
    constexpr int per_block = (256 / 8) * 4;
    hipLaunchKernelGGL(bwd_preprocess_kernel<64>, dim3((unsigned)((rows + per_block - 1) / per_block)), dim3(256), 0,
                       stream, p.o, p.d_o, p.delta, rows);
  }
  return hipGetLastError();
}

}  // namespace COROPE_NS
