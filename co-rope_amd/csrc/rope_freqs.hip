// cos/sin tables for the half-layout rotation, generated on the device.
//
// Device counterpart of the reference's precompute_freqs_cis (fused-rope/rope_attn_pytorch.py:10-49): theta_i =
// theta^(-2i/D) evaluated like the reference's fp32 expression, angle = position * theta_i in fp32, tables of
// `width` columns (D for the reference's duplicated-half layout, D/2 for the compact one the kernels read).
// `pos0` is the position of the first row, so a shard or a decode step can ask for its own slice of positions.
#include "common.hpp"
#include "kernels.hpp"

namespace corope {

struct InvFreqs {
  float w[128];  // theta^(-2i/D), evaluated on the host with the reference's fp32 expression
};

__global__ __launch_bounds__(256) void rope_freqs_kernel(float* __restrict__ cosp, float* __restrict__ sinp, int n_pos,
                                                         int D, int width, int64_t row_stride, int pos0, InvFreqs fr) {
  const int half = D / 2;
  const int idx = blockIdx.x * 256 + threadIdx.x;   // one (position, frequency) pair per thread
  if (idx >= n_pos * half) return;
  const int row = idx / half, i = idx % half;
  const float ang = (float)(pos0 + row) * fr.w[i];
  const float c = cosf(ang), s = sinf(ang);
  float* cr = cosp + (int64_t)row * row_stride;
  float* sr = sinp + (int64_t)row * row_stride;
  cr[i] = c;
  sr[i] = s;
  if (width >= D) {
    cr[i + half] = c;
    sr[i + half] = s;
  }
}

hipError_t launch_rope_freqs(float* cosp, float* sinp, int n_pos, int D, int width, int64_t row_stride, int pos0,
                             float theta, hipStream_t stream) {
  const int total = n_pos * (D / 2);
  InvFreqs fr{};
  for (int i = 0; i < D / 2; ++i) fr.w[i] = 1.0f / powf(theta, (float)(2 * i) / (float)D);
  hipLaunchKernelGGL(rope_freqs_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, cosp, sinp, n_pos, D, width,
                     row_stride, pos0, fr);
  return hipGetLastError();
}

}  // namespace corope
