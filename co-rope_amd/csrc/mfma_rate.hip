// Diagnostic program (not part of the library): what the gfx950 matrix pipes sustain on this machine.
//
// Loops of nothing but 32x32x16 bf16 MFMAs on all 256 CUs (8 waves each), with the A operand either held in registers
// or fetched from LDS as a fresh 1 KB fragment that feeds R MFMAs, on all-zero operands and on N(0,1) operands rounded to
// bf16.  Every run also measures the shader clock it ran at (core-clock counter against the constant 100 MHz counter),
// so the table shows how far the power management lowers the clock under the switching activity of real data: the
// figure to read the attention kernels' fractions of the published 2.5 PFLOP/s against.
//
//   build: python co-rope_amd/build.py        run: co-rope_amd/lib/mfma_rate
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

constexpr int kSrcWords = 65536;   // 16-byte words of operand data

template <int R, bool FROM_LDS>
__global__ __launch_bounds__(512) void mfma_loop(const u32x4* src, float* out, unsigned long long* clocks, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u32x4* tile = reinterpret_cast<u32x4*>(smem);   // 64 KB: 4096 x 16 B
  for (int e = threadIdx.x; e < 4096; e += 512) tile[e] = src[(blockIdx.x * 4096 + e) % kSrcWords];
  __syncthreads();
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  u32x4 b[R];
  f32x16 acc[R];
  for (int r = 0; r < R; ++r) {
    b[r] = src[(threadIdx.x * 7 + r * 13) % kSrcWords];
    acc[r] = f32x16{0};
  }
  u32x4 areg = src[(threadIdx.x * 3) % kSrcWords];
  const unsigned long long c0 = __builtin_readcyclecounter(), t0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int f = 0; f < 16; ++f) {
      u32x4 a = areg;
      if (FROM_LDS) a = tile[((wave * 16 + f + it) % 64) * 64 + lane];   // 1 KB per wave per fragment, conflict-free
#pragma unroll
      for (int r = 0; r < R; ++r)
        acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b[r]),
                                                         acc[r], 0, 0, 0);
    }
  }
  float s = 0;
  for (int r = 0; r < R; ++r)
    for (int i = 0; i < 16; ++i) s += acc[r][i];
  out[blockIdx.x * 512 + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clocks[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - t0;
  }
}

struct Result {
  double tflops, ghz;
};

template <int R, bool L>
Result run(const u32x4* src, float* out, unsigned long long* clocks, int iters) {
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(mfma_loop<R, L>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  for (int w = 0; w < 3; ++w) hipLaunchKernelGGL((mfma_loop<R, L>), dim3(256), dim3(512), 65536, 0, src, out, clocks, iters);
  (void)hipEventRecord(e0);
  for (int w = 0; w < 10; ++w) hipLaunchKernelGGL((mfma_loop<R, L>), dim3(256), dim3(512), 65536, 0, src, out, clocks, iters);
  (void)hipEventRecord(e1);
  (void)hipEventSynchronize(e1);
  float ms = 0;
  (void)hipEventElapsedTime(&ms, e0, e1);
  ms /= 10;
  std::vector<unsigned long long> h(512);
  (void)hipMemcpy(h.data(), clocks, h.size() * 8, hipMemcpyDeviceToHost);
  double ghz = 0;
  for (int i = 0; i < 256; ++i) ghz += (double)h[2 * i] / ((double)h[2 * i + 1] * 10.0) / 256;   // cycles per ns
  const double flop = 256.0 * 8 * iters * 16 * R * 32768.0;
  return {flop / (ms * 1e-3) * 1e-12, ghz};
}

int main() {
  u32x4* src;
  float* out;
  unsigned long long* clocks;
  if (hipMalloc(&src, kSrcWords * 16) != hipSuccess || hipMalloc(&out, 256 * 512 * 4) != hipSuccess ||
      hipMalloc(&clocks, 512 * 8) != hipSuccess) {
    fprintf(stderr, "mfma_rate: no HIP device\n");
    return 1;
  }
  const int iters = 2000;
  printf("| operands | A operand | MFMAs per fragment | TFLOP/s | of 2500 | shader clock GHz |\n|---|---|---|---|---|---|\n");
  for (int gaussian = 0; gaussian < 2; ++gaussian) {
    std::vector<unsigned> h(kSrcWords * 4, 0u);
    srand(1);
    auto gauss_bf16 = [&]() {   // N(0,1) rounded to bf16 (Box-Muller)
      float u1 = (rand() + 1.0f) / ((float)RAND_MAX + 2.0f), u2 = rand() / (float)RAND_MAX;
      float g = sqrtf(-2.f * logf(u1)) * cosf(6.2831853f * u2);
      unsigned bits;
      memcpy(&bits, &g, 4);
      return (bits + 0x8000u) >> 16;
    };
    if (gaussian)
      for (auto& x : h) x = gauss_bf16() | (gauss_bf16() << 16);
    (void)hipMemcpy(src, h.data(), h.size() * 4, hipMemcpyHostToDevice);
    for (int i = 0; i < 3; ++i) run<2, true>(src, out, clocks, iters);   // a long warm-up so that the clocks settle
    const char* name = gaussian ? "N(0,1) bf16" : "all zero";
    Result r;
    r = run<1, true>(src, out, clocks, iters);
    printf("| %s | LDS | 1 | %.0f | %.3f | %.2f |\n", name, r.tflops, r.tflops / 2500, r.ghz);
    r = run<2, true>(src, out, clocks, iters);
    printf("| %s | LDS | 2 | %.0f | %.3f | %.2f |\n", name, r.tflops, r.tflops / 2500, r.ghz);
    r = run<4, true>(src, out, clocks, iters);
    printf("| %s | LDS | 4 | %.0f | %.3f | %.2f |\n", name, r.tflops, r.tflops / 2500, r.ghz);
    r = run<2, false>(src, out, clocks, iters);
    printf("| %s | registers | - (2 accumulators) | %.0f | %.3f | %.2f |\n", name, r.tflops, r.tflops / 2500, r.ghz);
    r = run<4, false>(src, out, clocks, iters);
    printf("| %s | registers | - (4 accumulators) | %.0f | %.3f | %.2f |\n", name, r.tflops, r.tflops / 2500, r.ghz);
  }
  return hipGetLastError() == hipSuccess ? 0 : 1;
}
