// Sustained rate of the bf16 matrix cores of a gfx950 device, as a yardstick for the attention and
// projection kernels: every wave keeps eight independent accumulation chains of
// v_mfma_f32_32x32x16_bf16 busy and touches no memory inside the loop, so nothing but the matrix pipe
// (and the power it draws) limits it.  Operands are N(0, 1) values rounded to bf16, or zeros: the rate
// depends on the data, because the device lowers its clock under the power that switching operands
// draw.
//
//   mfma_rate [waves_per_simd 1|2] [zeros 0|1] [workgroups] [iterations]      (defaults: 2 0 256 16384)
//
// prints one JSON line: {"tflops": ..., "us_per_launch": ..., "waves_per_simd": ..., "zeros": ..., ...}
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

#define CHECK(call)                                                                          \
  do {                                                                                       \
    hipError_t e_ = (call);                                                                  \
    if (e_ != hipSuccess) {                                                                  \
      fprintf(stderr, "mfma_rate: %s failed: %s\n", #call, hipGetErrorString(e_));           \
      return 1;                                                                              \
    }                                                                                        \
  } while (0)

constexpr int kChains = 8;

__global__ void __launch_bounds__(512) mfma_rate_kernel(const uint4* in, float* out, int iters) {
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  const uint4* p = in + (int64_t)gid * 8;
  bf16x8 a[4], b[2];
#pragma unroll
  for (int j = 0; j < 4; ++j) a[j] = __builtin_bit_cast(bf16x8, p[j]);
#pragma unroll
  for (int j = 0; j < 2; ++j) b[j] = __builtin_bit_cast(bf16x8, p[4 + j]);
  f32x16 acc[kChains];
#pragma unroll
  for (int n = 0; n < kChains; ++n)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[n][v] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < kChains; ++n) acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[n & 3], b[n >> 2], acc[n], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int n = 0; n < kChains; ++n)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[n][v];
  out[gid] = s;
}

int main(int argc, char** argv) {
  const int waves_per_simd = argc > 1 ? atoi(argv[1]) : 2;
  const int zeros = argc > 2 ? atoi(argv[2]) : 0;
  const int blocks = argc > 3 ? atoi(argv[3]) : 256;
  const int iters = argc > 4 ? atoi(argv[4]) : 16384;
  if ((waves_per_simd != 1 && waves_per_simd != 2) || blocks < 1 || blocks > 65536 || iters < 1 || iters > (1 << 22)) {
    fprintf(stderr, "usage: mfma_rate [waves_per_simd 1|2] [zeros 0|1] [workgroups 1..65536] [iterations 1..4194304]\n");
    return 2;
  }
  const int threads = 256 * waves_per_simd;  // four SIMDs per CU
  const size_t lanes = (size_t)blocks * threads;
  std::vector<uint32_t> h(lanes * 8 * 4, 0u);
  if (!zeros) {
    uint64_t state = 0x9e3779b97f4a7c15ull;
    auto uniform = [&]() {  // xorshift64*, top 24 bits
      state ^= state >> 12; state ^= state << 25; state ^= state >> 27;
      return (float)((state * 0x2545f4914f6cdd1dull) >> 40) * (1.f / 16777216.f);
    };
    auto normal_bf16 = [&]() -> uint32_t {  // sum of twelve uniforms: close enough to N(0, 1) for bit statistics
      float f = -6.f;
      for (int j = 0; j < 12; ++j) f += uniform();
      union { float f; uint32_t u; } c;
      c.f = f;
      return (c.u + 0x7fffu + ((c.u >> 16) & 1u)) >> 16;
    };
    for (auto& v : h) v = normal_bf16() | (normal_bf16() << 16);
  }
  uint4* in = nullptr;
  float* out = nullptr;
  CHECK(hipMalloc(&in, h.size() * sizeof(uint32_t)));
  CHECK(hipMalloc(&out, lanes * sizeof(float)));
  CHECK(hipMemcpy(in, h.data(), h.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  for (int r = 0; r < 3; ++r) hipLaunchKernelGGL(mfma_rate_kernel, dim3(blocks), dim3(threads), 0, 0, in, out, iters);
  CHECK(hipDeviceSynchronize());
  const int reps = 10;
  CHECK(hipEventRecord(e0));
  for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(mfma_rate_kernel, dim3(blocks), dim3(threads), 0, 0, in, out, iters);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  CHECK(hipGetLastError());
  float ms = 0.f;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  const double flop = (double)blocks * (threads / 64) * iters * kChains * 2.0 * 32 * 32 * 16 * reps;
  printf("{\"tflops\": %.1f, \"us_per_launch\": %.1f, \"waves_per_simd\": %d, \"zeros\": %d, \"workgroups\": %d, \"iterations\": %d}\n",
         flop / ms / 1e9, ms * 1e3 / reps, waves_per_simd, zeros ? 1 : 0, blocks, iters);
  CHECK(hipFree(in));
  CHECK(hipFree(out));
  return 0;
}
