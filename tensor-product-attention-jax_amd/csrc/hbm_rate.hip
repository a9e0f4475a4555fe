// Sustained HBM rates of a gfx950 device, as a yardstick for the decode kernels: a plain read of a
// buffer much larger than the 256 MB memory-side cache (16-byte non-temporal loads, two in flight per
// lane, the values folded into one word per lane so that nothing is written back) and a plain copy
// (16-byte loads and stores).  No arithmetic, no LDS: nothing but the memory system limits them.
// Three workgroups of four waves per CU: of the launch shapes tried (1 to 16 workgroups of 256 to 1024
// threads per CU, 1 to 8 loads in flight) this one read fastest (6.9-7.1 TB/s; 5.4-6.0 with 8 or more
// workgroups per CU or with four loads in flight at strides that are powers of two).
//
//   hbm_rate [MiB per buffer, default 2048]
//
// prints one JSON line: {"read_gbs": ..., "copy_gbs": ..., "mib": ...}   (copy_gbs counts bytes read + written)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#define CHECK(call)                                                                          \
  do {                                                                                       \
    hipError_t e_ = (call);                                                                  \
    if (e_ != hipSuccess) {                                                                  \
      fprintf(stderr, "hbm_rate: %s failed: %s\n", #call, hipGetErrorString(e_));            \
      return 1;                                                                              \
    }                                                                                        \
  } while (0)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256, kInFlight = 2;

__global__ void __launch_bounds__(kThreads) read_kernel(const u32x4* in, uint32_t* out, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  u32x4 acc = {0, 0, 0, 0};
  // the grid covers n16 in whole rounds of kInFlight loads per lane (the host rounds n16 down accordingly)
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n16; i += stride * kInFlight) {
    u32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) v[u] = __builtin_nontemporal_load(in + i + u * stride);
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) acc ^= v[u];
  }
  out[(int64_t)blockIdx.x * kThreads + threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}

__global__ void __launch_bounds__(kThreads) copy_kernel(const u32x4* in, u32x4* out, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n16; i += stride * kInFlight) {
    u32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) v[u] = in[i + u * stride];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) out[i + u * stride] = v[u];
  }
}

int main(int argc, char** argv) {
  const int mib = argc > 1 ? atoi(argv[1]) : 2048;
  if (mib < 64 || mib > 8192) {
    fprintf(stderr, "usage: hbm_rate [MiB per buffer, 64..8192]\n");
    return 2;
  }
  const int blocks = 256 * 3;  // three workgroups of four waves per CU
  const int64_t round = (int64_t)blocks * kThreads * kInFlight;
  const int64_t n16 = ((int64_t)mib << 20) / 16 / round * round;  // whole rounds only: no tail, no bounds checks inside
  uint8_t *a = nullptr, *b = nullptr;
  uint32_t* sink = nullptr;
  CHECK(hipMalloc(&a, (size_t)mib << 20));
  CHECK(hipMalloc(&b, (size_t)mib << 20));
  CHECK(hipMalloc(&sink, (size_t)blocks * kThreads * sizeof(uint32_t)));
  CHECK(hipMemset(a, 0x5a, (size_t)mib << 20));
  CHECK(hipMemset(b, 0xa5, (size_t)mib << 20));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  const int reps = 10;
  float ms_read = 0.f, ms_copy = 0.f;
  for (int r = 0; r < 2; ++r) hipLaunchKernelGGL(read_kernel, dim3(blocks), dim3(kThreads), 0, 0, reinterpret_cast<const u32x4*>(r & 1 ? b : a), sink, n16);
  CHECK(hipDeviceSynchronize());
  CHECK(hipEventRecord(e0));
  for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(read_kernel, dim3(blocks), dim3(kThreads), 0, 0, reinterpret_cast<const u32x4*>(r & 1 ? b : a), sink, n16);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  CHECK(hipEventElapsedTime(&ms_read, e0, e1));
  for (int r = 0; r < 2; ++r) hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(kThreads), 0, 0, reinterpret_cast<const u32x4*>(a), reinterpret_cast<u32x4*>(b), n16);
  CHECK(hipDeviceSynchronize());
  CHECK(hipEventRecord(e0));
  for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(kThreads), 0, 0, reinterpret_cast<const u32x4*>(a), reinterpret_cast<u32x4*>(b), n16);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  CHECK(hipEventElapsedTime(&ms_copy, e0, e1));
  CHECK(hipGetLastError());
  const double bytes = (double)n16 * 16;
  printf("{\"read_gbs\": %.1f, \"copy_gbs\": %.1f, \"mib\": %d}\n", bytes * reps / ms_read / 1e6, 2 * bytes * reps / ms_copy / 1e6, mib);
  CHECK(hipFree(a));
  CHECK(hipFree(b));
  CHECK(hipFree(sink));
  return 0;
}
