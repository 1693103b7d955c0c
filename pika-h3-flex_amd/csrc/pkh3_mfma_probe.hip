// Roofline calibration probe: how fast does this GPU run a dependency-free stream of bf16 32x32x16 MFMAs
// (8 waves per CU, no memory traffic) when the operands are (a) all ones and (b) random values?
// The published 2.5 PFLOP/s bf16 dense figure corresponds to the boost clock; with operands that
// toggle every bit the part is power-limited and clocks lower.  The number under (b) is the practical
// ceiling any bf16 MFMA kernel with real data can reach on the box.
//
// Usage: pkh3_mfma_probe [iterations]     prints two JSON lines.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ unsigned mix(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

template <bool RANDOM>
__global__ __launch_bounds__(512) void mfma_stream(float* out, int iters) {
  bf16x8 a[8], b[8];
  for (int n = 0; n < 8; ++n)
    for (int j = 0; j < 8; ++j) {
      const unsigned h1 = mix(threadIdx.x * 131u + n * 17u + j), h2 = mix(h1 + 12345u);
      a[n][j] = RANDOM ? (__bf16)(((h1 & 0xffff) / 16384.0f) - 2.0f) : (__bf16)1.0f;
      b[n][j] = RANDOM ? (__bf16)(((h2 & 0xffff) / 16384.0f) - 2.0f) : (__bf16)1.0f;
    }
  f32x16 acc[4];
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) acc[n][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int n = 0; n < 4; ++n) acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b[(r + n) & 7], acc[n], 0, 0, 0);
  }
  float s = 0.f;
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) s += acc[n][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

#define CK(x)                                                                   \
  do {                                                                          \
    hipError_t e_ = (x);                                                        \
    if (e_ != hipSuccess) {                                                     \
      fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      return 1;                                                                 \
    }                                                                           \
  } while (0)

int main(int argc, char** argv) {
  const int iters = argc > 1 ? atoi(argv[1]) : 50000;
  hipDeviceProp_t prop;
  CK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  float* out;
  CK(hipMalloc(&out, (size_t)cus * 512 * sizeof(float)));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int random = 0; random < 2; ++random) {
    for (int rep = 0; rep < 2; ++rep) {  // first repetition warms up
      CK(hipEventRecord(e0));
      if (random)
        hipLaunchKernelGGL(mfma_stream<true>, dim3(cus), dim3(512), 0, 0, out, iters);
      else
        hipLaunchKernelGGL(mfma_stream<false>, dim3(cus), dim3(512), 0, 0, out, iters);
      CK(hipGetLastError());
      CK(hipEventRecord(e1));
      CK(hipEventSynchronize(e1));
      float ms = 0.f;
      CK(hipEventElapsedTime(&ms, e0, e1));
      const double flop = (double)cus * 8 * iters * 32 * (2.0 * 32 * 32 * 16);
      if (rep == 1)
        printf("{\"probe\": \"mfma_f32_32x32x16_bf16 stream\", \"operands\": \"%s\", \"cus\": %d, \"waves_per_cu\": 8, "
               "\"ms\": %.3f, \"tflops\": %.1f}\n", random ? "random" : "ones", cus, ms, flop / ms / 1e9);
    }
  }
  CK(hipFree(out));
  return 0;
}
