// Roofline calibration probe for the attention kernels: what does this GPU sustain on bf16 32x32x16 MFMA work,
// and at which core clock, when nothing but the matrix pipe (and, in the last case, the instruction mix of an
// attention tile) is in the way?
//
//   "ones"      dependency-free MFMA stream, all-ones operands, 8 waves per CU, no memory traffic
//   "random"    the same stream with random operands: every bit toggles, the part is power-limited and clocks lower
//   "lds"       the random-operand stream with the A operand of every MFMA read from LDS (one 1 KiB image per MFMA,
//               as the attention kernels do), 12 waves per CU, still no other instructions and no HBM traffic
//   "attention" 12 waves per CU walking an attention-shaped tile loop with no HBM traffic at all: 16 MFMAs whose A
//               operands are 1 KiB LDS images (two accumulate chains of 8, like S^T = K Q^T), 32 exp2 + 16 packed
//               bf16 conversions + 16 dot2 row sums, 16 more MFMAs with LDS A operands and the converted values
//               as B operands (like O^T += V^T P^T), one workgroup barrier per tile
//
// The published 2.5 PFLOP/s bf16 dense figure corresponds to every MFMA issue slot used at the boost clock.  The
// probe prints, for each case, the achieved rate, the average core clock over the run (core-clock counter against
// the 100 MHz wall-clock counter) and the share of MFMA issue slots used at that clock ("pipe").  "random" is the
// ceiling of any bf16 MFMA kernel with real data on the box; "lds" is what is left of it when the operands come
// through LDS (the reads cost power, the clock drops further); "attention" is the ceiling of this kernel structure
// before K/V streaming, Q/O traffic and softmax bookkeeping are added.
//
// Usage: pkh3_mfma_probe [iterations]     prints one JSON line per case.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ unsigned mix(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

__device__ bf16x8 random_image(unsigned seed) {
  bf16x8 r;
  for (int j = 0; j < 8; ++j) r[j] = (__bf16)(((mix(seed * 8u + j) & 0xffff) / 16384.0f) - 2.0f);
  return r;
}

struct Clocks {
  long long core, wall;  // ticks of the core clock / of the 100 MHz constant clock over the timed loop
};

__device__ void stamp(Clocks* clk, long long c0, long long w0) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    clk->core = clock64() - c0;
    clk->wall = wall_clock64() - w0;
  }
}

template <bool RANDOM>
__global__ __launch_bounds__(512) void mfma_stream(float* out, int iters, Clocks* clk) {
  bf16x8 a[8], b[8];
  for (int n = 0; n < 8; ++n)
    for (int j = 0; j < 8; ++j) {
      a[n][j] = RANDOM ? random_image(threadIdx.x * 131u + n * 17u)[j] : (__bf16)1.0f;
      b[n][j] = RANDOM ? random_image(threadIdx.x * 257u + n * 29u + 5u)[j] : (__bf16)1.0f;
    }
  f32x16 acc[4];
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) acc[n][i] = 0.f;
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int n = 0; n < 4; ++n) acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b[(r + n) & 7], acc[n], 0, 0, 0);
  }
  stamp(clk, c0, w0);
  float s = 0.f;
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) s += acc[n][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

constexpr int kAttnWaves = 12;

__global__ __launch_bounds__(64 * kAttnWaves, 1) void lds_fed_stream(float* out, int iters, Clocks* clk) {
  __shared__ __attribute__((aligned(1024))) char lds[32768];
  const int lane = threadIdx.x & 63;
  bf16x8 b[8];
  for (int n = 0; n < 8; ++n) b[n] = random_image(threadIdx.x * 31u + n);
  for (int i = threadIdx.x; i < 32768 / 16; i += 64 * kAttnWaves) ((bf16x8*)lds)[i] = random_image(i * 7u + 3u);
  __syncthreads();
  f32x16 acc[4];
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) acc[n][i] = 0.f;
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    asm volatile("" ::: "memory");  // the images are read again every iteration
    bf16x8 a[32];
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = *(const bf16x8*)(lds + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[i & 7], acc[i & 3], 0, 0, 0);
      if (i + 4 < 32) a[i + 4] = *(const bf16x8*)(lds + ((i + 4) * 64 + lane) * 16);
    }
    if ((it & 63) == 63) {
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[n][i] *= 1e-6f;
    }
  }
  stamp(clk, c0, w0);
  float s = 0.f;
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) s += acc[n][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

__global__ __launch_bounds__(64 * kAttnWaves, 1) void attention_shaped(float* out, int iters, Clocks* clk) {
  __shared__ __attribute__((aligned(1024))) char lds[32768];  // 16 "K" images, then 16 "V" images
  const int lane = threadIdx.x & 63;
  bf16x8 q[8];
  for (int n = 0; n < 8; ++n) q[n] = random_image(threadIdx.x * 31u + n);
  for (int i = threadIdx.x; i < 32768 / 16; i += 64 * kAttnWaves) ((bf16x8*)lds)[i] = random_image(i * 7u + 3u);
  __syncthreads();
  f32x16 o[4], s[2];
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) o[n][i] = 0.f;
  float l = 0.f;
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    __syncthreads();
    for (int kb = 0; kb < 2; ++kb)
      for (int i = 0; i < 16; ++i) s[kb][i] = 0.f;
    bf16x8 kf[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) kf[i] = *(const bf16x8*)(lds + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], q[i & 7], s[i >> 3], 0, 0, 0);
      if (i + 4 < 16) kf[i + 4] = *(const bf16x8*)(lds + ((i + 4) * 64 + lane) * 16);
    }
    bf16x8 pf[2][2];
    float rsum = 0.f;
    const bf16x2 one2 = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int b2 = 0; b2 < 2; ++b2) {
        bf16x8 pk;
        // logits of about +-1.5 in the log2 domain, like QK-normed attention
#pragma unroll
        for (int j = 0; j < 8; ++j) pk[j] = (__bf16)__builtin_amdgcn_exp2f(s[kb][8 * b2 + j] * 0.1f);
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
          const bf16x2 pr = {pk[j], pk[j + 1]};
          rsum = __builtin_amdgcn_fdot2_f32_bf16(pr, one2, rsum, false);
        }
        pf[kb][b2] = pk;
      }
    l += rsum;
    bf16x8 vg[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) vg[i] = *(const bf16x8*)(lds + 16384 + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      o[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vg[i], pf[i >> 3][(i >> 2) & 1], o[i & 3], 0, 0, 0);
      if (i + 4 < 16) vg[i + 4] = *(const bf16x8*)(lds + 16384 + ((i + 4) * 64 + lane) * 16);
    }
    if ((it & 63) == 63) {  // keep the accumulators finite over long runs
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[n][i] *= 1e-3f;
    }
  }
  stamp(clk, c0, w0);
  float t = l;
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) t += o[n][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = t;
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
  Clocks* clk;
  CK(hipMalloc(&out, (size_t)cus * 64 * kAttnWaves * sizeof(float)));
  CK(hipMalloc(&clk, sizeof(Clocks)));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  const char* names[4] = {"ones", "random", "lds", "attention"};
  for (int mode = 0; mode < 4; ++mode) {
    const int waves = mode >= 2 ? kAttnWaves : 8;
    float ms = 0.f;
    for (int rep = 0; rep < 2; ++rep) {  // first repetition warms up
      CK(hipEventRecord(e0));
      if (mode == 0) hipLaunchKernelGGL(mfma_stream<false>, dim3(cus), dim3(512), 0, 0, out, iters, clk);
      else if (mode == 1) hipLaunchKernelGGL(mfma_stream<true>, dim3(cus), dim3(512), 0, 0, out, iters, clk);
      else if (mode == 2) hipLaunchKernelGGL(lds_fed_stream, dim3(cus), dim3(64 * kAttnWaves), 0, 0, out, iters, clk);
      else hipLaunchKernelGGL(attention_shaped, dim3(cus), dim3(64 * kAttnWaves), 0, 0, out, iters, clk);
      CK(hipGetLastError());
      CK(hipEventRecord(e1));
      CK(hipEventSynchronize(e1));
      CK(hipEventElapsedTime(&ms, e0, e1));
    }
    Clocks h;
    CK(hipMemcpy(&h, clk, sizeof(h), hipMemcpyDeviceToHost));
    const double ghz = h.wall > 0 ? (double)h.core / ((double)h.wall / 100e6) / 1e9 : 0.0;
    const double flop = (double)cus * waves * iters * 32 * (2.0 * 32 * 32 * 16);
    const double tflops = flop / ms / 1e9;
    // MFMA issue slots used: 4 SIMDs x 512 FLOP per clock each when the pipe never idles
    const double pipe = ghz > 0 ? tflops * 1e12 / (cus * 4.0 * 2.0 * 32 * 32 * 16 / 32.0 * ghz * 1e9) : 0.0;
    printf("{\"probe\": \"mfma_f32_32x32x16_bf16\", \"operands\": \"%s\", \"cus\": %d, \"waves_per_cu\": %d, "
           "\"ms\": %.3f, \"tflops\": %.1f, \"core_clock_ghz\": %.3f, \"mfma_pipe_busy\": %.3f}\n",
           names[mode], cus, waves, ms, tflops, ghz, pipe);
  }
  CK(hipFree(out));
  CK(hipFree(clk));
  return 0;
}
