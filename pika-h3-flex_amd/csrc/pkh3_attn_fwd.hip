// Non-causal flash-style attention forward for gfx950 (CDNA4), head dim 128.
//
// Work split.  A workgroup is 4 waves (one per SIMD); each wave owns 64 queries of one (batch, head)
// and keeps for them, in registers, the Q operand images, the running row max / row sum and the
// fp32 output accumulator O^T (128 x 64).  The 4 waves share every 64-key K/V tile, which is copied
// HBM/L2 -> LDS with direct-to-LDS loads into a ring of buffers, one tile ahead of the math.
//
// Math per tile, all on the 32x32 MFMA shapes (see pkh3_common.h for the operand images):
//   S^T = K' Q'^T      A = K image (LDS), B = Q image (VGPR)      -> lane l holds query l%32, 16 keys / block
//   online softmax     row max: in-lane over the keys + one exchange with lane l^32; exp2 with the
//                      softmax scale folded in; row sum kept per half-wave and merged once at the end
//   O^T += V^T P^T     A = V image (LDS), B = P packed to bf16 straight from the S^T registers
// The transposed formulation keeps every per-query quantity (max, sum, rescale factor) a per-lane
// scalar: no cross-lane traffic in the rescale, none between the two GEMMs.
#include "pkh3_common.h"
#include "pkh3_internal.h"

namespace pkh3 {

constexpr int kWaves = 4;
constexpr int kQPerWave = 64;                     // 2 query blocks of 32
constexpr int kQPerWg = kWaves * kQPerWave;       // 256
constexpr int kNBuf = 3;                          // LDS ring depth
constexpr int kKvTileBytes = kKTileBytes + kVTileBytes;  // 32 KiB per tile (bf16 K)

__device__ __forceinline__ void lds_dma16(const char* g, char* l) {
  // 64 lanes x 16 B, global -> LDS without passing through VGPRs; LDS address = l + lane*16
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                   (__attribute__((address_space(3))) void*)l, 16, 0, 0);
}

// Issue this wave's quarter of one [K|V] tile copy.
__device__ __forceinline__ void prefetch_tile(const char* tile, char* buf, int wave, int lane) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int chunk = wave * 8 + i;
    lds_dma16(tile + chunk * 1024 + lane * 16, buf + chunk * 1024);
  }
}

__global__ __launch_bounds__(256, 1) void attn_fwd_dense_kernel(FwdParams p) {
  __shared__ __attribute__((aligned(1024))) char lds[kNBuf][kKvTileBytes];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int hh = lane >> 5;

  // Workgroups are handed to the 8 XCDs round-robin; give each XCD one contiguous run of
  // (batch, head, query tile) so the 32 CUs behind one L2 stream the same K/V at the same time.
  const int nQt = p.nQ64 / kWaves;
  const int total = p.B * p.H * nQt;
  const int per_xcd = (total + 7) / 8;
  const int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (lin >= total) return;
  const int bh = lin / nQt, qt = lin % nQt;
  const int b = bh / p.H, h = bh % p.H;

  const int sk = p.row_cnt ? p.row_cnt[b] : p.Sk;
  const int nt = (sk + kTileKeys - 1) / kTileKeys;
  const char* kv = p.kv + (int64_t)bh * p.kv_bh_stride;

  if (nt > 0) prefetch_tile(kv, lds[0], wave, lane);

  // Q images for this wave's 64 queries
  const int q64 = qt * kWaves + wave;
  bf16x8 qf[2][8];
  {
    const bf16x8* qsrc = (const bf16x8*)(p.qp + (int64_t)bh * p.q_bh_stride + (int64_t)q64 * p.q_blk_stride);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) qf[qb][ks] = qsrc[(qb * 8 + ks) * 64 + lane];
  }

  f32x16 o[2][4];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
  float m[2] = {-INFINITY, -INFINITY};
  float l[2] = {0.f, 0.f};
  const float c = p.c;

  for (int t = 0; t < nt; ++t) {
    // tile t has landed (this wave's part: vmcnt; everyone's: barrier); the barrier also says every
    // wave is done reading the buffer tile t+1 goes into (it held tile t-2).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t + 1 < nt) prefetch_tile(kv + (int64_t)(t + 1) * p.kv_tile_stride, lds[(t + 1) % kNBuf], wave, lane);
    const char* kbuf = lds[t % kNBuf];
    const char* vbuf = kbuf + kKTileBytes;

    f32x16 s[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[qb][kb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 kf = *(const bf16x8*)(kbuf + ((kb * 8 + ks) * 64 + lane) * 16);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          s[qb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], s[qb][kb], 0, 0, 0);
      }
    }

    if (t == nt - 1 && (sk & (kTileKeys - 1))) {
      const int lim = sk - t * kTileKeys;  // keys of this tile that exist
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kb * 32 + 8 * (i / 4) + 4 * hh + (i % 4);
          if (key >= lim) {
            s[0][kb][i] = -INFINITY;
            s[1][kb][i] = -INFINITY;
          }
        }
    }

    bf16x8 pf[2][2][2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float mx = s[qb][0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[qb][kb][i]);
      mx = fmaxf(mx, xhalf(mx));
      const float m_new = fmaxf(m[qb], mx * c);
      const float alpha = __builtin_amdgcn_exp2f(m[qb] - m_new);
      m[qb] = m_new;
      float rsum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int b2 = 0; b2 < 2; ++b2)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float e = __builtin_amdgcn_exp2f(fmaf(s[qb][kb][8 * b2 + j], c, -m_new));
            rsum += e;
            pf[qb][kb][b2][j] = (__bf16)e;
          }
      l[qb] = l[qb] * alpha + rsum;
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha;
      }
    }

#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int b2 = 0; b2 < 2; ++b2)
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const bf16x8 vf = *(const bf16x8*)(vbuf + (((kb * 2 + b2) * 4 + db) * 64 + lane) * 16);
#pragma unroll
          for (int qb = 0; qb < 2; ++qb)
            o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qb][kb][b2], o[qb][db], 0, 0, 0);
        }
  }

  // epilogue: O = O^T / l, bf16, 8-byte stores (4 consecutive d per register group)
  __bf16* ob = (__bf16*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const float lt = l[qb] + xhalf(l[qb]);
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    const int q = q64 * 64 + qb * 32 + (lane & 31);
    if (q < p.Sq) {
      __bf16* orow = ob + (int64_t)q * p.o_ss;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          bf16x4 w;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) w[rr] = (__bf16)(o[qb][db][4 * g + rr] * inv);
          *(bf16x4*)(orow + 32 * db + 8 * g + 4 * hh) = w;
        }
    }
  }
}

hipError_t launch_attn_fwd(const FwdParams& p, hipStream_t st) {
  const int nQt = p.nQ64 / kWaves;
  const int total = p.B * p.H * nQt;
  const int per_xcd = (total + 7) / 8;
  hipLaunchKernelGGL(attn_fwd_dense_kernel, dim3(per_xcd * 8), dim3(256), 0, st, p);
  return hipGetLastError();
}

}  // namespace pkh3
