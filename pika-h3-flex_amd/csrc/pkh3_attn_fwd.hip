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
#include <stdlib.h>

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

// Per-wave register state.
struct WaveState {
  bf16x8 qf[2][8];      // Q images: [query block][k-step]
  f32x16 sa[2], sb[2];  // S^T of two consecutive 32-key sub-tiles (ping-pong), per query block
  bf16x8 pa[2][2], pb[2][2];  // P of two consecutive sub-tiles: [query block][k-step of 16 keys]
  f32x16 o[2][4];       // O^T accumulators: [query block][32-wide block of d]
  float m[2], l[2];     // running row max (scaled, log2 domain) and per-half-wave row sum
  float alpha[2];       // factor the last step lowered the old terms by (1 unless the max moved)
};

constexpr float kRescaleSlack = 8.0f;  // the running max is only raised when exceeded by 2^8

__device__ __forceinline__ float max_across_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// One pipeline step on 32-key sub-tiles, three independent instruction streams the scheduler may interleave:
//   MFMA:  S_next = K'(u+1) Q'^T        (16 MFMAs, K images from LDS at kptr)
//   MFMA:  O^T   += V(u-1)^T P_prev     (16 MFMAs, V images from LDS at vptr)           [DO_PV]
//   VALU:  P_cur = softmax numerators of S_cur (sub-tile u), running max / sum update
// `lim`: number of keys of sub-tile u that exist (only read when MASK).
template <bool DO_PV, bool MASK>
__device__ __forceinline__ void pipe_step(const char* kptr, const char* vptr, const bf16x8 (&qf)[2][8],
                                          const f32x16 (&s_cur)[2], f32x16 (&s_nxt)[2], const bf16x8 (&p_prev)[2][2],
                                          bf16x8 (&p_cur)[2][2], f32x16 (&o)[2][4], float (&m)[2], float (&l)[2],
                                          float (&alpha)[2], float c, int lim, int lane) {
  const int hh = lane >> 5;
  // ---- rescale O^T where the previous step moved the running max: after that step's P.V (sub-tile
  //      u-2), before this step's P.V (sub-tile u-1, whose numerators use the new max).  Rare.
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    if (__any(alpha[qb] != 1.0f)) {
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha[qb];
    }
  }
  // ---- QK^T of the next sub-tile
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    const bf16x8 kf = *(const bf16x8*)(kptr + (ks * 64 + lane) * 16);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      if (ks == 0) {
        f32x16 z;
#pragma unroll
        for (int i = 0; i < 16; ++i) z[i] = 0.f;
        s_nxt[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], z, 0, 0, 0);
      } else {
        s_nxt[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], s_nxt[qb], 0, 0, 0);
      }
    }
  }
  // ---- P.V of the previous sub-tile
  if constexpr (DO_PV) {
#pragma unroll
    for (int b2 = 0; b2 < 2; ++b2)
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const bf16x8 vf = *(const bf16x8*)(vptr + ((b2 * 4 + db) * 64 + lane) * 16);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p_prev[qb][b2], o[qb][db], 0, 0, 0);
      }
  }
  // ---- softmax numerators of the current sub-tile
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    f32x16 s = s_cur[qb];
    if constexpr (MASK) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = 8 * (i / 4) + 4 * hh + (i % 4);
        if (key >= lim) s[i] = -INFINITY;
      }
    }
    float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
    for (int i = 3; i < 15; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
    mx = fmaxf(mx, s[15]);
    mx = max_across_halves(mx) * c;
    // raise the running max only when it is exceeded by more than the slack: P stays <= 2^slack and
    // the O^T rescale below becomes rare
    const float m_old = m[qb];
    const float m_new = (mx > m_old + kRescaleSlack) ? mx : m_old;
    alpha[qb] = __builtin_amdgcn_exp2f(m_old - m_new);
    m[qb] = m_new;
    float rsum = 0.f;
#pragma unroll
    for (int b2 = 0; b2 < 2; ++b2) {
      bf16x8 pk;
#pragma unroll
      for (int j = 0; j < 8; ++j) pk[j] = (__bf16)__builtin_amdgcn_exp2f(fmaf(s[8 * b2 + j], c, -m_new));
      // row sum over the bf16-rounded values, the same numbers the P.V MFMA consumes
      const bf16x2 one2 = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const bf16x2 pr = {pk[j], pk[j + 1]};
        rsum = __builtin_amdgcn_fdot2_f32_bf16(pr, one2, rsum, false);
      }
      p_cur[qb][b2] = pk;
    }
    l[qb] = l[qb] * alpha[qb] + rsum;
  }
  // keep the numerators' computation inside this step (next to the MFMAs it overlaps with)
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int b2 = 0; b2 < 2; ++b2) asm volatile("" : "+v"(p_cur[qb][b2]));
  // register-file hints: the S^T results feed VALU work (VGPRs), O^T is only touched by MFMAs (AGPRs)
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) asm volatile("" : "+v"(s_nxt[qb]));
#ifdef PKH3_HINT_O_AGPR
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int db = 0; db < 4; ++db) asm volatile("" : "+a"(o[qb][db]));
#endif
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
  const int q64 = qt * kWaves + wave;

  const int sk = p.row_cnt ? p.row_cnt[b] : p.Sk;
  const int nt = (sk + kTileKeys - 1) / kTileKeys;
  const char* kv = p.kv + (int64_t)bh * p.kv_bh_stride;

  WaveState w;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) w.o[qb][db][i] = 0.f;
    w.m[qb] = -INFINITY;
    w.l[qb] = 0.f;
    w.alpha[qb] = 1.0f;
  }

  if (nt > 0) {
    prefetch_tile(kv, lds[0], wave, lane);
    {
      const bf16x8* qsrc = (const bf16x8*)(p.qp + (int64_t)bh * p.q_bh_stride + (int64_t)q64 * p.q_blk_stride);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) w.qf[qb][ks] = qsrc[(qb * 8 + ks) * 64 + lane];
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (nt > 1) prefetch_tile(kv + (int64_t)p.kv_tile_stride, lds[1], wave, lane);

    // pre-step: S_a = QK^T of sub-tile (0, 0)
    {
      const char* kptr = lds[0];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) w.sa[qb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 kf = *(const bf16x8*)(kptr + (ks * 64 + lane) * 16);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          w.sa[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, w.qf[qb][ks], w.sa[qb], 0, 0, 0);
      }
    }

    const float c = p.c;
    const int last_lim = sk - (nt - 1) * kTileKeys;  // keys that exist in the last tile (1..64)
    // Ring slots of tiles t-1, t, t+1.  Each iteration runs the two sub-tile steps of tile t:
    //   step (t,0): S_b = QK^T(t,1);   O += P_b V(t-1,1);  P_a = softmax(S_a)
    //   sync:       tile t+1 has landed (own part: vmcnt, everyone's: barrier); all waves are past
    //               V(t-1), so its slot takes tile t+2
    //   step (t,1): S_a = QK^T(t+1,0); O += P_a V(t,0);    P_b = softmax(S_b)
    // The first tile has no previous P.V and the last one masks the keys past the end; both are
    // peeled so that the steady-state loop body has no branches besides the rare O^T rescale.
    int buf_p = kNBuf - 1, buf = 0, buf_n = 1;
#define PKH3_TILE_ITER(T, DO_PV0, MASKED)                                                                         \
  {                                                                                                               \
    pipe_step<DO_PV0, MASKED>(lds[buf] + 8 * 1024, lds[buf_p] + kKTileBytes + 8 * 1024, w.qf, w.sa, w.sb, w.pb,   \
                              w.pa, w.o, w.m, w.l, w.alpha, c, last_lim, lane);                                            \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                              \
    __syncthreads();                                                                                              \
    if ((T) + 2 < nt) prefetch_tile(kv + (int64_t)((T) + 2) * p.kv_tile_stride, lds[buf_p], wave, lane);          \
    pipe_step<true, MASKED>(lds[buf_n], lds[buf] + kKTileBytes, w.qf, w.sb, w.sa, w.pa, w.pb, w.o, w.m, w.l,      \
                            w.alpha, c, last_lim - 32, lane);                                                                 \
    buf_p = buf;                                                                                                  \
    buf = buf_n;                                                                                                  \
    buf_n = buf_n + 1 == kNBuf ? 0 : buf_n + 1;                                                                   \
  }
    if (nt == 1) {
      PKH3_TILE_ITER(0, false, true)
    } else {
      PKH3_TILE_ITER(0, false, false)
      for (int t = 1; t < nt - 1; ++t) PKH3_TILE_ITER(t, true, false)
      PKH3_TILE_ITER(nt - 1, true, true)
    }
#undef PKH3_TILE_ITER
    // drain: O += P_b V(nt-1, 1)
    {
      const char* vptr = lds[buf_p] + kKTileBytes + 8 * 1024;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) w.o[qb][db][i] *= w.alpha[qb];
#pragma unroll
      for (int b2 = 0; b2 < 2; ++b2)
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const bf16x8 vf = *(const bf16x8*)(vptr + ((b2 * 4 + db) * 64 + lane) * 16);
#pragma unroll
          for (int qb = 0; qb < 2; ++qb)
            w.o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, w.pb[qb][b2], w.o[qb][db], 0, 0, 0);
        }
    }
  }

  // epilogue: O = O^T / l, bf16, 8-byte stores (4 consecutive d per register group)
  __bf16* ob = (__bf16*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const float lt = w.l[qb] + xhalf(w.l[qb]);
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    const int q = q64 * 64 + qb * 32 + (lane & 31);
    if (q < p.Sq) {
      __bf16* orow = ob + (int64_t)q * p.o_ss;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          bf16x4 wv;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) wv[rr] = (__bf16)(w.o[qb][db][4 * g + rr] * inv);
          *(bf16x4*)(orow + 32 * db + 8 * g + 4 * hh) = wv;
        }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Variant: 8 waves (two per SIMD), 32 queries per wave.  The two waves that share a SIMD run the
// same per-tile work in opposite phase ("ping-pong"): after each workgroup barrier the waves of
// group A start with the QK^T MFMAs of tile t while the waves of group B start with the softmax
// VALU work of tile t (whose S^T they computed before the barrier), so the matrix pipe and the
// vector pipe of every SIMD are both fed from the first cycle after the barrier on.
struct W8State {
  bf16x8 qf[8];
  f32x16 s[2];
  f32x16 o[4];
  bf16x8 vf[8];  // V images of the first 32 keys of the tile, fetched while QK^T finishes
  float m, l;
};

#define PKH3_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
constexpr int kSgMfma = 0x008, kSgDsRead = 0x100, kSgValu = 0x002, kSgTrans = 0x400;

// S^T = K' Q'^T for the 64 keys of one tile.  LDS reads run 8 images (8 KiB per wave) ahead of the
// MFMAs that consume them; the tail of the MFMA chain covers the first V image reads.
#ifdef ABL_NOLDS
#define LDSRD(ptr) (w.qf[1])
#else
#define LDSRD(ptr) (*(const bf16x8*)(ptr))
#endif
__device__ __forceinline__ void w8_qk(W8State& w, const char* kbuf, const char* vbuf, int lane) {
  bf16x8 kf[16];
#pragma unroll
  for (int i = 0; i < 8; ++i) kf[i] = LDSRD(kbuf + (i * 64 + lane) * 16);
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) w.s[kb][i] = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int kb = i >> 3, ks = i & 7;
    w.s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], w.qf[ks], w.s[kb], 0, 0, 0);
    if (i < 8)
      kf[i + 8] = LDSRD(kbuf + ((i + 8) * 64 + lane) * 16);
    else
      w.vf[i - 8] = LDSRD(vbuf + ((i - 8) * 64 + lane) * 16);
  }
  PKH3_SGB(kSgDsRead, 8);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    PKH3_SGB(kSgMfma, 1);
    PKH3_SGB(kSgDsRead, 1);
  }
}

// softmax numerators of w.s (lim = keys of this tile that exist; only read when it is < 64), then O^T += V^T P^T
__device__ __forceinline__ void w8_softmax_pv(W8State& w, const char* vbuf, float c, int lim, int lane) {
  const int hh = lane >> 5;
  if (lim < kTileKeys) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = kb * 32 + 8 * (i / 4) + 4 * hh + (i % 4);
        if (key >= lim) w.s[kb][i] = -INFINITY;
      }
  }
#ifdef ABL_NOMAX
  float mx = w.s[0][0];
#else
  float mx = fmaxf(w.s[0][0], w.s[1][0]);
#pragma unroll
  for (int i = 1; i < 16; ++i) mx = fmaxf(fmaxf(mx, w.s[0][i]), w.s[1][i]);
  mx = max_across_halves(mx) * c;
#endif
  const float m_new = (mx > w.m + kRescaleSlack) ? mx : w.m;
  const float alpha = __builtin_amdgcn_exp2f(w.m - m_new);
  w.m = m_new;
  if (__any(alpha != 1.0f)) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) w.o[db][i] *= alpha;
  }
  bf16x8 pf[2][2];
  float rsum = 0.f;
  const bf16x2 one2 = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int b2 = 0; b2 < 2; ++b2) {
      bf16x8 pk;
#pragma unroll
#ifdef ABL_NOEXP
      for (int j = 0; j < 8; ++j) pk[j] = (__bf16)(w.s[kb][8 * b2 + j]);
#else
      for (int j = 0; j < 8; ++j) pk[j] = (__bf16)__builtin_amdgcn_exp2f(fmaf(w.s[kb][8 * b2 + j], c, -m_new));
#endif
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const bf16x2 pr = {pk[j], pk[j + 1]};
        rsum = __builtin_amdgcn_fdot2_f32_bf16(pr, one2, rsum, false);
      }
      pf[kb][b2] = pk;
    }
  w.l = w.l * alpha + rsum;
  bf16x8 vg[8];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int kb = i >> 3, b2 = (i >> 2) & 1, db = i & 3;
    w.o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(i < 8 ? w.vf[i] : vg[i - 8], pf[kb][b2], w.o[db], 0, 0, 0);
    if (i < 8) vg[i] = LDSRD(vbuf + ((i + 8) * 64 + lane) * 16);
  }
}

template <bool DMA>
__global__ __launch_bounds__(512, 1) void attn_fwd_w8_kernel(FwdParams p) {
  __shared__ __attribute__((aligned(1024))) char lds[DMA ? 3 : 2][kKvTileBytes];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int hh = lane >> 5;
  const int nQt = p.nQ64 / kWaves;
  const int total = p.B * p.H * nQt;
  const int per_xcd = (total + 7) / 8;
  const int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (lin >= total) return;
  const int bh = lin / nQt, qt = lin % nQt;
  const int b = bh / p.H, h = bh % p.H;
  const int q32 = qt * 8 + wave;  // 32-query block of this wave

  const int sk = p.row_cnt ? p.row_cnt[b] : p.Sk;
  const int nt = (sk + kTileKeys - 1) / kTileKeys;
  // this wave's 4 KiB slice of every [K|V] tile record
  const char* kv_w = p.kv + (int64_t)bh * p.kv_bh_stride + wave * 4096 + lane * 16;
  // DMA: direct-to-LDS copies two tiles ahead into a 3-slot ring.
  auto dma = [&](int t, int slot) {
    const char* g = kv_w + (int64_t)t * p.kv_tile_stride;
    char* d = lds[slot] + wave * 4096;
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_dma16(g + i * 1024, d + i * 1024);
  };
  // !DMA: HBM/L2 -> VGPRs at the top of an iteration, VGPRs -> LDS at its end, 2 slots.
  i32x4 stage[4];
  auto fetch = [&](int t) {
    const char* g = kv_w + (int64_t)t * p.kv_tile_stride;
#pragma unroll
    for (int i = 0; i < 4; ++i) stage[i] = *(const i32x4*)(g + i * 1024);
  };
  auto commit = [&](int slot) {
    char* d = lds[slot] + wave * 4096 + lane * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) *(i32x4*)(d + i * 1024) = stage[i];
  };

  W8State w;
  if (nt > 0) {
    if constexpr (DMA) {
      dma(0, 0);
      if (nt > 1) dma(1, 1);
    } else {
      fetch(0);
    }
    const bf16x8* qsrc =
        (const bf16x8*)(p.qp + (int64_t)bh * p.q_bh_stride + (int64_t)(q32 >> 1) * p.q_blk_stride) + (q32 & 1) * 8 * 64;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) w.qf[ks] = qsrc[ks * 64 + lane];
    if constexpr (!DMA) commit(0);
  }
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) w.o[db][i] = 0.f;
  w.m = -INFINITY;
  w.l = 0.f;
  const float c = p.c;
  const int last_lim = sk - (nt - 1) * kTileKeys;

  int slot = 0;
  for (int t = 0; t < nt; ++t) {
    // tile t (DMA: and t+1) is in LDS for everyone, and every wave is past tile t-1, whose slot is free
    if constexpr (DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const char* kbuf = lds[slot];
    if constexpr (DMA) {
      const int free_slot = slot == 0 ? 2 : slot - 1;
      if (t + 2 < nt) dma(t + 2, free_slot);
      slot = slot == 2 ? 0 : slot + 1;
    } else {
      if (t + 1 < nt) fetch(t + 1);
      slot ^= 1;
    }
    w8_qk(w, kbuf, kbuf + kKTileBytes, lane);
    w8_softmax_pv(w, kbuf + kKTileBytes, c, t == nt - 1 ? last_lim : kTileKeys, lane);
    if constexpr (!DMA) {
      if (t + 1 < nt) commit(slot);
    }
  }

  __bf16* ob = (__bf16*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
  const float lt = w.l + xhalf(w.l);
  const float inv = lt > 0.f ? 1.0f / lt : 0.f;
  const int q = q32 * 32 + (lane & 31);
  if (q < p.Sq) {
    __bf16* orow = ob + (int64_t)q * p.o_ss;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 wv;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) wv[rr] = (__bf16)(w.o[db][4 * g + rr] * inv);
        *(bf16x4*)(orow + 32 * db + 8 * g + 4 * hh) = wv;
      }
  }
}

// ------------------------------------------------------------------------------------------------
// Variant: 8 waves x 32 queries, software-pipelined inside each wave on 32-key sub-tiles:
//   step u:  S(u+1) = K'(u+1) Q'^T   (8 MFMAs)  |
//            O^T   += V(u-1)^T P(u-1) (8 MFMAs)  |  interleaved with the VALU work of
//            P(u)   = softmax numerators of S(u) |  the same step
// Everything lives in VGPRs (no AGPR traffic): O^T 64, S 2x16, Q 32, P 2x8, operand images in flight.
constexpr int kNBufP = 4;

struct W8PState {
  bf16x8 qf[8];
  f32x16 sa, sb;
  bf16x8 pa[2], pb[2];
  f32x16 o[4];
  float m, l, alpha;
};

template <bool DO_PV, bool MASK>
__device__ __forceinline__ void w8p_step(const char* kptr, const char* vptr, const bf16x8 (&qf)[8], const f32x16& s_cur,
                                         f32x16& s_nxt, const bf16x8 (&p_prev)[2], bf16x8 (&p_cur)[2], f32x16 (&o)[4],
                                         float& m, float& l, float& alpha, float c, int lim, int lane) {
  const int hh = lane >> 5;
  if (__any(alpha != 1.0f)) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
  }
  // ---- MFMA stream: QK^T of the next sub-tile interleaved with P.V of the previous one
  {
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const bf16x8 kf = *(const bf16x8*)(kptr + (i * 64 + lane) * 16);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[i], acc, 0, 0, 0);
      if constexpr (DO_PV) {
        const int b2 = i >> 2, db = i & 3;
        const bf16x8 vf = *(const bf16x8*)(vptr + ((b2 * 4 + db) * 64 + lane) * 16);
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p_prev[b2], o[db], 0, 0, 0);
      }
    }
    s_nxt = acc;
  }
  // ---- VALU stream: softmax numerators of the current sub-tile
  f32x16 s = s_cur;
  if constexpr (MASK) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = 8 * (i / 4) + 4 * hh + (i % 4);
      if (key >= lim) s[i] = -INFINITY;
    }
  }
  float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
  for (int i = 3; i < 15; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
  mx = fmaxf(mx, s[15]);
  mx = max_across_halves(mx) * c;
  const float m_old = m;
  const float m_new = (mx > m_old + kRescaleSlack) ? mx : m_old;
  alpha = __builtin_amdgcn_exp2f(m_old - m_new);
  m = m_new;
  float rsum = 0.f;
  const bf16x2 one2 = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
  for (int b2 = 0; b2 < 2; ++b2) {
    bf16x8 pk;
#pragma unroll
    for (int j = 0; j < 8; ++j) pk[j] = (__bf16)__builtin_amdgcn_exp2f(fmaf(s[8 * b2 + j], c, -m_new));
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      const bf16x2 pr = {pk[j], pk[j + 1]};
      rsum = __builtin_amdgcn_fdot2_f32_bf16(pr, one2, rsum, false);
    }
    p_cur[b2] = pk;
  }
  l = l * alpha + rsum;
  // keep this step's numerators inside the step (next to the MFMAs they overlap with)
#pragma unroll
  for (int b2 = 0; b2 < 2; ++b2) asm volatile("" : "+v"(p_cur[b2]));
#ifdef PKH3_SCHED
  // issue order: one MFMA, one LDS image read, then a slice of the softmax VALU work
  PKH3_SGB(kSgDsRead, PKH3_SCHED_AHEAD);
#pragma unroll
  for (int i = 0; i < (DO_PV ? 16 : 8); ++i) {
    PKH3_SGB(kSgMfma, 1);
    if (i + PKH3_SCHED_AHEAD < (DO_PV ? 16 : 8)) PKH3_SGB(kSgDsRead, 1);
    PKH3_SGB(kSgValu, PKH3_SCHED);
#ifdef PKH3_SCHED_TRANS
    PKH3_SGB(kSgTrans, PKH3_SCHED_TRANS);
#endif
  }
#endif
}

__global__ __launch_bounds__(512, 1) void attn_fwd_w8p_kernel(FwdParams p) {
  __shared__ __attribute__((aligned(1024))) char lds[kNBufP][kKvTileBytes];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int hh = lane >> 5;
  const int nQt = p.nQ64 / kWaves;
  const int total = p.B * p.H * nQt;
  const int per_xcd = (total + 7) / 8;
  const int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (lin >= total) return;
  const int bh = lin / nQt, qt = lin % nQt;
  const int b = bh / p.H, h = bh % p.H;
  const int q32 = qt * 8 + wave;

  const int sk = p.row_cnt ? p.row_cnt[b] : p.Sk;
  const int nt = (sk + kTileKeys - 1) / kTileKeys;
  // this wave's 4 KiB slice of every [K|V] tile record
  const char* kv_w = p.kv + (int64_t)bh * p.kv_bh_stride + wave * 4096 + lane * 16;

  auto prefetch = [&](int t, int slot) {
    const char* g = kv_w + (int64_t)t * p.kv_tile_stride;
    char* d = lds[slot] + wave * 4096;
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_dma16(g + i * 1024, d + i * 1024);
  };

  W8PState w;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) w.o[db][i] = 0.f;
  w.m = -INFINITY;
  w.l = 0.f;
  w.alpha = 1.0f;

  if (nt > 0) {
    prefetch(0, 0);
    if (nt > 1) prefetch(1, 1);
    if (nt > 2) prefetch(2, 2);
    {
      const bf16x8* qsrc = (const bf16x8*)(p.qp + (int64_t)bh * p.q_bh_stride + (int64_t)(q32 >> 1) * p.q_blk_stride) +
                           (q32 & 1) * 8 * 64;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) w.qf[ks] = qsrc[ks * 64 + lane];
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // pre-step: S_a = QK^T of sub-tile (0, 0)
    {
#pragma unroll
      for (int i = 0; i < 16; ++i) w.sa[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 kf = *(const bf16x8*)(lds[0] + (ks * 64 + lane) * 16);
        w.sa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, w.qf[ks], w.sa, 0, 0, 0);
      }
    }
    const float c = p.c;
    const int last_lim = sk - (nt - 1) * kTileKeys;
    // Ring slots: tile t-1 in sp, t in s0, t+1 in s1; tile t+3 goes into sp's slot after the barrier.
    int sp = kNBufP - 1, s0 = 0, s1 = 1;
#define PKH3_W8P_ITER(T, DO_PV0, MASKED)                                                                          \
  {                                                                                                               \
    w8p_step<DO_PV0, MASKED>(lds[s0] + 8 * 1024, lds[sp] + kKTileBytes + 8 * 1024, w.qf, w.sa, w.sb, w.pb, w.pa,  \
                             w.o, w.m, w.l, w.alpha, c, last_lim, lane);                                          \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                              \
    __syncthreads();                                                                                              \
    if ((T) + 3 < nt) prefetch((T) + 3, sp);                                                                      \
    w8p_step<true, MASKED>(lds[s1], lds[s0] + kKTileBytes, w.qf, w.sb, w.sa, w.pa, w.pb, w.o, w.m, w.l, w.alpha,  \
                           c, last_lim - 32, lane);                                                               \
    sp = s0;                                                                                                      \
    s0 = s1;                                                                                                      \
    s1 = s1 + 1 == kNBufP ? 0 : s1 + 1;                                                                           \
  }
    if (nt == 1) {
      PKH3_W8P_ITER(0, false, true)
    } else {
      PKH3_W8P_ITER(0, false, false)
      for (int t = 1; t < nt - 1; ++t) PKH3_W8P_ITER(t, true, false)
      PKH3_W8P_ITER(nt - 1, true, true)
    }
#undef PKH3_W8P_ITER
    // drain: pending rescale, then O += P_b V(nt-1, 1)
    {
      const char* vptr = lds[sp] + kKTileBytes + 8 * 1024;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) w.o[db][i] *= w.alpha;
#pragma unroll
      for (int b2 = 0; b2 < 2; ++b2)
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const bf16x8 vf = *(const bf16x8*)(vptr + ((b2 * 4 + db) * 64 + lane) * 16);
          w.o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, w.pb[b2], w.o[db], 0, 0, 0);
        }
    }
  }

  __bf16* ob = (__bf16*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
  const float lt = w.l + xhalf(w.l);
  const float inv = lt > 0.f ? 1.0f / lt : 0.f;
  const int q = q32 * 32 + (lane & 31);
  if (q < p.Sq) {
    __bf16* orow = ob + (int64_t)q * p.o_ss;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 wv;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) wv[rr] = (__bf16)(w.o[db][4 * g + rr] * inv);
        *(bf16x4*)(orow + 32 * db + 8 * g + 4 * hh) = wv;
      }
  }
}

hipError_t launch_attn_fwd(const FwdParams& p, hipStream_t st) {
  const int nQt = p.nQ64 / kWaves;
  const int total = p.B * p.H * nQt;
  const int per_xcd = (total + 7) / 8;
  static const int variant = getenv("PKH3_KERNEL") ? atoi(getenv("PKH3_KERNEL")) : 0;
  if (variant == 2)
    hipLaunchKernelGGL(attn_fwd_w8p_kernel, dim3(per_xcd * 8), dim3(512), 0, st, p);
  else if (variant == 1)
    hipLaunchKernelGGL(attn_fwd_w8_kernel<true>, dim3(per_xcd * 8), dim3(512), 0, st, p);
  else if (variant == 3)
    hipLaunchKernelGGL(attn_fwd_w8_kernel<false>, dim3(per_xcd * 8), dim3(512), 0, st, p);
  else
    hipLaunchKernelGGL(attn_fwd_dense_kernel, dim3(per_xcd * 8), dim3(256), 0, st, p);
  return hipGetLastError();
}

}  // namespace pkh3
