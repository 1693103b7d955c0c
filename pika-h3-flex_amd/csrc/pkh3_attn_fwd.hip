// Non-causal flash-style attention forward for gfx950 (CDNA4), head dim 128.
//
// Work split.  A workgroup is 12 waves (dense; three per SIMD) or 8 waves (block-sparse; two per SIMD);
// each wave owns 32 queries of one (batch, head) and keeps for them, in VGPRs, the Q operand images, the
// running row max / row sum and the fp32 output accumulator O^T (128 x 32, sixteen 16x16 blocks).  All waves share every 64-key
// K/V tile, which is copied HBM/L2 -> LDS with direct-to-LDS loads into a 3-slot ring, two tiles ahead of
// the math.  Several waves per SIMD is what overlaps the softmax VALU work of one wave with the MFMAs of
// another; the whole per-wave state stays in VGPRs (<= 168 dense, <= 256 sparse) so no accumulator ever
// moves between register files.  Q is read in place: RMSNorm, rotation and fp8 quantisation of the Q rows
// happen in registers while the first K/V tiles are in flight.
//
// Math per tile, all on the 16x16 MFMA shapes (see pkh3_common.h for the operand images and why these shapes):
//   S^T = K' Q'^T      A = K image (LDS), B = Q image (VGPR)      -> lane l holds queries l%16 and 16 + l%16, 4 keys
//                      per 16-key block (bf16: 32 x 16x16x32, Q' carries softmax_scale * log2(e) so S^T is in the
//                      log2 domain; fp8: 8 x 16x16x128 on e4m3 images, S^T rescaled by the per-64-row-block
//                      dequantisation scales in the softmax multiply)
//   softmax            bounded-logit path (the usual one): |q_i| * max_j |k_j| bounds every logit of the wave's
//                      queries; when that bound is small, exp2(logit) needs no maximum at all.  Otherwise the
//                      online form: row max in-lane over the keys + two row swaps across the four lane groups,
//                      raised only when exceeded by 2^8 so the O^T rescale is rare.  Row sum kept per lane group,
//                      merged once at the end.
//   O^T += V^T P^T     A = V image (LDS), B = P packed to bf16 straight from the S^T registers (32 x 16x16x32)
// The transposed formulation keeps every per-query quantity (max, sum, rescale factor) a per-lane
// scalar: no cross-lane traffic in the rescale, none between the two GEMMs.  O leaves through LDS, turned
// around into whole 256-byte rows.
//
// Other forms of the dense kernel (see attn_fwd_body): the short-key form (at most 16 key tiles: 4 waves per
// workgroup, 32-key half tiles, three workgroups per CU), and the long form with the key tiles of a unit shared out
// among several workgroups that merge through global scratch, for a thinly filled last round of a long call.
//
// Block-sparse variant.  A workgroup covers 4 query row-blocks (64 queries each, a wave pair per row-block).
// Phase 1 walks the key tiles all four row-blocks keep, exactly like the dense kernel.  Phase 2 walks the
// remaining tiles per row-block: every iteration gives each wave pair one 32-key half of a tile of its own
// list in its own LDS area, so all 8 waves stay busy.  The lists are built on the device by a plan kernel.
#include <atomic>

#include "pkh3_common.h"
#include "pkh3_internal.h"

namespace pkh3 {

constexpr int kDenseWaves = 12;  // dense kernel: three waves per SIMD (<= 168 VGPRs each), 384 queries per workgroup
constexpr int kShortWaves = 4;   // short-key dense kernel: three 4-wave workgroups per CU
constexpr int kMaxParts = 8;     // long dense form: most workgroups a unit's key tiles are shared out among ...
constexpr int kMinPartTiles = 24;  // ... and fewest key tiles such a workgroup is worth starting for
constexpr int kSparseWaves = 2 * kSparseRows;  // block-sparse: a wave pair per row-block; two such workgroups share a CU
constexpr int kRing = 3;               // LDS ring depth (tiles)
constexpr float kRescaleSlack = 8.0f;  // the running max is only raised when exceeded by 2^8
constexpr float kStaticMaxLimit = 48.0f;  // rows whose |logit| bound is below this skip the running max (terms 2^-48 .. 2^48)

#define PKH3_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
// Each tile loop ends on an MFMA into the O^T accumulators.  The compiler was seen to place the register
// copies that merge the two loop variants (v_mov_b64 reading the accumulator's last registers) four scalar
// instructions after that MFMA, before its result is written back; the block-sparse kernel then returned a stale
// O^T block.  32 idle issue cycles after every loop let the last MFMA retire whatever follows.  The accumulators
// are operands of the statement, so every read or copy of them the compiler emits after the loop is ordered
// after the idle cycles.
#define PKH3_MFMA_DRAIN(W)                                                                                               \
  asm volatile("s_nop 15\n\ts_nop 15"                                                                                    \
               : "+v"((W).o[0][0]), "+v"((W).o[0][1]), "+v"((W).o[1][0]), "+v"((W).o[1][1]), "+v"((W).o[2][0]),          \
                 "+v"((W).o[2][1]), "+v"((W).o[3][0]), "+v"((W).o[3][1]), "+v"((W).o[4][0]), "+v"((W).o[4][1]),          \
                 "+v"((W).o[5][0]), "+v"((W).o[5][1]), "+v"((W).o[6][0]), "+v"((W).o[6][1]), "+v"((W).o[7][0]),          \
                 "+v"((W).o[7][1])::"memory")
constexpr int kSgMfma = 0x008, kSgDsRead = 0x100;

__device__ __forceinline__ void lds_dma16(const char* g, unsigned lane_off, char* l) {
  // 64 lanes x 16 B, global -> LDS without passing through VGPRs: lane i copies g[lane_off_i .. +16) to
  // l + i*16.  `g` and `l` are wave-uniform (the address arithmetic stays on the scalar unit), `lane_off` is
  // the per-lane byte offset.
  // Issued through inline assembly on purpose: once the compiler sees a direct-to-LDS load it stops trusting
  // the in-order LDS counter and turns every later wait on an LDS read into lgkmcnt(0), which serialises the
  // operand image reads.  Completion is tracked by hand: the s_waitcnt vmcnt(0) at the top of each tile loop.
  const unsigned lds_addr = (unsigned)(size_t)(__attribute__((address_space(3))) char*)l;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_off), "s"(g), "s"(lds_addr)
               : "memory", "m0");
}

// Wave-uniform reads of tables earlier kernels wrote (tile lists, fp8 scales): through the scalar cache, so
// they count on lgkmcnt and never make the wave wait for its outstanding HBM->LDS copies (vmcnt).
template <typename T>
__device__ __forceinline__ T uniform_load(const T* p, int i) {
  return ((const __attribute__((address_space(4))) T*)p)[i];
}

// Stores and loads that are coherent across the whole device (all XCDs) one by one: they go past the caches that
// are not, so data handed from one workgroup to another needs no cache write-back or invalidation around it --
// only the writer's wait for its stores before it signals, and the reader's signal check before its loads.
__device__ __forceinline__ void store_device(float* p, f32x4 v) {
  const unsigned long long lo = ((unsigned long long)__float_as_uint(v[1]) << 32) | __float_as_uint(v[0]);
  const unsigned long long hi = ((unsigned long long)__float_as_uint(v[3]) << 32) | __float_as_uint(v[2]);
  __hip_atomic_store((unsigned long long*)p, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store((unsigned long long*)p + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_device(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f32x4 load_device4(const float* p) {
  const unsigned long long lo = __hip_atomic_load((const unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long hi = __hip_atomic_load((const unsigned long long*)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return f32x4{__uint_as_float((unsigned)lo), __uint_as_float((unsigned)(lo >> 32)), __uint_as_float((unsigned)hi),
               __uint_as_float((unsigned)(hi >> 32))};
}
__device__ __forceinline__ float load_device(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// maximum over the four lanes l % 16 == const (one per 16-lane group): two row swaps, no LDS crossbar
__device__ __forceinline__ float max_across_groups(float x) {
  const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(r16[0]), __uint_as_float(r16[1]));
  const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r32[0]), __uint_as_float(r32[1]));
}

// Per-wave state.  Lane (c = l % 16, g = l / 16) works for the two queries 16*qb + c, qb = 0, 1, of the wave's 32.
template <bool FP8>
struct WaveState {
  bf16x8 qf[FP8 ? 1 : 2][FP8 ? 1 : 4];  // bf16 Q images (qb, ks): Q'[16*qb + c][32*ks + 8*g + j]
  i32x8 q8[FP8 ? 2 : 1];                // fp8 Q images (qb): bytes 8*ks + j = element 32*ks + 8*g + j
  f32x4 s[4][2];                        // S^T of the tile (kb, qb): keys 16*kb + 4*g + i
  f32x4 o[8][2];                        // O^T accumulators (db, qb): head-dim rows 16*db + 4*g + i
  bf16x8 vf[8];                         // V images of the first 32 keys, fetched while QK^T finishes
  float m[2], l[2];                     // per query block: running row max (scaled, log2 domain), this lane group's row sum
  int qe;                               // fp8 with power-of-two scales: exponent byte (E8M0) of the Q block's scale
};

#define PKH3_MFMA16(A, B, C) __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, B, C, 0, 0, 0)
// format codes 0/0 = e4m3 x e4m3; scale operands 0 select the unscaled form of the instruction
#define PKH3_MFMA16_F8(A, B, C) __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, C, 0, 0, 0, 0, 0, 0)
// the scaled form: the product is multiplied by 2^(EA - 127) * 2^(EB - 127), EA / EB = byte 0 of each lane's scale
// operand (every lane passes the same exponents: one scale per 64-row block, not per 32 elements)
#define PKH3_MFMA16_F8S(A, B, C, EA, EB) __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, C, 0, 0, 0, EA, 0, EB)

// S^T = K' Q'^T for the 64 keys of one tile: image i of the K tile is (half, ks, kb2) = (i >> 3, (i >> 1) & 3, i & 1)
// and feeds the two query blocks, so four accumulators rotate inside each half.  LDS reads run 8 images ahead of
// the MFMAs that consume them; the tail of the MFMA chain covers the first V image reads.
// LEAN (three waves per SIMD, 168 VGPRs): the reads run only 4 images ahead and V is left to the P.V loop.
// AHEAD: images the LEAN reads run ahead (the copies of the loop that run once per workgroup take 2 and fit the registers)
// POW2 (fp8): the block scales are powers of two and go into the MFMA as its scale operands (`ke`: exponent byte of
// this K tile's scale), so S^T leaves the MFMA dequantised.
template <bool FP8, bool LEAN, int AHEAD = 4, bool POW2 = false>
__device__ __forceinline__ void qk_tile(WaveState<FP8>& w, const char* kbuf, const char* vbuf, int lane, int ke = 0) {
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  if constexpr (!FP8 && LEAN) {
    bf16x8 kf[16];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) kf[i] = *(const bf16x8*)(kbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int ks = (i >> 1) & 3, kb = 2 * (i >> 3) + (i & 1);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.s[kb][qb] = PKH3_MFMA16(kf[i], w.qf[qb][ks], ks == 0 ? zero : w.s[kb][qb]);
      if (i + AHEAD < 16) kf[i + AHEAD] = *(const bf16x8*)(kbuf + ((i + AHEAD) * 64 + lane) * 16);
    }
    PKH3_SGB(kSgDsRead, AHEAD);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      PKH3_SGB(kSgMfma, 2);
      if (i + AHEAD < 16) PKH3_SGB(kSgDsRead, 1);
    }
  } else if constexpr (!FP8) {
    bf16x8 kf[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) kf[i] = *(const bf16x8*)(kbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int ks = (i >> 1) & 3, kb = 2 * (i >> 3) + (i & 1);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.s[kb][qb] = PKH3_MFMA16(kf[i], w.qf[qb][ks], ks == 0 ? zero : w.s[kb][qb]);
      if (i < 8)
        kf[i + 8] = *(const bf16x8*)(kbuf + ((i + 8) * 64 + lane) * 16);
      else
        w.vf[i - 8] = *(const bf16x8*)(vbuf + ((i - 8) * 64 + lane) * 16);
    }
    PKH3_SGB(kSgDsRead, 8);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      PKH3_SGB(kSgMfma, 2);
      PKH3_SGB(kSgDsRead, 1);
    }
  } else {
    i32x4 kc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) kc[i] = *(const i32x4*)(kbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const i32x4 a0 = kc[2 * kb], a1 = kc[2 * kb + 1];
      const i32x8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
        w.s[kb][qb] = POW2 ? PKH3_MFMA16_F8S(a, w.q8[qb], zero, ke, w.qe) : PKH3_MFMA16_F8(a, w.q8[qb], zero);
      // the MFMA chain covers the first V image reads: 8 images, or 4 where registers are short (LEAN)
      if constexpr (LEAN) {
        w.vf[kb] = *(const bf16x8*)(vbuf + (kb * 64 + lane) * 16);
      } else {
        w.vf[2 * kb] = *(const bf16x8*)(vbuf + ((2 * kb) * 64 + lane) * 16);
        w.vf[2 * kb + 1] = *(const bf16x8*)(vbuf + ((2 * kb + 1) * 64 + lane) * 16);
      }
    }
  }
}

// exp2 of one logit.  bf16 path, and fp8 with power-of-two scales: Q' already carries softmax_scale * log2(e) (and the
// MFMA applied the scales), so S^T is in the log2 domain and `c` is unused; fp8 with absmax scales (MUL): `c` carries
// that factor times the dequantisation scales.  STATIC: the logits are bounded in magnitude (see kStaticMaxLimit), so
// no maximum is subtracted at all.
template <bool MUL, bool STATIC>
__device__ __forceinline__ float softmax_numerator(float s, float c, float m) {
  if constexpr (MUL) return __builtin_amdgcn_exp2f(STATIC ? s * c : fmaf(s, c, -m));
  else return __builtin_amdgcn_exp2f(STATIC ? s : s - m);
}

// Softmax numerators of NKB key blocks of w.s (a whole tile: 4, a 32-key half: 2) into the P^T operands of
// the P.V MFMAs: operand (half, qb) takes, for lane group g, the keys v_image_key(g, j) of its half, i.e. registers
// 0..3 of key block 2*half and of key block 2*half + 1 -- P never leaves its lane.  Also the running max / rescale
// of the online path and the row sums.  `lim` = keys of these blocks that exist (only read when MASKED).
// STATIC: w.m is not used: every logit is bounded (|q_i| * max_j |k_j| * c), small enough that exp2(logit) is a
// normal number; the running max, its exchange across the lane groups and the O^T rescale are then not needed at
// all, and the numerators of the first 32 keys do not wait for the second half of S^T.
template <bool FP8, bool STATIC, bool MASKED, int NKB, bool POW2 = false>
__device__ __forceinline__ void softmax_blocks(WaveState<FP8>& w, bf16x8 (&pf)[NKB / 2][2], float c, int lim, int lane) {
  constexpr bool MUL = FP8 && !POW2;  // the logits still need their dequantisation scales
  const int g = lane >> 4;
  if (MASKED) {
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (16 * kb + 4 * g + i >= lim) {
          w.s[kb][0][i] = -INFINITY;
          w.s[kb][1][i] = -INFINITY;
        }
  }
  float m_new[2] = {w.m[0], w.m[1]}, alpha[2] = {1.0f, 1.0f};
  if constexpr (!STATIC) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float mx = w.s[0][qb][0];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, w.s[kb][qb][i]);
      mx = max_across_groups(mx) * (MUL ? c : 1.0f);
      m_new[qb] = (mx > w.m[qb] + kRescaleSlack) ? mx : w.m[qb];
      alpha[qb] = __builtin_amdgcn_exp2f(w.m[qb] - m_new[qb]);
      w.m[qb] = m_new[qb];
    }
    if (__any(alpha[0] != 1.0f || alpha[1] != 1.0f)) {
#pragma unroll
      for (int db = 0; db < 8; ++db)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int i = 0; i < 4; ++i) w.o[db][qb][i] *= alpha[qb];
    }
  }
  const bf16x2 one2 = {(__bf16)1.0f, (__bf16)1.0f};
  float rsum[2] = {0.f, 0.f};
#pragma unroll
  for (int half = 0; half < NKB / 2; ++half)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      bf16x8 pk;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        pk[j] = (__bf16)softmax_numerator<MUL, STATIC>(w.s[2 * half + (j >> 2)][qb][j & 3], c, m_new[qb]);
      // row sum over the bf16-rounded values, the same numbers the P.V MFMA consumes
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const bf16x2 pr = {pk[j], pk[j + 1]};
        rsum[qb] = __builtin_amdgcn_fdot2_f32_bf16(pr, one2, rsum[qb], false);
      }
      pf[half][qb] = pk;
    }
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) w.l[qb] = STATIC ? w.l[qb] + rsum[qb] : w.l[qb] * alpha[qb] + rsum[qb];
}

// Softmax of w.s, then O^T += V^T P^T for one tile: V image i is (half, db) = (i >> 3, i & 7) and feeds the two
// query blocks, sixteen accumulators in rotation.  `c` = softmax scale * log2(e) (times the fp8 dequantisation
// scales of this tile); `lim` = keys of this tile that exist (only read when MASKED).
template <bool FP8, bool STATIC, bool LEAN, bool MASKED, bool POW2 = false>
__device__ __forceinline__ void softmax_pv_tile(WaveState<FP8>& w, const char* vbuf, float c, int lim, int lane) {
  bf16x8 pf[2][2];
  softmax_blocks<FP8, STATIC, MASKED, 4, POW2>(w, pf, c, lim, lane);
  if constexpr (LEAN) {
    bf16x8 vg[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) vg[i] = FP8 ? w.vf[i] : *(const bf16x8*)(vbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.o[i & 7][qb] = PKH3_MFMA16(vg[i], pf[i >> 3][qb], w.o[i & 7][qb]);
      if (i + 4 < 16) vg[i + 4] = *(const bf16x8*)(vbuf + ((i + 4) * 64 + lane) * 16);
    }
  } else {
    bf16x8 vg[8];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.o[i & 7][qb] = PKH3_MFMA16(i < 8 ? w.vf[i] : vg[i - 8], pf[i >> 3][qb], w.o[i & 7][qb]);
      if (i < 8) vg[i] = *(const bf16x8*)(vbuf + ((i + 8) * 64 + lane) * 16);
    }
  }
}

// ---- 32-key half tiles: the short-key form of the dense kernel, phase 2 of the block-sparse one ----
// S^T (32 keys x 32 queries) into w.s[0..1]; kbuf/vbuf point at this half's K images (8 bf16 / 4 fp8 chunks)
// and V images (8).
// LEAN (three waves per SIMD): the K reads run 4 images ahead and only the fp8 path prefetches V (4 images).
template <bool FP8, bool LEAN = false, bool POW2 = false>
__device__ __forceinline__ void qk_half(WaveState<FP8>& w, const char* kbuf, const char* vbuf, int lane, int ke = 0) {
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  if constexpr (!FP8 && LEAN) {
    bf16x8 kf[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) kf[i] = *(const bf16x8*)(kbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.s[i & 1][qb] = PKH3_MFMA16(kf[i], w.qf[qb][i >> 1], i < 2 ? zero : w.s[i & 1][qb]);
      if (i + 4 < 8) kf[i + 4] = *(const bf16x8*)(kbuf + ((i + 4) * 64 + lane) * 16);
    }
  } else if constexpr (!FP8) {
    bf16x8 kf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) kf[i] = *(const bf16x8*)(kbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.s[i & 1][qb] = PKH3_MFMA16(kf[i], w.qf[qb][i >> 1], i < 2 ? zero : w.s[i & 1][qb]);
      w.vf[i] = *(const bf16x8*)(vbuf + (i * 64 + lane) * 16);
    }
  } else {
    i32x4 kc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) kc[i] = *(const i32x4*)(kbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const i32x4 a0 = kc[2 * kb], a1 = kc[2 * kb + 1];
      const i32x8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
        w.s[kb][qb] = POW2 ? PKH3_MFMA16_F8S(a, w.q8[qb], zero, ke, w.qe) : PKH3_MFMA16_F8(a, w.q8[qb], zero);
#pragma unroll
      for (int i = 0; i < (LEAN ? 2 : 4); ++i) {
        const int v = (LEAN ? 2 : 4) * kb + i;
        w.vf[v] = *(const bf16x8*)(vbuf + (v * 64 + lane) * 16);
      }
    }
  }
}

// Softmax numerators of w.s[0..1] and O^T += V^T P^T for one half tile (V images already in w.vf).
// `lim` = keys of this half that exist (<= 0: none; only read when < 32).
// LEAN: the V images (beyond the 4 the fp8 path prefetched) are read here, 4 ahead of their MFMAs, from vbuf.
// FULL: the caller guarantees lim == 32, no masking code at all.
template <bool FP8, bool STATIC, bool LEAN = false, bool FULL = false, bool POW2 = false>
__device__ __forceinline__ void softmax_pv_half(WaveState<FP8>& w, float c, int lim, int lane, const char* vbuf = nullptr) {
  bf16x8 pf[1][2];
  // the running-max form always takes the masking copy (two copies of it do not fit the registers of some variants)
  if (!FULL && (!STATIC || lim < 32)) softmax_blocks<FP8, STATIC, true, 2, POW2>(w, pf, c, lim, lane);
  else softmax_blocks<FP8, STATIC, false, 2, POW2>(w, pf, c, lim, lane);
  if constexpr (LEAN) {
    bf16x8 vg[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) vg[i] = FP8 ? w.vf[i] : *(const bf16x8*)(vbuf + (i * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.o[i][qb] = PKH3_MFMA16(vg[i], pf[0][qb], w.o[i][qb]);
      if (i + 4 < 8) vg[i + 4] = *(const bf16x8*)(vbuf + ((i + 4) * 64 + lane) * 16);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) w.o[i][qb] = PKH3_MFMA16(w.vf[i], pf[0][qb], w.o[i][qb]);
  }
}

// WAVES == kShortWaves selects the short-key form of the dense kernel: 4 waves (one per SIMD, <= 168 VGPRs) and a
// ring of 32-key half tiles in 48 KiB of LDS, so three workgroups share a CU and the Q load and O store of one
// run under the tiles of the others.  With few key tiles that overlap is worth more than the three-fold K/V
// copies cost (the K/V of such calls sit in L2).
// PARTS (long dense form only): `parts` workgroups share a unit's queries and walk 1/parts of the key tiles each, so
// such a workgroup lasts 1/parts as long as a whole one: the way a call's last, thinly filled round of workgroups is
// cut into pieces that fill the chip (see launch_fp).  Each wave leaves its partial result (un-normalised O^T, row
// sums, row maxima) in global scratch; the wave that arrives last of the `parts` adds the others' to its own and
// writes the output.
constexpr int kMergeBytes = kPartialBytes;  // one wave's partial result in fp32

// bytes of LDS a form of the kernel needs
template <bool FP8, bool SPARSE, int WAVES>
constexpr int fwd_lds_bytes() {
  constexpr bool HALFMODE = !SPARSE && WAVES == kShortWaves;
  constexpr int kRingT = (SPARSE && !FP8 && WAVES < 8) ? 2 : kRing;
  constexpr int kStages2 = (SPARSE && FP8 && WAVES < 8) ? 3 : 2;
  constexpr int kTileBytes = (FP8 ? kK8TileBytes : kKTileBytes) + kVTileBytes;
  constexpr int kHalfBytes = kTileBytes / 2;
  constexpr int kStageBytes = 32 * kD * 2;    // one wave's 32 x 128 bf16 output block, staged for the row-wise store
  // dense / phase 1: ring of kRingT whole tiles; sparse phase 2: kStages2 stages of row-private half tiles
  constexpr int kPhase2Bytes = SPARSE ? kStages2 * kSparseRows * kHalfBytes : 0;
  constexpr int kRingBytes = HALFMODE ? kRing * kHalfBytes
                             : (kPhase2Bytes > kRingT * kTileBytes ? kPhase2Bytes : kRingT * kTileBytes);
  constexpr int kAfterBytes = WAVES * kStageBytes;  // LDS use after the loops
  return kRingBytes > kAfterBytes ? kRingBytes : kAfterBytes;
}

// POW2 (fp8 only): power-of-two block scales, applied by the scaled MFMA; softmax_scale * log2(e) rides in Q' before
// it is quantised, so the softmax has no multiply left (the instruction count of the bf16 form).
// One workgroup's work.  `blk`: index of the workgroup inside its section of the launch; the section covers the
// units [unit0, unit0 + units), a unit being one workgroup's block of queries (`parts` workgroups per unit; their
// partial results start at slot `part_base` of the scratch, their counters at unit slot `cnt_base`).
template <bool FP8, bool SPARSE, int WAVES, bool POW2>
__device__ __forceinline__ void attn_fwd_body(const FwdParams& p, int blk, int unit0, int units, int parts, int part_base,
                                              int cnt_base, char* lds_raw, int fetched = -1) {
  static_assert(!SPARSE || WAVES == kSparseWaves, "block-sparse layout: a wave pair per row-block of the plan");
  static_assert(FP8 || !POW2, "power-of-two scales belong to the fp8 form");
  constexpr bool SHORT = !SPARSE && WAVES == kShortWaves;
  constexpr bool LEAN = !SPARSE;                        // dense long-key form: three waves per SIMD, lean read-ahead
  // whole-tile ring depth: three tiles, except where two workgroups share the CU's LDS and a bf16 tile is 32 KiB
  constexpr int kRingT = (SPARSE && !FP8 && WAVES < 8) ? 2 : kRing;
  constexpr int kAhead = kRingT - 1;                    // tiles in flight ahead of the one being used
  constexpr int kStages2 = (SPARSE && FP8 && WAVES < 8) ? 3 : 2;  // sparse phase 2: stages of row-private half tiles
  constexpr bool HALFMODE = SHORT;                      // ring of 32-key half tiles
  constexpr bool PARTS = !SPARSE && !SHORT;             // the long dense form: the key tiles may be shared out (`parts`)
  constexpr int kKBytes = FP8 ? kK8TileBytes : kKTileBytes;
  constexpr int kTileBytes = kKBytes + kVTileBytes;
  constexpr int kChunks = kTileBytes / 1024;  // 1 KiB pieces of a tile, dealt round-robin to the waves
  constexpr int kHalfBytes = kTileBytes / 2;  // K and V images of 32 keys
  constexpr int kStageBytes = 32 * kD * 2;    // one wave's 32 x 128 bf16 output block, staged for the row-wise store
  char(*lds)[kTileBytes] = (char(*)[kTileBytes])lds_raw;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  // Workgroups are handed to the 8 XCDs round-robin; give each XCD one contiguous run of
  // (batch, head, query tile) so the 32 CUs behind one L2 stream the same K/V at the same time.
  // (Every section of a launch starts at a workgroup index that is a multiple of 8.)
  // (`fetched` >= 0: the unit came from the work queues instead, see attn_fwd_dense_kernel.)
  const int total = units * parts;
  const int per_xcd = (total + 7) / 8;
  const int lin = fetched >= 0 ? fetched : (blk & 7) * per_xcd + (blk >> 3);
  if (lin >= total) return;
  // unit inside the section, and which share of its keys: share-major, so that the workgroups an XCD runs at the
  // same time walk the same key tiles of (mostly) the same head, as the whole units before them do
  const int part = lin / units, ul = lin % units;
  const int unit = unit0 + ul;
  const int wq = wave;                                    // which 32-query block of the unit
  const int nQt = (p.nQ64 * 2 + WAVES - 1) / WAVES;       // units per (batch, head)
  const int bh = unit / nQt, qt = unit % nQt;
  const int q32 = qt * WAVES + wq;
  const int b = bh / p.H, h = bh % p.H;

  const int sk = p.row_cnt ? p.row_cnt[b] : p.Sk;
  const int nkt = (sk + kTileKeys - 1) / kTileKeys;
  // sparse: [tiles every row-block of this workgroup keeps | tiles only row-block 0 keeps | ... 1 | ...]
  const int* plan = SPARSE ? p.plan + (int64_t)qt * p.plan_stride : nullptr;
  const int* plan_cnt = SPARSE ? p.plan_cnt + qt * kSparseLists : nullptr;
  const int nt = SPARSE ? uniform_load(plan_cnt, 0) : nkt;  // tiles all the waves walk together
  // the tiles [t_begin, t_end) of those are this workgroup's share
  // (32-bit arithmetic: at most 2^18 tiles times kMaxParts; the results address the tile copies from scalar registers)
  const int t_begin = PARTS ? __builtin_amdgcn_readfirstlane(part * nt / parts) : 0;
  const int t_end = PARTS ? __builtin_amdgcn_readfirstlane((part + 1) * nt / parts) : nt;

  // this wave's pieces of every [K|V] tile record: 1 KiB chunks wave, wave + WAVES, ...
  const char* kv_w = p.kv + (int64_t)bh * p.kv_bh_stride + wave * 1024;
  const unsigned lane_off = lane * 16;
  auto dma = [&](int tile, int slot) {
    const char* g = kv_w + (int64_t)tile * p.kv_tile_stride;
    char* d = lds[slot] + wave * 1024;
#pragma unroll
    for (int i = 0; i < (kChunks + WAVES - 1) / WAVES; ++i) {
      if ((i + 1) * WAVES <= kChunks) lds_dma16(g + i * WAVES * 1024, lane_off, d + i * WAVES * 1024);
      else if (i * WAVES + wave < kChunks) lds_dma16(g + i * WAVES * 1024, lane_off, d + i * WAVES * 1024);
    }
  };
  auto entry = [&](int i) { return SPARSE ? uniform_load(plan, i) : i; };  // i-th shared tile

  // half-tile form: [K half | V half] per ring slot, every wave copies the same share
  constexpr int kKHalfB = kKBytes / 2, kVHalfB = kVTileBytes / 2;
  const int n_half = (sk + 31) / 32;
  const int h_begin = 0, n_mine = n_half;
  char* ring = lds_raw;
  auto dma_short = [&](int half, int slot) {
    static_assert((kKHalfB / 1024) % kShortWaves == 0 && (kVHalfB / 1024) % kShortWaves == 0, "equal shares");
    const char* g = p.kv + (int64_t)bh * p.kv_bh_stride + (int64_t)(half >> 1) * p.kv_tile_stride;
    char* d = ring + slot * kHalfBytes;
    const int kb = half & 1;
#pragma unroll
    for (int i = 0; i < kKHalfB / 1024 / kShortWaves; ++i) {
      const int ch = wq * (kKHalfB / 1024 / kShortWaves) + i;
      lds_dma16(g + kb * kKHalfB + ch * 1024, lane_off, d + ch * 1024);
    }
#pragma unroll
    for (int i = 0; i < kVHalfB / 1024 / kShortWaves; ++i) {
      const int ch = wq * (kVHalfB / 1024 / kShortWaves) + i;
      lds_dma16(g + kKBytes + kb * kVHalfB + ch * 1024, lane_off, d + kKHalfB + ch * 1024);
    }
  };

  WaveState<FP8> w;
  if constexpr (HALFMODE) {
    if (n_mine > 0) dma_short(h_begin, 0);
    if (n_mine > 1) dma_short(h_begin + 1, 1);
  } else if (t_end > t_begin) {
    dma(entry(t_begin), 0);
    if (kAhead > 1 && t_end > t_begin + 1) dma(entry(t_begin + 1), 1);
  }
  // Q load, fused with QK-RMSNorm, rotation and (fp8) quantisation, in the layout of the MFMA B images themselves:
  // lane (c, g) reads, for each of the wave's two 16-query blocks qb, the 32 elements d = 32*ks + 8*g + j of query
  // row q32*32 + 16*qb + c (four lanes per row, norm_rope_quarter), so the operand images are formed in the lane
  // that uses them and Q' never exists in memory.
  float qscale = 1.0f;
  float qn2 = 0.f;  // largest squared norm of this lane's Q' rows (bf16: before the rounding; fp8: dequantised)
  {
    const int c16 = lane & 15, g4 = lane >> 4;
    const RowTransform tf{p.q_norm_w, p.q_eps, p.q_rope_mode, p.q_cos, p.q_sin};
    NormQuarter norm;
    if (p.q_norm_w) load_norm_quarter(norm, tf, g4);
    float x[2][32];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int qrow = q32 * 32 + 16 * qb + c16;
      const bool valid = qrow < p.Sq;
      const __bf16* row = (const __bf16*)p.q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + (int64_t)(valid ? qrow : 0) * p.q_ss + 8 * g4;
      bf16x8 raw[4];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) raw[ks] = *(const bf16x8*)(row + 32 * ks);
      RopeQuarter rope;
      if (p.q_rope_mode != 0 && valid) load_rope_quarter(rope, tf, qrow, g4);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j) x[qb][ks * 8 + j] = valid ? (float)raw[ks][j] : 0.f;
      norm_rope_quarter(x[qb], tf, norm, rope, valid, g4);
    }
    if constexpr (!FP8) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        float n2 = 0.f;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          bf16x8 t;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            // softmax_scale * log2(e) rides in Q', so S^T comes out of the MFMAs in the log2 domain
            const float xs = x[qb][ks * 8 + j] * p.c;
            t[j] = (__bf16)xs;
            n2 = fmaf(xs, xs, n2);   // the norm before the rounding: the bound below carries the margin for it
          }
          w.qf[qb][ks] = t;
        }
        qn2 = fmaxf(qn2, wave_sum_groups(n2));
      }
    } else {
      // one absmax scale per 64-query block = this wave and its neighbour (wave ^ 1)
      __shared__ float q_amax[WAVES];
      float amax = 0.f;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 32; ++i) {
          // power-of-two scales: softmax_scale * log2(e) goes into Q' before the quantisation, as in the bf16 form
          if constexpr (POW2) x[qb][i] *= p.c;
          amax = fmaxf(amax, fabsf(x[qb][i]));
        }
      amax = wave_max(amax);
      if (lane == 0) q_amax[wave] = amax;
      __syncthreads();
      amax = fmaxf(amax, q_amax[wave ^ 1]);
      qscale = fp8_block_scale(amax, POW2);
      w.qe = e8m0_of(qscale);
      const float inv = 1.0f / qscale;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        float n2 = 0.f;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const i32x2 q = quant_fp8_piece(x[qb] + 8 * ks, inv);   // bytes 8*ks + j of the image = element 32*ks + 8*g + j
          w.q8[qb][2 * ks] = q[0];
          w.q8[qb][2 * ks + 1] = q[1];
#pragma unroll
          for (int wd = 0; wd < 2; ++wd) {
            const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(q[wd], false);
            const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(q[wd], true);
            n2 += lo[0] * lo[0] + lo[1] * lo[1] + hi[0] * hi[0] + hi[1] * hi[1];
          }
        }
        qn2 = fmaxf(qn2, wave_sum_groups(n2) * qscale * qscale);
      }
    }
  }
#pragma unroll
  for (int db = 0; db < 8; ++db)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int i = 0; i < 4; ++i) w.o[db][qb][i] = 0.f;
  w.m[0] = w.m[1] = -INFINITY;
  w.l[0] = w.l[1] = 0.f;
  const float c = POW2 ? 1.0f : p.c * qscale;  // what the softmax still multiplies the logits by (fp8 absmax form only)
  const float* kscale = FP8 ? p.kscale + (int64_t)bh * p.nKt : nullptr;
  const int tail = sk & (kTileKeys - 1);  // keys in the last tile when it is partial

  // Upper bound of the magnitude of this query's logits (log2 domain): |q_i| * max_j |k_j| * c.  When it is
  // small for the whole wave, exp2(logit) is a normal number in fp32 and in bf16 whatever the data, and so are
  // the row sums and O^T (at most 2^bound * keys * |v|), so no running max is needed at all.
  bool static_max = false;
  if (HALFMODE ? n_half > 0 : nt > 0) {
    // margins: Q' and K' are rounded to bf16 (relative step 2^-9 each; fp8: K' to e4m3, relative step 2^-4) after
    // their norms were taken
    const float bound = sqrtf(qn2) * uniform_load(p.kmax, bh) * (FP8 ? (POW2 ? 1.08f : p.c * 1.08f) : 1.01f);
    static_max = __all(bound <= kStaticMaxLimit);
  }

  int slot = 0, slot_prev = (HALFMODE ? kRing : kRingT) - 1;  // ring slots of tile i and of tile i-1 (which takes the newest copy)
  // Only the last key tile can be partial.  It is peeled off the loop so that the loop body has no masking
  // branch between S^T and the softmax, which lets the numerators of the first 32 keys be scheduled under
  // the MFMAs of the second 32.
  const int n_masked = (tail && t_end > t_begin && entry(t_end - 1) == nkt - 1) ? 1 : 0;
  float ks_next = (FP8 && !HALFMODE && t_end > t_begin) ? uniform_load(kscale, entry(t_begin)) : 1.0f;
#define PKH3_TILE_LOOP(STATIC, MASKED, FROM, TO)                                                        \
  for (int i = FROM; i < TO; ++i) {                                                                     \
    /* tile i (and, with a ring of three, i+1) is in LDS for every wave (own slices: vmcnt, the others': */ \
    /* barrier), and every wave is past tile i-1, whose slot takes the newest copy */                   \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                    \
    __syncthreads();                                                                                    \
    const char* kbuf = lds[slot];                                                                       \
    /* the K scale of this tile was asked for an iteration ago (with power-of-two scales the first MFMA */ \
    /* needs it); the one of the next tile is asked for now */                                          \
    const float ks = ks_next;                                                                           \
    if (FP8) ks_next = uniform_load(kscale, entry(min(i + 1, t_end - 1)));                              \
    qk_tile<FP8, LEAN, (MASKED) ? 2 : 4, POW2>(w, kbuf, kbuf + kKBytes, lane, e8m0_of(ks));             \
    /* the copies of the tile two ahead are issued under the MFMAs of S^T, not in front of them: right */ \
    /* after the barrier their scalar address chain would run in every wave at once with the pipe idle */ \
    /* (power-of-two fp8 form: issued without a branch, a spare copy of the last tile at the end, which leaves */ \
    /* the tile body one straight run of code; that schedule measured 2.4 % faster there and 1 - 3 % slower in */ \
    /* the other forms) */                                                                              \
    if (POW2) dma(entry(min(i + kAhead, t_end - 1)), slot_prev);                                        \
    else if (i + kAhead < t_end) dma(entry(i + kAhead), slot_prev);                                     \
    slot_prev = slot;                                                                                   \
    slot = slot == kRingT - 1 ? 0 : slot + 1;                                                           \
    const float ct = (FP8 && !POW2) ? c * ks : c;                                                       \
    softmax_pv_tile<FP8, STATIC, LEAN, MASKED, POW2>(w, kbuf + kKBytes, ct, tail, lane);                \
  }
  // Half-tile loop.  The leading full halves take the copy of the code without masking; the one partial half at the
  // very end of the keys, if any, takes the general copy.
#define PKH3_SHORT_LOOP(STATIC, FULL, FROM, TO)                                                         \
  for (int i = FROM; i < TO; ++i) {                                                                     \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                    \
    __syncthreads();                                                                                    \
    const char* hbuf = ring + slot * kHalfBytes;                                                        \
    const int half = h_begin + i;                                                                       \
    const bool live = FULL || i < n_mine;                                                               \
    const float ks = (FP8 && live) ? uniform_load(kscale, half >> 1) : 1.0f;                            \
    if (live) qk_half<FP8, true, POW2>(w, hbuf, hbuf + kKHalfB, lane, e8m0_of(ks));                     \
    /* copies of the half two ahead: under the MFMAs of S^T (see the whole-tile loop) */               \
    if (i + 2 < n_mine) dma_short(h_begin + i + 2, slot_prev);                                          \
    slot_prev = slot;                                                                                   \
    slot = slot == kRing - 1 ? 0 : slot + 1;                                                            \
    if (live) {                                                                                         \
      const float ct = (FP8 && !POW2) ? c * ks : c;                                                     \
      softmax_pv_half<FP8, STATIC, true, FULL, POW2>(w, ct, sk - 32 * half, lane, hbuf + kKHalfB);      \
    }                                                                                                   \
  }
  if constexpr (HALFMODE) {
    const int n_iter = n_half;
    const int n_lead = sk / 32;  // leading full halves
    if (static_max) {
      PKH3_SHORT_LOOP(true, true, 0, n_lead)
      PKH3_SHORT_LOOP(true, false, n_lead, n_iter)
      PKH3_MFMA_DRAIN(w);
    } else {
      PKH3_SHORT_LOOP(false, true, 0, n_lead)
      PKH3_SHORT_LOOP(false, false, n_lead, n_iter)
      PKH3_MFMA_DRAIN(w);
    }
  } else if (static_max) {
    PKH3_TILE_LOOP(true, false, t_begin, t_end - n_masked)
    PKH3_TILE_LOOP(true, true, t_end - n_masked, t_end)
    PKH3_MFMA_DRAIN(w);
  } else {
    PKH3_TILE_LOOP(false, false, t_begin, t_end - n_masked)
    PKH3_TILE_LOOP(false, true, t_end - n_masked, t_end)
    PKH3_MFMA_DRAIN(w);
  }
#undef PKH3_TILE_LOOP
#undef PKH3_SHORT_LOOP

  if constexpr (SPARSE) {
    // Phase 2: the tiles that only some row-blocks keep.  Each row-block (a wave pair) walks its own list in
    // 32-key halves; an iteration gives every pair one half tile in its own LDS area, so all 8 waves stay
    // busy whichever rows a tile belongs to.  Two stages, the next half tile is copied while this one is used.
    const int r = wave >> 1;  // row-block of this wave inside the workgroup
    const int* mine = plan + (1 + r) * p.nKt;
    const int n_mine = uniform_load(plan_cnt, 1 + r);
    int n_longest = 0;  // every wave runs as many iterations as the longest list needs, so the barriers match
#pragma unroll
    for (int rr = 0; rr < kSparseRows; ++rr) n_longest = max(n_longest, uniform_load(plan_cnt, 1 + rr));
    const int n_iter = 2 * n_longest;
    constexpr int kKHalf = kKBytes / 2, kVHalf = kVTileBytes / 2;
    // this wave copies half of its pair's K half (and V half): K images are 1 KiB x (8 bf16 | 4 fp8) per half
    auto dma_half = [&](int it, int stage) {
      const int tile = uniform_load(mine, it >> 1);
      const int kb = it & 1;
      const char* g = p.kv + (int64_t)bh * p.kv_bh_stride + (int64_t)tile * p.kv_tile_stride;
      char* d = lds_raw + (stage * kSparseRows + r) * kHalfBytes;
      const int sub = wave & 1;
#pragma unroll
      for (int i = 0; i < kKHalf / 2048; ++i)
        lds_dma16(g + kb * kKHalf + (sub * (kKHalf / 2048) + i) * 1024, lane_off, d + (sub * (kKHalf / 2048) + i) * 1024);
#pragma unroll
      for (int i = 0; i < kVHalf / 2048; ++i)
        lds_dma16(g + kKBytes + kb * kVHalf + (sub * (kVHalf / 2048) + i) * 1024, lane_off,
                  d + kKHalf + (sub * (kVHalf / 2048) + i) * 1024);
    };
    __syncthreads();  // every wave is done with the phase-1 ring
    // kStages2 - 1 half tiles ahead: half tile `it` lives in stage it % kStages2
#pragma unroll
    for (int a = 0; a < kStages2 - 1; ++a)
      if (a < 2 * n_mine) dma_half(a, a);
    int st2 = 0, st2_free = kStages2 - 1;  // stage of half tile `it`, and the one the newest copy goes to
    // list entry and K scale of the half tile an iteration uses are asked for an iteration ahead
    int tile_next = n_mine > 0 ? uniform_load(mine, 0) : 0;
    float ks2_next = (FP8 && n_mine > 0) ? uniform_load(kscale, tile_next) : 1.0f;
#define PKH3_HALF_LOOP(STATIC)                                                                          \
  for (int it = 0; it < n_iter; ++it) {                                                                 \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                    \
    __syncthreads();                                                                                    \
    const char* hbuf = lds_raw + (st2 * kSparseRows + r) * kHalfBytes;                                  \
    const int st2_write = st2_free;                                                                     \
    st2_free = st2;                                                                                     \
    st2 = st2 == kStages2 - 1 ? 0 : st2 + 1;                                                            \
    if (it >= 2 * n_mine) continue; /* wave-uniform: this row-block has run out of tiles (and of copies) */ \
    const int tile = tile_next;                                                                         \
    const float ks = ks2_next;                                                                          \
    tile_next = uniform_load(mine, min(it + 1, 2 * n_mine - 1) >> 1);                                   \
    if (FP8) ks2_next = uniform_load(kscale, tile_next);                                                \
    /* the running-max copy needs registers for the rescale: it takes the lean read-ahead (4 images) */ \
    qk_half<FP8, !STATIC, POW2>(w, hbuf, hbuf + kKHalf, lane, e8m0_of(ks));                             \
    /* copies of the next half tile of this row-block: under the MFMAs of S^T (see the whole-tile loop) */ \
    if (it + kStages2 - 1 < 2 * n_mine) dma_half(it + kStages2 - 1, st2_write);                         \
    const float ct = (FP8 && !POW2) ? c * ks : c;                                                       \
    const int lim = (tail && tile == nkt - 1) ? tail - 32 * (it & 1) : 32;                              \
    softmax_pv_half<FP8, STATIC, !STATIC, false, POW2>(w, ct, lim, lane, hbuf + kKHalf);                \
  }
    if (static_max) {
      PKH3_HALF_LOOP(true)
      PKH3_MFMA_DRAIN(w);
    } else {
      PKH3_HALF_LOOP(false)
      PKH3_MFMA_DRAIN(w);
    }
#undef PKH3_HALF_LOOP
  }

  // Epilogue: O = O^T / l in bf16.  A lane holds 4 consecutive d of a query per accumulator, which would make 8-byte
  // stores scattered over 16 rows; instead each wave turns its 32 x 128 block around in its own 8 KiB of LDS
  // (16-byte chunks XOR-swizzled by the row so both directions are conflict-free) and stores whole 256-byte rows,
  // 16 bytes per lane.
  __bf16* ob = (__bf16*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
  __syncthreads();  // every wave is done reading K/V tiles: the LDS becomes staging space
  if constexpr (PARTS) {
    if (parts > 1) {
      // `parts` workgroups hold a share of this unit's result each.  Every wave leaves its partial result in global
      // scratch and counts itself in; the wave that finds all the others counted adds their partials to its own and
      // goes on to write the output, the others are done.  Partials and counter move through device-coherent
      // stores, loads and atomics: a wave counts itself in only after its stores have completed, and reads the
      // others' partials only after it has seen their counts.
      const int64_t wslot = kMergeBytes / 4;   // floats per wave
      float* mine = p.split_scratch + ((int64_t)(part_base + ul * parts + part) * WAVES + wave) * wslot;
#pragma unroll
      for (int db = 0; db < 8; ++db)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) store_device(mine + ((db * 2 + qb) * 64 + lane) * 4, w.o[db][qb]);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        store_device(mine + 64 * 64 + qb * 64 + lane, w.l[qb]);
        store_device(mine + 64 * 64 + 128 + qb * 64 + lane, w.m[qb]);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      int arrived = 0;
      if (lane == 0)
        arrived = __hip_atomic_fetch_add(p.split_cnt + (cnt_base + ul) * WAVES + wave, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      arrived = __builtin_amdgcn_readfirstlane(arrived);
      if (arrived != parts - 1) return;
      // The partials are added up in the order of the shares, whichever wave does it (its own comes back from the
      // scratch like the others), so the result does not depend on which workgroup finished last.
#pragma unroll 1
      for (int src = 0; src < parts; ++src) {
        const float* theirs = p.split_scratch + ((int64_t)(part_base + ul * parts + src) * WAVES + wave) * wslot;
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          const float l2 = load_device(theirs + 64 * 64 + qb * 64 + lane), m2 = load_device(theirs + 64 * 64 + 128 + qb * 64 + lane);
          // On the bounded-logit path nothing was subtracted, so numerators and row sums just add; on the
          // running-max path each side is first brought to the common maximum.  Share 0 starts the sum.
          float a1 = src == 0 ? 0.0f : 1.0f, a2 = 1.0f;
          if (!static_max && src != 0) {
            const float mn = fmaxf(w.m[qb], m2);
            a1 = mn == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(w.m[qb] - mn);
            a2 = mn == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m2 - mn);
            w.m[qb] = mn;
          } else if (src == 0) {
            w.m[qb] = m2;
          }
          w.l[qb] = src == 0 ? l2 : w.l[qb] * a1 + l2 * a2;
#pragma unroll
          for (int db = 0; db < 8; ++db) {
            const f32x4 v4 = load_device4(theirs + ((db * 2 + qb) * 64 + lane) * 4);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) w.o[db][qb][rr] = src == 0 ? v4[rr] : w.o[db][qb][rr] * a1 + v4[rr] * a2;
          }
        }
      }
    }
  }
  float inv[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const float lt = wave_sum_groups(w.l[qb]);
    inv[qb] = lt > 0.f ? 1.0f / lt : 0.f;
  }
  char* stage = lds_raw + wq * kStageBytes;
  {
    const int c16 = lane & 15, g = lane >> 4;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        bf16x4 wv;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) wv[rr] = (__bf16)(w.o[db][qb][rr] * inv[qb]);
        // elements d = 16*db + 4*g .. +3 of row 16*qb + c16: 16-byte chunk 2*db + g/2, its half g%2
        const int chunk = (2 * db + (g >> 1)) ^ c16;
        *(bf16x4*)(stage + (16 * qb + c16) * 256 + chunk * 16 + 8 * (g & 1)) = wv;
      }
  }
  // same wave wrote and reads: the LDS counter orders the two, no barrier
  if (p.o_images) {
    // operand images of the out-projection GEMM: image (16-row block, k-step h*4 + ks) holds, in lane (c = l % 16,
    // g = l / 16), elements 32*ks + 8*g .. +7 of this head for row c of the block -- one 1 KiB store per image
    if (q32 * 32 >= p.Sq) return;  // a block without rows: the buffer may end before it
    const int c16 = lane & 15, g4 = lane >> 4;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      const int r = 16 * rb + c16;
      const bool live = q32 * 32 + r < p.Sq;
      char* img = (char*)p.o + (int64_t)(q32 * 2 + rb) * p.o_img_blk_stride + (int64_t)h * (kD / 32) * 1024;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        bf16x8 v = *(const bf16x8*)(stage + r * 256 + (((4 * ks + g4) ^ (r & 15)) * 16));
        if (!live) v = bf16x8{};
        *(bf16x8*)(img + (ks * 64 + lane) * 16) = v;
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = 4 * i + (lane >> 4), c = lane & 15;
    const bf16x8 v = *(const bf16x8*)(stage + row * 256 + ((c ^ (row & 15)) * 16));
    const int q = q32 * 32 + row;
    if (q < p.Sq) *(bf16x8*)(ob + (int64_t)q * p.o_ss + 8 * c) = v;
  }
}

// The block-sparse kernel and the short-key dense kernel (the block-sparse one takes its units from the work queues
// when the launch has them: its workgroups differ in length with the tile lists on top of the XCDs' clocks).
template <bool FP8, bool SPARSE, int WAVES, bool POW2>
__global__ __launch_bounds__(64 * WAVES, (SPARSE ? 8 / WAVES : 3)) void attn_fwd_kernel(FwdParams p) {
  __shared__ __attribute__((aligned(1024))) char lds_raw[fwd_lds_bytes<FP8, SPARSE, WAVES>()];
  __shared__ int fetched_unit;
  int fetched = -1;
  if (p.queue_next) {   // wave-uniform
    if (threadIdx.x == 0) fetched_unit = fetch_unit(p.queue_next, blockIdx.x & (kQueues - 1), p.sec_units[0]);
    __syncthreads();
    fetched = __builtin_amdgcn_readfirstlane(fetched_unit);
    if (fetched < 0) return;
  }
  attn_fwd_body<FP8, SPARSE, WAVES, POW2>(p, blockIdx.x, 0, p.sec_units[0], 1, 0, 0, lds_raw, fetched);
}

// The long dense kernel: a launch of up to kSections sections, handed out in this order as CUs fall free.  Section 0
// holds whole units (one workgroup each); the later ones the units of a thinly filled last round, each shared out
// among sec_parts[] workgroups.  When the launch has work queues, every section's work is taken from queues of its own.
template <bool FP8, bool POW2>
__global__ __launch_bounds__(64 * kDenseWaves, 1) void attn_fwd_dense_kernel(FwdParams p) {
  __shared__ __attribute__((aligned(1024))) char lds_raw[fwd_lds_bytes<FP8, false, kDenseWaves>()];
  __shared__ int fetched_unit;
  static_assert(kSections == 3 && kSections * kQueues <= kQueueSlots, "the section look-up below is written out for three");
  const int bid = blockIdx.x, b0 = p.sec_blocks[0], b1 = p.sec_blocks[1];
  const int sec = (bid >= b0 ? 1 : 0) + (bid >= b0 + b1 ? 1 : 0);
  const int blk = bid - (sec >= 1 ? b0 : 0) - (sec >= 2 ? b1 : 0);
  const int unit0 = (sec >= 1 ? p.sec_units[0] : 0) + (sec >= 2 ? p.sec_units[1] : 0);
  const int units = sec == 0 ? p.sec_units[0] : sec == 1 ? p.sec_units[1] : p.sec_units[2];
  const int parts = sec == 0 ? p.sec_parts[0] : sec == 1 ? p.sec_parts[1] : p.sec_parts[2];
  // partial results and counters of section 2 lie behind those of section 1 (section 0 has none)
  const bool behind = sec == 2 && p.sec_parts[1] > 1;
  const int part_base = behind ? p.sec_units[1] * p.sec_parts[1] : 0, cnt_base = behind ? p.sec_units[1] : 0;
  int fetched = -1;
  if (p.queue_next) {   // wave-uniform; every section has queues of its own over its workgroups' work
    if (threadIdx.x == 0) fetched_unit = fetch_unit(p.queue_next + sec * kQueues, blk & (kQueues - 1), units * parts);
    __syncthreads();
    fetched = __builtin_amdgcn_readfirstlane(fetched_unit);
    if (fetched < 0) return;
  }
  attn_fwd_body<FP8, false, kDenseWaves, POW2>(p, blk, unit0, units, parts, part_base, cnt_base, lds_raw, fetched);
}

static int blocks_of(int workgroups) { return (workgroups + 7) / 8 * 8; }

// How a long dense call ends.  One 12-wave workgroup per CU at a time: the call runs in rounds of `cus` workgroups, and
// `rest` units left for a last round leave CUs idle for a whole workgroup's duration.  Sharing each of those units out
// among P workgroups (1/P of the key tiles each) gives workgroups of 1/P of the duration that again run in rounds of
// `cus`; one or two such sections (P1 for the units that fill a round, P2 for what is left) end the call in
// 1/P1 + 1/P2 of a whole round.  The cheapest plan within the scratch (one partial result per workgroup) is taken.
struct TailPlan {
  int units[2], parts[2];
};
static TailPlan plan_tail(int rest, int cus, int n_tiles, int64_t max_workgroups) {
  TailPlan best{{rest, 0}, {1, 1}};
  if (rest <= 0 || cus <= 0) return best;
  const int pmax = max(1, min(kMaxParts, n_tiles / kMinPartTiles));
  double best_cost = 1.0;
  auto consider = [&](int u1, int p1, int u2, int p2) {
    const int64_t wgs = (p1 > 1 ? (int64_t)u1 * p1 : 0) + (p2 > 1 ? (int64_t)u2 * p2 : 0);
    if (wgs > max_workgroups) return;
    const double cost = 1.0 / p1 + (u2 > 0 ? 1.0 / p2 : 0.0);
    if (cost < best_cost - 1e-9) best_cost = cost, best = TailPlan{{u1, u2}, {p1, p2}};
  };
  const int p_all = min(pmax, cus / rest);     // every unit of the rest in one round of workgroups
  if (p_all > 1) consider(rest, p_all, 0, 1);
  for (int p1 = 2; p1 <= pmax; ++p1) {
    const int u1 = cus / p1;                   // units that fill one round at p1
    if (u1 <= 0 || u1 >= rest) continue;
    const int p2 = min(pmax, cus / (rest - u1));
    if (p2 >= 1) consider(u1, p1, rest - u1, p2);
  }
  return best;
}

template <bool FP8, bool POW2 = false>
static hipError_t launch_fp(FwdParams p, int cus, hipStream_t st) {
  const int nQ32 = p.nQ64 * 2;
  auto units = [&](int blocks) { return p.B * p.H * ((nQ32 + blocks - 1) / blocks); };
  for (int i = 0; i < kSections; ++i) p.sec_units[i] = p.sec_blocks[i] = 0, p.sec_parts[i] = 1;
  if (p.plan) {
    const int n = units(kSparseWaves);
    p.sec_units[0] = n;
    int wgs = n;
    if (p.queue_next && cus > 0 && n >= cus) {
      // at least a round of workgroups: units from the work queues, an eighth more workgroups than units
      hipError_t e = launch_fill_zero((unsigned*)p.queue_next, kQueues, st);
      if (e != hipSuccess) return e;
      wgs += max(kQueues, n / 8);
    } else {
      p.queue_next = nullptr;
    }
    hipLaunchKernelGGL((attn_fwd_kernel<FP8, true, kSparseWaves, POW2>), dim3(blocks_of(wgs)), dim3(64 * kSparseWaves), 0, st, p);
    return hipGetLastError();
  }
  if (p.nKt <= kShortMaxTiles && !p.long_key_kernel) {
    p.queue_next = nullptr;
    p.sec_units[0] = units(kShortWaves);
    hipLaunchKernelGGL((attn_fwd_kernel<FP8, false, kShortWaves, POW2>), dim3(blocks_of(p.sec_units[0])), dim3(64 * kShortWaves), 0, st, p);
    return hipGetLastError();
  }
  const int n = units(kDenseWaves);
  const int whole = cus > 0 ? n / cus * cus : n, rest = n - whole;
  p.sec_units[0] = n;
  int shared = 0;   // units whose key tiles are shared out: they have arrival counters
  if (whole > 0 && rest > 0 && !p.long_key_kernel && p.split_cnt && p.split_scratch_bytes) {
    const int64_t cap = (int64_t)(p.split_scratch_bytes / ((size_t)kDenseWaves * kMergeBytes));
    const TailPlan t = plan_tail(rest, cus, p.nKt, cap);
    if (t.parts[0] > 1 || t.parts[1] > 1) {
      p.sec_units[0] = whole;
      p.sec_units[1] = t.units[0], p.sec_parts[1] = t.parts[0];
      p.sec_units[2] = t.units[1], p.sec_parts[2] = t.parts[1];
      shared = (t.parts[0] > 1 ? t.units[0] : 0) + (t.parts[1] > 1 ? t.units[1] : 0);
    }
  }
  // calls of at least one round of workgroups take their whole units from the work queues
  const bool queues = whole > 0 && !p.long_key_kernel && p.queue_next;
  if (!queues) p.queue_next = nullptr;
  if (queues || shared > 0) {
    // queue positions and arrival counters start at zero (the arrival counters follow the queue slots)
    hipError_t e = launch_fill_zero((unsigned*)(p.split_cnt - kQueueSlots), kQueueSlots + shared * kDenseWaves, st);
    if (e != hipSuccess) return e;
  }
  int blocks = 0;
  for (int i = 0; i < kSections; ++i) {
    int wgs = p.sec_units[i] * p.sec_parts[i];
    // the spare workgroups of the faster XCDs: an eighth on top of the whole units; as many again for the shared
    // units of the call's end, where an XCD that is through early can take most of a slower one's share
    if (queues && wgs > 0) wgs += i == 0 ? max(kQueues, wgs / 8) : wgs;
    blocks += p.sec_blocks[i] = blocks_of(wgs);
  }
  hipLaunchKernelGGL((attn_fwd_dense_kernel<FP8, POW2>), dim3(blocks), dim3(64 * kDenseWaves), 0, st, p);
  return hipGetLastError();
}

// CUs of the current device, asked once per device; threads that race here store the same value
hipError_t device_cu_count(int* out) {
  static std::atomic<int> cu_count[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  int cus = 0;
  if (dev >= 0 && dev < 64) {
    cus = cu_count[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
      e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      if (e != hipSuccess) return e;
      cu_count[dev].store(cus, std::memory_order_relaxed);
    }
  }
  *out = cus;
  return hipSuccess;
}

hipError_t launch_attn_fwd(const FwdParams& p, hipStream_t st) {
  int cus = 0;
  hipError_t e = device_cu_count(&cus);
  if (e != hipSuccess) return e;
  if (p.fp8 && p.fp8_pow2) return launch_fp<true, true>(p, cus, st);
  if (p.fp8) return launch_fp<true>(p, cus, st);
  return launch_fp<false>(p, cus, st);
}

// ------------------------------------------------------------------------------------------------
// Block-sparse plan.  For each workgroup (kSparseRows consecutive 64-query row-blocks) 1 + kSparseRows ascending
// tile lists, each `nKt` ints apart: [0] the key tiles every one of its row-blocks keeps (walked by all its waves
// together), [1+r] the tiles row-block r keeps that are not in [0] (walked by that row-block's wave pair).  One
// workgroup per attention workgroup merges the CSR rows through an LDS mask array, key tiles in chunks.
constexpr int kPlanChunk = 8192;

__global__ __launch_bounds__(256) void sparse_plan_kernel(const int* __restrict__ row_ptr, const int* __restrict__ col_idx,
                                                          int nRow64, int nKt, int* __restrict__ plan, int plan_stride,
                                                          int* __restrict__ plan_cnt) {
  __shared__ unsigned char mask[kPlanChunk];
  __shared__ int wave_tot[4];
  __shared__ int carry[kSparseLists];
  const int qt = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int* out = plan + (int64_t)qt * plan_stride;
  const int rows_here = max(0, min(kSparseRows, nRow64 - qt * kSparseRows));
  const int full = (1 << rows_here) - 1;
  if (tid < kSparseLists) carry[tid] = 0;
  for (int base = 0; base < nKt; base += kPlanChunk) {
    for (int i = tid; i < kPlanChunk; i += 256) mask[i] = 0;
    __syncthreads();
    for (int r = 0; r < rows_here; ++r) {
      const int row = qt * kSparseRows + r;
      const int beg = row_ptr[row], end = row_ptr[row + 1];
      for (int j = beg + tid; j < end; j += 256) {
        const int col = col_idx[j] - base;
        // within one r two threads touch the same byte only when the row repeats a column, and then both store the
        // same value; columns outside [0, nKt) are ignored; a row whose end lies before its start is empty
        if (col >= 0 && col < kPlanChunk && col + base < nKt) mask[col] |= (unsigned char)(1 << r);
      }
      __syncthreads();
    }
    for (int list = 0; list < kSparseLists; ++list) {
      for (int c0 = 0; c0 < kPlanChunk && base + c0 < nKt; c0 += 256) {
        const int col = c0 + tid;
        const int mk = (base + col < nKt) ? mask[col] : 0;
        const bool take = list == 0 ? (mk == full && full != 0) : (((mk >> (list - 1)) & 1) && mk != full);
        const unsigned long long bal = __ballot(take);
        const int before = __popcll(bal & ((1ull << lane) - 1ull));
        if (lane == 0) wave_tot[wave] = __popcll(bal);
        __syncthreads();
        int off = carry[list];
        for (int wv = 0; wv < wave; ++wv) off += wave_tot[wv];
        if (take) out[list * nKt + off + before] = base + col;
        __syncthreads();
        if (tid == 0) carry[list] += wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
        __syncthreads();
      }
    }
  }
  if (tid < kSparseLists) plan_cnt[qt * kSparseLists + tid] = carry[tid];
}

hipError_t launch_sparse_plan(const int* row_ptr, const int* col_idx, int nRow64, int nQ64, int nKt, int* plan,
                              int plan_stride, int* plan_cnt, hipStream_t st) {
  hipLaunchKernelGGL(sparse_plan_kernel, dim3(nQ64 / kSparseRows), dim3(256), 0, st, row_ptr, col_idx, nRow64, nKt, plan, plan_stride,
                     plan_cnt);
  return hipGetLastError();
}

}  // namespace pkh3
