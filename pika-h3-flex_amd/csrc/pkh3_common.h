// Shared device-side definitions for the gfx950 attention kernels: vector types, the fragment
// ("frag") layouts the prologue writes and the attention kernels consume, and small wave helpers.
//
// Fragment layouts.  All matrix work uses the CDNA4 32x32 MFMA shapes.  For those, lane l of a
// wave supplies row/column (l % 32) of an operand and a contiguous run of the contraction index
// selected by its half hh = l / 32; the 32x32 fp32 result puts column (l % 32) in lane l and rows
// 8*(i/4) + 4*hh + (i%4) in its 16 registers i.  The prologue stores Q, K and V in HBM already cut
// into 1 KiB operand images (64 lanes x 16 B), so the attention kernel moves them HBM -> LDS ->
// VGPR as straight 16-byte copies with no shuffles and no LDS bank conflicts.
//
//   K tile (64 keys, bf16): image (kb, ks), kb in 0..1, ks in 0..7, at byte ((kb*8+ks)*64 + l)*16
//       holds K'[32*kb + l%32][16*ks + 8*hh + j], j = 0..7            (A operand of S^T = K' Q'^T)
//   Q block (32 queries, bf16): image ks at ((ks)*64 + l)*16 holds Q'[l%32][16*ks + 8*hh + j]
//       (B operand of S^T)
//   V tile (64 keys, bf16): image (kb, b2, db), b2 in 0..1, db in 0..3, at (((kb*2+b2)*4+db)*64 + l)*16
//       holds V[32*kb + 8*(2*b2 + j/4) + 4*hh + j%4][32*db + l%32]      (A operand of O^T = V^T P^T)
//       -- the key order is the one the S^T result registers 8*b2 .. 8*b2+7 already have, so P goes
//       from the softmax registers into the next MFMA without leaving the lane.
//   fp8 K tile / Q block: image (kb, ks64), 32 B per lane: byte j of lane l is element
//       d = 16*(4*ks64 + j/8) + 8*hh + j%8 of row 32*kb + l%32 -- the same lane-to-d assignment as
//       the bf16 images, four of them concatenated; Q and K use it alike, which is all the
//       contraction needs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pkh3 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;

constexpr int kD = 128;            // head dim (fixed)
constexpr int kTileKeys = 64;      // keys per K/V tile, also the block-sparse tile edge
constexpr int kKTileBytes = 16384; // bf16 K tile
constexpr int kK8TileBytes = 8192; // fp8 K tile
constexpr int kVTileBytes = 16384; // bf16 V tile
constexpr int kQBlkBytes = 8192;   // bf16 Q block of 32 queries
constexpr int kQ8BlkBytes = 4096;  // fp8 Q block of 32 queries
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kFp8Max = 448.0f;  // OCP e4m3fn

__device__ __forceinline__ float xhalf(float x) {
  // value held by the lane 32 away (the other half of the wave)
  return __shfl_xor(x, 32, 64);
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}

// RMSNorm + rotation of one row, shared by the K prologue and the attention kernel's Q load.
// `x` holds this lane's 64 elements d = 16*ks + 8*hh + j (index ks*8 + j) of the row; lane l^32 holds
// the other 64, so the sum of squares needs one exchange and both pairings of the rotation
// (interleaved (2i,2i+1) / half-split (i,i+64)) stay inside the lane.
struct RowTransform {
  const float* norm_w;  // [D] or null
  float eps;
  int rope_mode;        // 0 none, 1 interleaved, 2 half-split
  const float* cos_t;   // [rows, D/2]
  const float* sin_t;
};

// `row` must be readable even when !valid (callers point it at row 0); the values are then zeroed.
__device__ __forceinline__ void load_row(float (&x)[64], const __bf16* row, bool valid, int hh) {
  bf16x8 t[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) t[ks] = *(const bf16x8*)(row + 16 * ks + 8 * hh);
#pragma unroll
  for (int ks = 0; ks < 8; ++ks)
#pragma unroll
    for (int j = 0; j < 8; ++j) x[ks * 8 + j] = valid ? (float)t[ks][j] : 0.f;
}

__device__ __forceinline__ void norm_rope_row(float (&x)[64], const RowTransform& t, int64_t table_row, bool valid,
                                              int hh) {
  if (t.norm_w) {
    float ssq = 0.f;
#pragma unroll
    for (int i = 0; i < 64; ++i) ssq += x[i] * x[i];
    ssq += xhalf(ssq);
    // an all-zero row with eps == 0 stays all zero instead of 0 * inf
    const float ms = ssq * (1.0f / kD) + t.eps;
    const float rs = ms > 0.f ? rsqrtf(ms) : 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const f32x4 w0 = *(const f32x4*)(t.norm_w + 16 * ks + 8 * hh);
      const f32x4 w1 = *(const f32x4*)(t.norm_w + 16 * ks + 8 * hh + 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[ks * 8 + j] *= rs * w0[j];
        x[ks * 8 + 4 + j] *= rs * w1[j];
      }
    }
  }
  if (t.rope_mode == 1 && valid) {
    // interleaved pairs (2i, 2i+1): pair index 8*ks + 4*hh + jj for this lane's elements 2jj, 2jj+1
    const float* ct = t.cos_t + table_row * (kD / 2);
    const float* st = t.sin_t + table_row * (kD / 2);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const f32x4 c = *(const f32x4*)(ct + 8 * ks + 4 * hh);
      const f32x4 s = *(const f32x4*)(st + 8 * ks + 4 * hh);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const float a0 = x[ks * 8 + 2 * jj], a1 = x[ks * 8 + 2 * jj + 1];
        x[ks * 8 + 2 * jj] = a0 * c[jj] - a1 * s[jj];
        x[ks * 8 + 2 * jj + 1] = a1 * c[jj] + a0 * s[jj];
      }
    }
  } else if (t.rope_mode == 2 && valid) {
    // half-split pairs (i, i + 64): element d < 64 of this lane sits at ks < 4, its partner at ks + 4
    const float* ct = t.cos_t + table_row * (kD / 2);
    const float* st = t.sin_t + table_row * (kD / 2);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const f32x4 c0 = *(const f32x4*)(ct + 16 * ks + 8 * hh), c1 = *(const f32x4*)(ct + 16 * ks + 8 * hh + 4);
      const f32x4 s0 = *(const f32x4*)(st + 16 * ks + 8 * hh), s1 = *(const f32x4*)(st + 16 * ks + 8 * hh + 4);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float cj = j < 4 ? c0[j & 3] : c1[j & 3], sj = j < 4 ? s0[j & 3] : s1[j & 3];
        const float lo = x[ks * 8 + j], hi = x[(ks + 4) * 8 + j];
        x[ks * 8 + j] = lo * cj - hi * sj;
        x[(ks + 4) * 8 + j] = hi * cj + lo * sj;
      }
    }
  }
}

// values 16*c .. 16*c+15 of a lane's row -> one 16-byte chunk of an fp8 e4m3 image
__device__ __forceinline__ i32x4 quant_fp8_chunk(const float (&x)[64], int c, float inv) {
  i32x4 t;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int e = 16 * c + 4 * w;
    int v = 0;
    v = __builtin_amdgcn_cvt_pk_fp8_f32(x[e] * inv, x[e + 1] * inv, v, false);
    v = __builtin_amdgcn_cvt_pk_fp8_f32(x[e + 2] * inv, x[e + 3] * inv, v, true);
    t[w] = v;
  }
  return t;
}

}  // namespace pkh3
