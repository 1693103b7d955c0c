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

}  // namespace pkh3
