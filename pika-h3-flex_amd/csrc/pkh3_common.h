// Shared device-side definitions for the gfx950 attention kernels: vector types, the operand-image
// layouts the prologue (or the projection GEMM's epilogue) writes and the attention kernel consumes,
// and small wave helpers.
//
// Operand images.  The attention kernel runs on the CDNA4 16x16 MFMA shapes (16x16x32 bf16, 16x16x128 fp8):
// at the same peak rate they move a quarter of the accumulator registers per instruction of the 32x32 shapes,
// and the part sustains about 10 % more of them per second on real data.  For those shapes lane l of a wave
// supplies row/column c = l % 16 of an operand and the 8 consecutive contraction elements selected by its group
// g = l / 16; the 16x16 fp32 result puts column c in lane l and rows 4*g + i in its 4 registers i.  K and V are
// stored in HBM already cut into 1 KiB images (64 lanes x 16 B) in exactly that order, so the attention kernel
// moves them HBM -> LDS -> VGPR as straight 16-byte copies with no shuffles and no LDS bank conflicts.
//
//   K tile (64 keys, bf16, 16 KiB): image (half, ks, kb2), half in 0..1, ks in 0..3, kb2 in 0..1, at byte
//       (((half*4 + ks)*2 + kb2)*64 + l)*16 holds K'[32*half + 16*kb2 + c][32*ks + 8*g + j], j = 0..7
//       (A operand of S^T = K' Q'^T; the 32-key halves are contiguous for the half-tile forms of the kernel)
//   Q block (32 queries, bf16, registers only): image (qb, ks) holds Q'[16*qb + c][32*ks + 8*g + j]
//       (B operand of S^T)
//   V tile (64 keys, bf16, 16 KiB): image (half, db), db in 0..7, at ((half*8 + db)*64 + l)*16 holds
//       V[32*half + 16*(j/4) + 4*g + j%4][16*db + c], j = 0..7      (A operand of O^T = V^T P^T)
//       -- the key order is the one the S^T result registers of key blocks 2*half and 2*half+1 already have,
//       so P goes from the softmax registers into the next MFMA without leaving the lane.
//   fp8 K tile (8 KiB): key block kb in 0..3 is 2 KiB, 32 B per lane as two 16-byte chunks c2 at
//       ((kb*2 + c2)*64 + l)*16; byte 8*(ks%2) + j of chunk c2 = ks/2 is element d = 32*ks + 8*g + j of row
//       16*kb + c -- the same lane-to-d assignment as the bf16 images; Q uses it alike, which is all the
//       contraction needs.
//
// Rows are prepared (RMSNorm, rotation, quantisation) in the layout of the images themselves, four lanes per row
// (norm_rope_quarter below): by the K prologue, by the K epilogue of the projection GEMM and by the attention
// kernel's Q load.
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

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}

// RMSNorm + rotation of one row: what is done to it (norm_rope_quarter below does it).
struct RowTransform {
  const float* norm_w;  // [D] or null
  float eps;
  int rope_mode;        // 0 none, 1 interleaved, 2 half-split
  const float* cos_t;   // [rows, D/2]
  const float* sin_t;
};

// *slot = max(*slot, v) for non-negative floats kept as their bit patterns (they order like unsigned integers).
// Thousands of waves raise the same few words: atomics on one address are served one after the other, so the word is
// read first and the atomic only issued by a wave that would raise it (the value only grows, so a wave that sees an
// older, smaller one merely issues an atomic it did not need).
__device__ __forceinline__ void raise_max(unsigned* slot, float v) {
  const unsigned bits = __float_as_uint(v);
  if (bits > __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(slot, bits);
}

__device__ __forceinline__ float wave_sum_groups(float x) {
  // sum over the four lanes l % 16 == const (one per 16-lane group)
  x += __shfl_xor(x, 16, 64);
  x += __shfl_xor(x, 32, 64);
  return x;
}

// ---- four lanes per row: the layout of the 16x16 operand images themselves ----
// Lane (c = l % 16, g = l / 16) holds the pieces p8 = 4*ks + g of row c of a 16-row block, i.e. elements
// d = 32*ks + 8*g + j at x[8*ks + j]; the three other lane groups (lanes l ^ 16, l ^ 32, l ^ 48) hold the rest of the
// row, so the sum of squares needs two exchanges and both pairings of the rotation (interleaved (2i, 2i+1) /
// half-split (i, i+64): ks and ks + 2) stay inside the lane.  What a lane holds is exactly its 16 bytes of the four K
// images (ks = 0..3) of its 16-row block, so rows prepared this way are stored, or fed to the MFMA, without any lane
// movement.

// The rotation tables of one row as its lane group uses them (8 vectors of 4).  Interleaved: c[ks] = pairs
// 16*ks + 4*g .. +3 (elements 2jj, 2jj+1 of piece ks).  Half-split: c[2*ks], c[2*ks+1] = pairs 32*ks + 8*g .. +7
// (element j of piece ks with its partner in piece ks + 2), ks = 0, 1.
struct RopeQuarter {
  f32x4 c[4], s[4];
};

__device__ __forceinline__ void load_rope_quarter(RopeQuarter& r, const RowTransform& t, int64_t table_row, int g) {
  const float* ct = t.cos_t + table_row * (kD / 2);
  const float* st = t.sin_t + table_row * (kD / 2);
  if (t.rope_mode == 1) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      r.c[ks] = *(const f32x4*)(ct + 16 * ks + 4 * g);
      r.s[ks] = *(const f32x4*)(st + 16 * ks + 4 * g);
    }
  } else if (t.rope_mode == 2) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      r.c[2 * ks] = *(const f32x4*)(ct + 32 * ks + 8 * g), r.c[2 * ks + 1] = *(const f32x4*)(ct + 32 * ks + 8 * g + 4);
      r.s[2 * ks] = *(const f32x4*)(st + 32 * ks + 8 * g), r.s[2 * ks + 1] = *(const f32x4*)(st + 32 * ks + 8 * g + 4);
    }
  }
}

// The RMSNorm weights of this lane's 32 elements: w[2*ks], w[2*ks + 1] = weights 32*ks + 8*g .. +7
struct NormQuarter {
  f32x4 w[8];
};

__device__ __forceinline__ void load_norm_quarter(NormQuarter& n, const RowTransform& t, int g) {
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    n.w[2 * ks] = *(const f32x4*)(t.norm_w + 32 * ks + 8 * g);
    n.w[2 * ks + 1] = *(const f32x4*)(t.norm_w + 32 * ks + 8 * g + 4);
  }
}

// RMSNorm and rotation of this lane's 32 elements of a row, with the weights and the row's tables already in registers
__device__ __forceinline__ void norm_rope_quarter(float (&x)[32], const RowTransform& t, const NormQuarter& n, const RopeQuarter& r,
                                                  bool valid, int g) {
  if (t.norm_w) {
    float ssq = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) ssq += x[i] * x[i];
    ssq = wave_sum_groups(ssq);
    // an all-zero row with eps == 0 stays all zero instead of 0 * inf
    const float ms = ssq * (1.0f / kD) + t.eps;
    const float rs = ms > 0.f ? rsqrtf(ms) : 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[ks * 8 + j] *= rs * n.w[2 * ks][j];
        x[ks * 8 + 4 + j] *= rs * n.w[2 * ks + 1][j];
      }
  }
  if (t.rope_mode == 1 && valid) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const float a0 = x[ks * 8 + 2 * jj], a1 = x[ks * 8 + 2 * jj + 1];
        x[ks * 8 + 2 * jj] = a0 * r.c[ks][jj] - a1 * r.s[ks][jj];
        x[ks * 8 + 2 * jj + 1] = a1 * r.c[ks][jj] + a0 * r.s[ks][jj];
      }
  } else if (t.rope_mode == 2 && valid) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float cj = r.c[2 * ks + (j >> 2)][j & 3], sj = r.s[2 * ks + (j >> 2)][j & 3];
        const float lo = x[ks * 8 + j], hi = x[(ks + 2) * 8 + j];
        x[ks * 8 + j] = lo * cj - hi * sj;
        x[(ks + 2) * 8 + j] = hi * cj + lo * sj;
      }
  }
}

__device__ __forceinline__ void norm_rope_quarter(float (&x)[32], const RowTransform& t, int64_t table_row, bool valid, int g) {
  NormQuarter n;
  RopeQuarter r;
  if (t.norm_w) load_norm_quarter(n, t, g);
  if (t.rope_mode != 0 && valid) load_rope_quarter(r, t, table_row, g);
  norm_rope_quarter(x, t, n, r, valid, g);
}

// eight values -> eight fp8 e4m3 bytes
__device__ __forceinline__ i32x2 quant_fp8_piece(const float* x, float inv) {
  i32x2 t;
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    int v = 0;
    v = __builtin_amdgcn_cvt_pk_fp8_f32(x[4 * w] * inv, x[4 * w + 1] * inv, v, false);
    v = __builtin_amdgcn_cvt_pk_fp8_f32(x[4 * w + 2] * inv, x[4 * w + 3] * inv, v, true);
    t[w] = v;
  }
  return t;
}

// key (inside its 32-key half) that element j of lane group g carries in a V image / in the P operand
__device__ __forceinline__ int v_image_key(int g, int j) { return 16 * (j >> 2) + 4 * g + (j & 3); }

// Dequantisation scale of an fp8 block whose largest magnitude is `amax`: amax / 448, or, with `pow2`, the smallest
// power of two that is at least that (the form the scaled MFMA takes as an operand: an 8-bit exponent).  The product
// amax * fl(1/448) is rounded to float32 first and the power of two is taken of that number.  A block of zeros gets 1.
__device__ __forceinline__ float fp8_block_scale(float amax, bool pow2) {
  if (!(amax > 0.f)) return 1.0f;
  const float s = amax * (1.0f / kFp8Max);
  if (!pow2) return s;
  const unsigned bits = __float_as_uint(s);
  unsigned e = (bits >> 23) & 0xffu;
  if (bits & 0x7fffffu) ++e;
  e = e < 1u ? 1u : (e > 254u ? 254u : e);
  return __uint_as_float(e << 23);
}

// the 8-bit exponent (E8M0: value 2^(e - 127)) of a power-of-two scale, as the scaled MFMA takes it
__device__ __forceinline__ int e8m0_of(float pow2_scale) { return (int)((__float_as_uint(pow2_scale) >> 23) & 0xffu); }

constexpr int kQueues = 8;       // work queues of a launch: one per XCD

// Work queues of a launch's units.  The XCDs of one part hold different clocks under the power cap
// (a few per cent apart), and the hardware deals workgroups to them round-robin, an eighth each whatever their speed,
// so with a fixed workgroup -> unit map the call lasts as long as its slowest XCD needs for its eighth.  Instead every
// XCD has a queue (a counter) over its contiguous run of units: a workgroup takes the next unit of its own XCD's queue
// and, when that is empty, of the queue with the most units left; the launch holds an eighth more workgroups than
// units, so an XCD that is through early keeps getting workgroups, which take units off the slower ones.  A workgroup
// that finds every queue empty exits.  Returns the unit (index inside the section) or -1.
__device__ __forceinline__ int fetch_unit(int* queue_next, int home, int units) {
  const int per = (units + kQueues - 1) / kQueues;
  int q = home;
  // Every pass either takes a unit, or finds all queues empty, or lost a unit to another workgroup (which is
  // progress of the launch as a whole: the positions only grow), so the loop ends.
#pragma unroll 1
  for (;;) {
    const int size = max(0, min(per, units - q * per));
    // a look first: a queue that is empty stays empty, no need to count it further up
    if (__hip_atomic_load(queue_next + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < size) {
      const int i = __hip_atomic_fetch_add(queue_next + q, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (i < size) return q * per + i;
    }
    int best = -1, most = 0;
    for (int j = 0; j < kQueues; ++j) {
      const int left = max(0, min(per, units - j * per)) - __hip_atomic_load(queue_next + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (left > most) most = left, best = j;
    }
    if (best < 0) return -1;
    q = best;
  }
}

}  // namespace pkh3
