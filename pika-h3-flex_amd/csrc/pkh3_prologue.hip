// Prologue kernels: everything that touches each Q/K/V row exactly once before the S x S work.
//   - key-mask compaction (prefix sum of the padding mask -> list of valid key rows)
//   - QK-RMSNorm + rotary embedding (+ optional fp8 e4m3 quantisation with per-64-row absmax scales),
//     written as MFMA operand images
//   - V re-laid out as the A-operand images of O^T = V^T P^T
//   - rotary cos/sin tables from the float64 position grid
// All of it is HBM-bound streaming work (a few hundred MB per layer call against ~29 TFLOP of
// attention), so the kernels are plain coalesced-store loops with no LDS staging.
#include "pkh3_common.h"
#include "pkh3_internal.h"

namespace pkh3 {

// ------------------------------------------------------------------------------------------------
// Key-mask compaction: idx[b][slot] = key index of the slot-th valid key, cnt[b] = number of valid keys.
// One workgroup of 1024 threads per batch walks the mask in chunks, carrying the running count.
__global__ __launch_bounds__(1024) void mask_compact_kernel(const uint8_t* __restrict__ mask, int Sk,
                                                            int* __restrict__ idx, int* __restrict__ cnt) {
  __shared__ int wave_tot[16];
  __shared__ int carry;
  const int b = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint8_t* m = mask + (int64_t)b * Sk;
  int* out = idx + (int64_t)b * Sk;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < Sk; base += 1024) {
    const int key = base + tid;
    const bool on = key < Sk && m[key] != 0;
    const unsigned long long bal = __ballot(on);
    const int before = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_tot[wave] = __popcll(bal);
    __syncthreads();
    int off = carry;
    for (int w = 0; w < wave; ++w) off += wave_tot[w];
    if (on) out[off + before] = key;
    __syncthreads();
    if (tid == 0) {
      int t = carry;
      for (int w = 0; w < 16; ++w) t += wave_tot[w];
      carry = t;
    }
    __syncthreads();
  }
  if (tid == 0) cnt[b] = carry;
}

hipError_t launch_mask_compact(const uint8_t* mask, int B, int Sk, int* idx, int* cnt, hipStream_t st) {
  hipLaunchKernelGGL(mask_compact_kernel, dim3(B), dim3(1024), 0, st, mask, Sk, idx, cnt);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// RMSNorm + RoPE (+ fp8 quantisation) of K rows into operand images (the Q side does the same math
// inside the attention kernel, on the rows each wave owns).
// One wave owns one 64-row tile of one (batch, head) and walks its four 16-row blocks, four lanes per row: lane
// (c = l%16, g = l/16) holds the 32 elements d = 32*ks + 8*g + j of row 16*kb + c -- its own 16 bytes of the block's
// four K images, so every load instruction reads 64 contiguous bytes of 16 rows, norm and rotation need two
// cross-lane exchanges (the sum of squares), and every store instruction writes one whole 1 KiB image.
template <bool FP8>
__global__ __launch_bounds__(256) void qk_prologue_kernel(QkPrologueParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // heads vary fastest across workgroups: neighbouring workgroups then read neighbouring pieces of the same
  // [S, H, D] rows at the same time
  const int blk = blockIdx.y * 4 + wave;
  if (blk >= p.nBlk64) return;
  const int h = blockIdx.x, b = blockIdx.z;
  const int c = lane & 15, g = lane >> 4;
  const int rows = p.row_cnt ? p.row_cnt[b] : p.S;
  const RowTransform tf{p.norm_w, p.eps, p.rope_mode, p.cos_t, p.sin_t};
  NormQuarter norm;
  if (p.norm_w) load_norm_quarter(norm, tf, g);
  char* ob = p.out + (int64_t)(b * p.H + h) * p.out_bh_stride + (int64_t)blk * p.out_blk_stride;
  float x[4][32];
  float nmax = 0.f, amax = 0.f;
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    const int row = blk * 64 + kb * 16 + c;
    const bool valid = row < rows;
    int src = 0;
    if (valid) src = p.gather_idx ? p.gather_idx[(int64_t)b * p.S + row] : row;
    RopeQuarter rope;
    if (p.rope_mode != 0 && valid) load_rope_quarter(rope, tf, src, g);
    const __bf16* xr = (const __bf16*)p.x + (int64_t)b * p.sb + (int64_t)src * p.ss + (int64_t)h * p.sh + 8 * g;
    bf16x8 raw[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) raw[ks] = *(const bf16x8*)(xr + 32 * ks);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) x[kb][ks * 8 + j] = valid ? (float)raw[ks][j] : 0.f;
    norm_rope_quarter(x[kb], tf, norm, rope, valid, g);
    float ssq = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      ssq += x[kb][i] * x[kb][i];
      amax = fmaxf(amax, fabsf(x[kb][i]));
    }
    nmax = fmaxf(nmax, wave_sum_groups(ssq));
    if constexpr (!FP8) {
      // image (half, ks, kb2) of the tile, half = kb / 2, kb2 = kb % 2: this lane's piece ks at its own place
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        bf16x8 t;
#pragma unroll
        for (int j = 0; j < 8; ++j) t[j] = (__bf16)x[kb][ks * 8 + j];
        *(bf16x8*)(ob + ((((kb >> 1) * 4 + ks) * 2 + (kb & 1)) * 64 + lane) * 16) = t;
      }
    }
  }
  if (p.norm_max) {
    // largest row norm of this (batch, head) after norm and rotation: an upper bound for every logit is
    // |q_i| * max_j |k_j|, which lets the attention kernel drop the running max when the bound is small
    nmax = sqrtf(wave_max(nmax));
    if (lane == 0) raise_max(p.norm_max + b * p.H + h, nmax);
  }
  if constexpr (FP8) {
    // one scale per 64-row tile; key block kb is 2 KiB, chunk c2 of a lane holds its pieces ks = 2*c2 and 2*c2 + 1
    amax = wave_max(amax);
    const float scale = fp8_block_scale(amax, p.fp8_pow2 != 0);
    const float inv = 1.0f / scale;
    if (lane == 0) p.scale_out[(int64_t)(b * p.H + h) * p.nBlk64 + blk] = scale;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        const i32x2 q0 = quant_fp8_piece(x[kb] + 16 * c2, inv), q1 = quant_fp8_piece(x[kb] + 16 * c2 + 8, inv);
        *(i32x4*)(ob + ((kb * 2 + c2) * 64 + lane) * 16) = i32x4{q0[0], q0[1], q1[0], q1[1]};
      }
  }
}

hipError_t launch_qk_prologue(const QkPrologueParams& p, hipStream_t st) {
  dim3 grid(p.H, (p.nBlk64 + 3) / 4, p.B);
  if (p.fp8)
    hipLaunchKernelGGL(qk_prologue_kernel<true>, grid, dim3(256), 0, st, p);
  else
    hipLaunchKernelGGL(qk_prologue_kernel<false>, grid, dim3(256), 0, st, p);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// V rows -> A-operand images of O^T = V^T P^T.  One wave per 64-key tile of one (batch, head).
// Lane (c, g) of image (half, db) needs V[32*half + v_image_key(g, j)][16*db + c] for j = 0..7: eight rows at
// one column.  Reads are 2-byte gathers (32 B contiguous per lane group, served from L1/L2); the
// stores are full 1 KiB lines.
__global__ __launch_bounds__(256) void v_prologue_kernel(VPrologueParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = blockIdx.y * 4 + wave;
  if (t >= p.nKt) return;
  const int h = blockIdx.x, b = blockIdx.z;  // heads fastest, as in the K prologue
  const int c = lane & 15, g = lane >> 4;
  if (t == 0 && lane == 0) p.zero_init[b * p.H + h] = 0u;
  const int rows = p.row_cnt ? p.row_cnt[b] : p.S;
  const __bf16* vb = (const __bf16*)p.v + (int64_t)b * p.sb + (int64_t)h * p.sh;
  char* ob = p.out + (int64_t)(b * p.H + h) * p.out_bh_stride + (int64_t)t * p.out_tile_stride;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    bf16x8 img[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = t * 64 + half * 32 + v_image_key(g, j);
      const bool valid = row < rows;
      int src = 0;
      if (valid) src = p.gather_idx ? p.gather_idx[(int64_t)b * p.S + row] : row;
      const __bf16* vr = vb + (int64_t)src * p.ss + c;
#pragma unroll
      for (int db = 0; db < 8; ++db) img[db][j] = valid ? vr[16 * db] : (__bf16)0.0f;
    }
#pragma unroll
    for (int db = 0; db < 8; ++db) *(bf16x8*)(ob + ((half * 8 + db) * 64 + lane) * 16) = img[db];
  }
}

hipError_t launch_v_prologue(const VPrologueParams& p, hipStream_t st) {
  dim3 grid(p.H, (p.nKt + 3) / 4, p.B);
  hipLaunchKernelGGL(v_prologue_kernel, grid, dim3(256), 0, st, p);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// cos/sin tables from the [S,3] float64 position grid.  Pair p of the D/2 = 64 pairs belongs to the
// axis whose slice contains it; inside its slice of n = axis_dims[a]/2 pairs, pair i rotates by
// pos[a] * theta^(-2i / axis_dims[a]).  Computed in float64, stored fp32.
__global__ void rope_tables_kernel(const double* __restrict__ pos, int S, int d0, int d1, int d2, double log_theta,
                                   float* __restrict__ cos_out, float* __restrict__ sin_out) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (int64_t)S * (kD / 2)) return;
  const int s = (int)(gid / (kD / 2)), pr = (int)(gid % (kD / 2));
  int a, i, dim;
  if (pr < d0 / 2) { a = 0; i = pr; dim = d0; }
  else if (pr < (d0 + d1) / 2) { a = 1; i = pr - d0 / 2; dim = d1; }
  else { a = 2; i = pr - (d0 + d1) / 2; dim = d2; }
  const double freq = exp(-log_theta * (2.0 * i) / (double)dim);
  const double ang = pos[(int64_t)s * 3 + a] * freq;
  cos_out[gid] = (float)cos(ang);
  sin_out[gid] = (float)sin(ang);
}

hipError_t launch_rope_tables(const double* pos, int S, const int* axis_dims, double theta, float* cos_out,
                              float* sin_out, hipStream_t st) {
  const int64_t n = (int64_t)S * (kD / 2);
  hipLaunchKernelGGL(rope_tables_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, pos, S, axis_dims[0],
                     axis_dims[1], axis_dims[2], log(theta), cos_out, sin_out);
  return hipGetLastError();
}

}  // namespace pkh3
