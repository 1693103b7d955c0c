// Projection GEMMs around the attention kernel (gfx950, bf16 MFMA 32x32x16, fp32 accumulation):
//   to_q / to_k / to_v  (+ LoRA)  from the modulated hidden states, with the K side's RMSNorm + rotation
//                       (+ fp8 quantisation) and the K / V operand-image layout done in the epilogue, so that
//                       K and V go from the accumulators straight into the records the attention kernel reads
//   to_out.0 (+ LoRA)   from the attention output, with bias, per-row gate and residual in the epilogue
//   LoRA down-projection x A^T, written as operand images for the second K segment of the GEMMs above
//
// Operands.  Both operands come as 1 KiB operand images (32 rows x 16 contraction elements, lane l holds row
// l%32, elements 8*(l/32)..+7): activations as [token block][k-step], weights as [feature block][k-step] (packed
// once when the weights are loaded).  They move HBM/L2 -> LDS -> VGPR as straight 16-byte copies, like the K/V
// tiles of the attention kernel: direct-to-LDS loads into a 4-slot ring, three chunks ahead, one barrier per chunk.
// Since the two MFMA operands have the same register form, one pair of images serves both orientations:
//   C^T = W x^T  (features down the accumulator registers, one token per lane)   Q, K, row-major outputs
//   C   = x W^T  (tokens down the registers, one feature per lane)               V images
// Weight rows are stored permuted inside each 128-feature head so that, in the C^T form, the 64 accumulator
// values of a lane are exactly the 64 head-dim elements d = 16*ks + 8*hh + j the row transform
// (norm_rope_row) works on: whole 8-element pieces of the row, which the epilogue stores at their places in the
// attention kernel's K tile (a different image shape: that kernel runs on the 16x16 MFMAs, these GEMMs on 32x32).
//
// Work split.  Workgroup = 8 waves = 256 tokens x 256 features; wave (fh, tq) owns features fh*128..+127 (one
// head) x tokens tq*64..+63 (one K/V tile): 8 accumulators of 32x32.  Per 32-wide k-chunk a wave reads 8 weight
// and 4 activation images for 16 MFMAs.  LoRA is a second K segment: k-chunks beyond the hidden size take their
// activation images from the down-projected rows (x A^T, scaled) and their weight images from B.
#include <type_traits>

#include "pkh3_common.h"
#include "pkh3_internal.h"

namespace pkh3 {

constexpr int kGemmWaves = 8;
constexpr int kGemmTile = 256;                      // tokens and features per workgroup
constexpr int kGemmChunkK = 32;                     // contraction elements per ring slot
constexpr int kGemmStageBytes = 2 * kGemmTile * kGemmChunkK * 2;  // weight part + activation part
constexpr int kGemmRing = 4;

__device__ __forceinline__ void gemm_dma16(const char* g, unsigned lane_off, char* l) {
  // see lds_dma16 in pkh3_attn_fwd.hip: wave-uniform base addresses, per-lane byte offset, tracked by vmcnt
  const unsigned lds_addr = (unsigned)(size_t)(__attribute__((address_space(3))) char*)l;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_off), "s"(g), "s"(lds_addr)
               : "memory", "m0");
}

// In the C^T form, accumulator value (db, i) of a lane with half hh is head-dim element
// 16 * (2*db + (i >> 3)) + 8*hh + (i & 7) of the lane's token: element (ks, j) = (2*db + (i >> 3), i & 7) of the
// lane's row in the layout of norm_rope_row, i.e. index 16*db + i of its x[64] (see pack_rows_kernel for the
// weight-row permutation that makes it so).

// WAVES = 8 (the form that ships): wave tile 128 features x 64 tokens, two waves per SIMD, accumulators in 128 VGPRs.
// WAVES = 4 (wave tile 128 x 128, one wave per SIMD, 256 accumulator registers, half the LDS reads per MFMA) compiles
// and passes the same tests but measured four times slower: with more than 256 registers the compiler moves
// accumulators between the two register files inside the loop.
template <int EPI, int WAVES>
__device__ __forceinline__ void gemm_tile(const GemmParams& p, const GemmTarget& tg, int m_tile, int n_tile_in_target,
                                          char* lds_raw) {
  constexpr int TB = 16 / WAVES;                     // 32-token blocks per wave
  constexpr int PP = 32 / WAVES;                     // 1 KiB pieces of a chunk each wave copies
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int hh = lane >> 5, r = lane & 31;
  const int fh = wave & 1, tq = wave >> 1;           // feature half (one head), token slice
  const int head = n_tile_in_target * 2 + fh;        // 128-feature head inside the target
  const bool head_live = head * 128 < tg.n;
  const int nk1 = p.nk1, nk = p.nk1 + tg.nk2;
  const unsigned lane_off = lane * 16;

  // this wave's 1 KiB pieces of every chunk: pieces PP*wave.. of [8 weight blocks x 2 k-steps | 8 token blocks x 2]
  const int piece0 = wave * PP;
  const bool w_side = piece0 < 16;
  const int blk0 = (piece0 & 15) >> 1;               // first of the 32-row blocks this wave copies
  const char* seg1 = w_side ? tg.w_img + (int64_t)(n_tile_in_target * 8 + blk0) * tg.w_blk_stride
                            : p.a_img + (int64_t)(m_tile * 8 + blk0) * p.a_blk_stride;
  const int64_t seg1_step = w_side ? tg.w_blk_stride : p.a_blk_stride;
  const char* seg2 = w_side ? tg.w2_img + (int64_t)(n_tile_in_target * 8 + blk0) * tg.w2_blk_stride
                            : tg.a2_img + (int64_t)(m_tile * 8 + blk0) * tg.a2_blk_stride;
  const int64_t seg2_step = w_side ? tg.w2_blk_stride : tg.a2_blk_stride;
  // this wave's copies of one chunk: PP pieces of 1 KiB from `g` (two consecutive k-step images of one block are
  // contiguous, 2 KiB; the next block is `step` bytes on) into ring slot `slot`
  auto dma_from = [&](const char* g, int64_t step, int slot) {
    char* d = lds_raw + slot * kGemmStageBytes + piece0 * 1024;
#pragma unroll
    for (int b = 0; b < PP / 2; ++b) {
      gemm_dma16(g + b * step, lane_off, d + b * 2048);
      gemm_dma16(g + b * step + 1024, lane_off, d + b * 2048 + 1024);
    }
  };
  auto dma = [&](int kc, int slot) {
    const bool first = kc < nk1;
    dma_from(first ? seg1 + (int64_t)kc * 2048 : seg2 + (int64_t)(kc - nk1) * 2048, first ? seg1_step : seg2_step, slot);
  };
  // waits until at most `chunks` of this wave's newest chunk copies are still in flight
  auto wait_dma = [&](int chunks) {
    if (chunks >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PP) : "memory");
    else if (chunks == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PP) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };

  f32x16 acc[TB][4];
#pragma unroll
  for (int t2 = 0; t2 < TB; ++t2)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[t2][db][i] = 0.f;

  // Ring of four chunks.  Entering iteration kc: chunk kc is in LDS for every wave and its first k-step's images are
  // already on their way to this wave's registers; chunks kc+1 and kc+2 are in flight.  The barrier at the top makes
  // chunk kc+1 visible and frees the slot of chunk kc-1 for chunk kc+3, so the first images of the next chunk can be
  // read at the tail of this iteration and no wave starts a chunk by waiting for LDS.
  const int n_pre = nk < 3 ? nk : 3;
  for (int c = 0; c < n_pre; ++c) dma(c, c);
  wait_dma(n_pre - 1);
  __syncthreads();
  const int w_off = (fh * 4) * 2048 + lane * 16;            // weight blocks fh*4..+3 of a slot
  const int a_off = 16384 + (tq * TB) * 2048 + lane * 16;   // this wave's token blocks
  bf16x8 wf[2][4], xf[2][TB];
  auto read_frags = [&](int slot, int ks, bf16x8 (&w4)[4], bf16x8 (&xt)[TB]) {
    const char* base = lds_raw + slot * kGemmStageBytes + ks * 1024;
#pragma unroll
    for (int db = 0; db < 4; ++db) w4[db] = *(const bf16x8*)(base + w_off + db * 2048);
#pragma unroll
    for (int t2 = 0; t2 < TB; ++t2) xt[t2] = *(const bf16x8*)(base + a_off + t2 * 2048);
  };
  auto mfmas = [&](const bf16x8 (&w4)[4], const bf16x8 (&xt)[TB]) {
#pragma unroll
    for (int t2 = 0; t2 < TB; ++t2)
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        if constexpr (EPI == kEpiVImg) acc[t2][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xt[t2], w4[db], acc[t2][db], 0, 0, 0);
        else acc[t2][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w4[db], xt[t2], acc[t2][db], 0, 0, 0);
      }
  };
  if (head_live) read_frags(0, 0, wf[0], xf[0]);
  int slot = 0;
  // source of the next chunk to copy (chunk kc + 3 in the steady loop): a running pointer inside its K segment
  const char* g_next = nullptr;
  int64_t step_next = seg1_step;
  int left_next = 0;  // chunks left in the segment g_next walks, this one included
  if (nk > 3) {
    const bool first = 3 < nk1;
    g_next = first ? seg1 + 3 * 2048 : seg2 + (int64_t)(3 - nk1) * 2048;
    step_next = first ? seg1_step : seg2_step;
    left_next = first ? nk1 - 3 : nk - 3;
  }
  // One chunk.  MORE1/2/3: chunks kc+1 / kc+2 / kc+3 exist (compile-time, so the steady loop carries no tests).
  auto chunk = [&](auto more1, auto more2, auto more3) {
    if constexpr (more1()) {
      // chunk kc+1 has landed (this wave's pieces; the barrier covers the others'); only chunk kc+2's copies may be pending
      if constexpr (more2()) wait_dma(1);
      else wait_dma(0);
      __syncthreads();
    }
    const int next = (slot + 1) & 3;
    if (head_live) {  // wave-uniform: a head past the end of the target only copies and synchronises
      read_frags(slot, 1, wf[1], xf[1]);
      mfmas(wf[0], xf[0]);
    }
    // the copies of chunk kc+3 are issued under the first k-step's MFMAs, not in front of them: their address
    // arithmetic is a scalar chain every wave of the workgroup would otherwise run at the same time, right after
    // the barrier, with the MFMA pipe idle
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (more3()) {
      dma_from(g_next, step_next, (slot + 3) & 3);
      g_next += 2048;
      if (--left_next == 0) {
        g_next = seg2;
        step_next = seg2_step;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (head_live) {
      if constexpr (more1()) read_frags(next, 0, wf[0], xf[0]);
      mfmas(wf[1], xf[1]);
    }
    slot = next;
  };
  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  int kc = 0;
  for (; kc + 3 < nk; ++kc) chunk(yes, yes, yes);
  if (kc + 2 < nk) { chunk(yes, yes, no); ++kc; }
  if (kc + 1 < nk) { chunk(yes, no, no); ++kc; }
  chunk(no, no, no);
  // let the last MFMA retire before anything the compiler places after the loop reads the accumulators
#pragma unroll
  for (int t2 = 0; t2 < TB; ++t2)
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc[t2][0]), "+v"(acc[t2][1]), "+v"(acc[t2][2]), "+v"(acc[t2][3])::"memory");
  if (!head_live) return;

  const float* bias = tg.bias ? tg.bias + head * 128 : nullptr;
  // the wave's token blocks, two at a time: one 64-token K/V tile per pair
#pragma unroll
  for (int tp = 0; tp < TB / 2; ++tp) {
    const int tok0 = m_tile * kGemmTile + tq * (32 * TB) + tp * 64;
    const int tile = m_tile * 4 + tq * (TB / 2) + tp;
    if (tok0 >= p.M) break;                          // tiles past the last token: nothing to write

    if constexpr (EPI == kEpiVImg) {
      // lane = feature 32*db + r of the head, registers = tokens 8*(i/4) + 4*hh + i%4 of a 32-token block.  The V
      // image (half = token block, db16) wants lane (g, c) = feature 16*db16 + c with tokens 16*(j/4) + 4*g + j%4:
      // this lane's registers 4*(2*(j/4) + a) + j%4 are that piece for g = 2*a + hh, db16 = 2*db + r/16, c = r%16.
      char* rec = tg.out + (int64_t)head * tg.out_head_stride + (int64_t)tile * tg.out_blk_stride;
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int db = 0; db < 4; ++db) {
            const float bv = bias ? bias[32 * db + r] : 0.f;
            bf16x8 img;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const int i = 4 * (2 * (j >> 2) + a) + (j & 3);
              const int token = tok0 + 32 * t2 + 8 * (i >> 2) + 4 * hh + (i & 3);
              img[j] = token < p.M ? (__bf16)(acc[2 * tp + t2][db][i] + bv) : (__bf16)0.0f;
            }
            *(bf16x8*)(rec + ((t2 * 8 + 2 * db + (r >> 4)) * 64 + 16 * (2 * a + hh) + (r & 15)) * 16) = img;
          }
    } else {
      // lane = token, its 64 accumulator values per token block = head-dim elements 16*ks + 8*hh + j in x[ks*8 + j]
      float x[2][64];
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) x[t2][16 * db + i] = acc[2 * tp + t2][db][i] * tg.out_scale;   // x index = ks*8 + j
      if (bias) {
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) {
            const f32x4 b0 = *(const f32x4*)(bias + 16 * ks + 8 * hh), b1 = *(const f32x4*)(bias + 16 * ks + 8 * hh + 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              x[t2][ks * 8 + j] += b0[j];
              x[t2][ks * 8 + 4 + j] += b1[j];
            }
          }
      }
      if constexpr (EPI == kEpiKImg || EPI == kEpiAImg) {
        const RowTransform tf{tg.norm_w, tg.norm_eps, tg.rope_mode, tg.cos_t, tg.sin_t};
        float nmax = 0.f, amax = 0.f;
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          const int token = tok0 + 32 * t2 + r;
          const bool valid = token < p.M;
          if (!valid) {
#pragma unroll
            for (int i = 0; i < 64; ++i) x[t2][i] = 0.f;
          }
          norm_rope_row(x[t2], tf, valid ? token : 0, valid, hh);
          float ssq = 0.f;
#pragma unroll
          for (int i = 0; i < 64; ++i) {
            ssq += x[t2][i] * x[t2][i];
            amax = fmaxf(amax, fabsf(x[t2][i]));
          }
          nmax = fmaxf(nmax, ssq + xhalf(ssq));
        }
        if (tg.norm_max) {
          nmax = sqrtf(wave_max(nmax));
          if (lane == 0) atomicMax(tg.norm_max + head, __float_as_uint(nmax));
        }
        char* rec = tg.out + (int64_t)head * tg.out_head_stride + (int64_t)tile * tg.out_blk_stride;
        if (!tg.fp8) {
#pragma unroll
          for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
              bf16x8 t;
#pragma unroll
              for (int j = 0; j < 8; ++j) t[j] = (__bf16)x[t2][ks * 8 + j];
              // kEpiKImg: the attention kernel's K tile; kEpiAImg: operand images of these GEMMs ([token block][k-step])
              if constexpr (EPI == kEpiKImg) *(bf16x8*)(rec + k_piece_offset(32 * t2 + r, 2 * ks + hh)) = t;
              else *(bf16x8*)(rec + t2 * tg.out_sub_stride + (ks * 64 + lane) * 16) = t;
            }
        } else {
          amax = wave_max(amax);
          const float scale = amax > 0.f ? amax * (1.0f / kFp8Max) : 1.0f;
          const float inv = 1.0f / scale;
          if (lane == 0) tg.scale_out[(int64_t)head * tg.scale_head_stride + tile] = scale;
#pragma unroll
          for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2) {
              const i32x4 q0 = quant_fp8_chunk(x[t2], 2 * c2, inv), q1 = quant_fp8_chunk(x[t2], 2 * c2 + 1, inv);
#pragma unroll
              for (int a = 0; a < 2; ++a) {
                const i32x4 t = {q0[2 * a], q0[2 * a + 1], q1[2 * a], q1[2 * a + 1]};
                *(i32x4*)(rec + k8_chunk_offset(32 * t2 + r, 2 * (4 * c2 + a) + hh)) = t;
              }
            }
        }
      } else {
        // row-major bf16 rows: y = residual + gate[row_index] * (acc*scale + bias); 16-byte pieces per lane
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          const int token = tok0 + 32 * t2 + r;
          if (token >= p.M) continue;
          __bf16* orow = (__bf16*)tg.out + (int64_t)token * tg.out_row_stride + (int64_t)head * tg.out_head_elems;
          const __bf16* res = tg.residual ? (const __bf16*)tg.residual + (int64_t)token * tg.res_row_stride + head * 128 : nullptr;
          const __bf16* gate = tg.gate ? (const __bf16*)tg.gate + (int64_t)(tg.row_index ? tg.row_index[token] : 0) * tg.gate_row_stride + head * 128
                                       : nullptr;
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) {
            const int d0 = 16 * ks + 8 * hh;
            bf16x8 o;
            bf16x8 gv, rv;
            if (gate) gv = *(const bf16x8*)(gate + d0);
            if (res) rv = *(const bf16x8*)(res + d0);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              float v = x[t2][ks * 8 + j];
              if (gate) v *= (float)gv[j];
              if (res) v += (float)rv[j];
              o[j] = (__bf16)v;
            }
            *(bf16x8*)(orow + d0) = o;
          }
        }
      }
    }
  }
}

template <int WAVES>
__global__ __launch_bounds__(64 * WAVES, 1) void gemm_kernel(GemmParams p) {
  __shared__ __attribute__((aligned(1024))) char lds_raw[kGemmRing * kGemmStageBytes];
  // Workgroups go to the 8 XCDs round-robin; each XCD takes one contiguous run of the tile order below, in which 32
  // consecutive tiles (the workgroups the 32 CUs behind one L2 run together) form a block of 4 token tiles x 8
  // feature tiles: every activation panel is then shared by 8 and every weight panel by 4 of them.
  constexpr int kBlockN = 8;
  const int total = p.m_tiles * p.n_tiles;
  const int per_xcd = (total + 7) / 8;
  const int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (lin >= total) return;
  const int full = p.n_tiles / kBlockN * kBlockN;       // feature tiles in whole column blocks
  int m_tile, n_tile;
  if (lin < full * p.m_tiles) {
    const int nb = lin / (kBlockN * p.m_tiles), rem = lin % (kBlockN * p.m_tiles);
    m_tile = rem / kBlockN;
    n_tile = nb * kBlockN + rem % kBlockN;
  } else {
    const int rest = lin - full * p.m_tiles, width = p.n_tiles - full;
    m_tile = rest / width;
    n_tile = full + rest % width;
  }
  int t = 0;
  while (t + 1 < p.n_targets && n_tile >= p.tg[t].n_tiles) { n_tile -= p.tg[t].n_tiles; ++t; }
  const GemmTarget& tg = p.tg[t];
  switch (tg.epi) {
    case kEpiRows: gemm_tile<kEpiRows, WAVES>(p, tg, m_tile, n_tile, lds_raw); break;
    case kEpiKImg: gemm_tile<kEpiKImg, WAVES>(p, tg, m_tile, n_tile, lds_raw); break;
    case kEpiAImg: gemm_tile<kEpiAImg, WAVES>(p, tg, m_tile, n_tile, lds_raw); break;
    default: gemm_tile<kEpiVImg, WAVES>(p, tg, m_tile, n_tile, lds_raw); break;
  }
}

hipError_t launch_gemm(const GemmParams& p, hipStream_t st) {
  const int total = p.m_tiles * p.n_tiles;
  hipLaunchKernelGGL(gemm_kernel<kGemmWaves>, dim3((total + 7) / 8 * 8), dim3(64 * kGemmWaves), 0, st, p);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Rows -> operand images, optionally through the AdaLN modulation of the block:
//   y = norm(x) * (1 + scale[row_index]) + shift[row_index]
// with norm = LayerNorm without affine parameters, RMSNorm without weight, or nothing, statistics in fp32.
// One wave per row: lane l holds the 16-byte pieces l, l + 64, ... of the row.  Image of (32-row block rb,
// k-step ks) at ((rb * K/16 + ks) * 64 + lane') * 16 with lane' = 32 * ((k / 8) & 1) + row % 32.
// `head_perm`: the rows are weight rows (output features) and are stored permuted inside each 128-row head
// (see gemm_tile): image row 32*db + 8*a + 4*hh + b takes source row 32*db + 16*(a>>1) + 8*hh + 4*(a&1) + b.
constexpr int kPackMaxPieces = 8;  // 16-byte pieces per lane: rows of up to 64 * 8 * 8 = 4096 elements

template <int NORM>
__global__ __launch_bounds__(256) void pack_rows_kernel(PackParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = blockIdx.x * 4 + wave;             // destination row
  if (row >= p.rows_padded) return;
  int src = row;
  if (p.head_perm) {
    const int in_head = row & 127, db = in_head >> 5, q = in_head & 31, a = q >> 3, h2 = (q >> 2) & 1, b = q & 3;
    src = (row & ~127) + 32 * db + 16 * (a >> 1) + 8 * h2 + 4 * (a & 1) + b;
  }
  const bool valid = src < p.rows;
  const int pieces = p.K / 8;                        // 16-byte pieces per row
  float v[kPackMaxPieces][8];
  float sum = 0.f, ssq = 0.f;
#pragma unroll
  for (int c = 0; c < kPackMaxPieces; ++c) {
    const int pc = lane + 64 * c;
    bf16x8 t = {};
    if (valid && pc < pieces) t = *(const bf16x8*)((const __bf16*)p.x + (int64_t)src * p.row_stride + 8 * pc);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      v[c][j] = (float)t[j];
      sum += v[c][j];
      ssq += v[c][j] * v[c][j];
    }
  }
  if constexpr (NORM != kNormNone) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      sum += __shfl_xor(sum, o, 64);
      ssq += __shfl_xor(ssq, o, 64);
    }
    const float inv_k = 1.0f / (float)p.K;
    const float mean = NORM == kNormLayer ? sum * inv_k : 0.f;
    const float var = NORM == kNormLayer ? fmaxf(ssq * inv_k - mean * mean, 0.f) : ssq * inv_k;
    const float rs = rsqrtf(var + p.eps);
    const int mrow = valid && p.row_index ? p.row_index[src] : 0;
    const __bf16* sh = p.shift ? (const __bf16*)p.shift + (int64_t)mrow * p.table_stride : nullptr;
    const __bf16* sc = p.scale ? (const __bf16*)p.scale + (int64_t)mrow * p.table_stride : nullptr;
#pragma unroll
    for (int c = 0; c < kPackMaxPieces; ++c) {
      const int pc = lane + 64 * c;
      if (pc >= pieces) continue;
      bf16x8 s8 = {}, h8 = {};
      if (sc) s8 = *(const bf16x8*)(sc + 8 * pc);
      if (sh) h8 = *(const bf16x8*)(sh + 8 * pc);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float y = (v[c][j] - mean) * rs;
        if (sc) y *= 1.0f + (float)s8[j];
        if (sh) y += (float)h8[j];
        v[c][j] = valid ? y : 0.f;
      }
    }
  }
  char* ob = p.out + (int64_t)(row >> 5) * p.out_blk_stride;
#pragma unroll
  for (int c = 0; c < kPackMaxPieces; ++c) {
    const int pc = lane + 64 * c;
    if (pc >= pieces) continue;
    bf16x8 t;
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = (__bf16)v[c][j];
    *(bf16x8*)(ob + ((int64_t)(pc >> 1) * 64 + 32 * (pc & 1) + (row & 31)) * 16) = t;
  }
}

hipError_t launch_pack_rows(const PackParams& p, hipStream_t st) {
  const dim3 grid((p.rows_padded + 3) / 4), block(256);
  switch (p.norm) {
    case kNormLayer: hipLaunchKernelGGL(pack_rows_kernel<kNormLayer>, grid, block, 0, st, p); break;
    case kNormRms: hipLaunchKernelGGL(pack_rows_kernel<kNormRms>, grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL(pack_rows_kernel<kNormNone>, grid, block, 0, st, p); break;
  }
  return hipGetLastError();
}

// clears `n` 32-bit words (used for the per-head K row-norm maxima before the K epilogue max-reduces into them)
__global__ void fill_zero_kernel(unsigned* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

hipError_t launch_fill_zero(unsigned* p, int n, hipStream_t st) {
  hipLaunchKernelGGL(fill_zero_kernel, dim3((n + 255) / 256), dim3(256), 0, st, p, n);
  return hipGetLastError();
}

}  // namespace pkh3
