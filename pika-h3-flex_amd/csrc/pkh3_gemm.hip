// Projection GEMMs around the attention kernel (gfx950, bf16 MFMA 16x16x32, fp32 accumulation):
//   to_q / to_k / to_v  (+ LoRA)  from the modulated hidden states, with the K side's RMSNorm + rotation
//                       (+ fp8 quantisation) and the K / V operand-image layout done in the epilogue, so that
//                       K and V go from the accumulators straight into the records the attention kernel reads
//   to_out.0 (+ LoRA)   from the attention output, with bias, per-row gate and residual in the epilogue
//   LoRA down-projection x A^T, written as operand images for the second K segment of the GEMMs above
//
// Operands.  Both operands come as 1 KiB operand images (16 rows x 32 contraction elements, lane l holds row
// l%16, elements 8*(l/16)..+7 -- the shape of the attention kernel's K images): activations as [16-token
// block][k-step], weights as [16-feature block][k-step] (packed once when the weights are loaded).  They move
// HBM/L2 -> LDS -> VGPR as straight 16-byte copies, like the K/V tiles of the attention kernel: direct-to-LDS loads
// into a 4-slot ring, three chunks ahead, one barrier per chunk.  Since the two MFMA operands have the same register
// form, one pair of images serves both orientations:
//   C^T = W x^T  (features down the accumulator registers, one token per lane)   Q, K, row-major outputs
//   C   = x W^T  (tokens down the registers, one feature per lane)               V images
// Weight rows are stored permuted inside each 128-feature head so that, in the C^T form, the 32 accumulator
// values a lane holds for a token are the four 8-element pieces p8 = 4*ks + g (elements 32*ks + 8*g .. +7) of that
// token's head row: exactly what lane (g, c) of the attention kernel's K images carries, so the K epilogue stores
// its accumulators (after norm and rotation) without any lane movement, and so do the row-major and the V epilogues.
//
// Work split.  Workgroup = 8 waves = 256 tokens x 256 features; wave (fh, tq) owns features fh*128..+127 (one
// head) x tokens tq*64..+63 (one K/V tile): 32 accumulators of 16x16.  Per 32-wide k-chunk a wave reads 8 weight
// and 4 activation images for 32 MFMAs.  LoRA is a second K segment: k-chunks beyond the hidden size take their
// activation images from the down-projected rows (x A^T, scaled) and their weight images from B.
#include <type_traits>

#include "pkh3_common.h"
#include "pkh3_internal.h"

namespace pkh3 {

constexpr int kGemmWaves = 8;
constexpr int kGemmTile = 256;                      // tokens and features per workgroup
constexpr int kGemmChunkK = 32;                     // contraction elements per ring slot = one k-step
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

template <int EPI>
__device__ __forceinline__ void gemm_tile(const GemmParams& p, const GemmTarget& tg, int m_tile, int n_tile_in_target,
                                          char* lds_raw) {
  constexpr int WAVES = kGemmWaves;
  constexpr int PP = 32 / WAVES;                     // 1 KiB pieces of a chunk each wave copies
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, c = lane & 15;
  const int fh = wave & 1, tq = wave >> 1;           // feature half (one head), 64-token slice
  const int head = n_tile_in_target * 2 + fh;        // 128-feature head inside the target
  const bool head_live = head * 128 < tg.n;
  const int nk1 = p.nk1, nk = p.nk1 + tg.nk2;
  const unsigned lane_off = lane * 16;

  // this wave's 1 KiB pieces of every chunk: pieces PP*wave.. of [16 weight blocks | 16 token blocks]
  const int piece0 = wave * PP;
  const bool w_side = piece0 < 16;
  const int blk0 = piece0 & 15;                      // first of the 16-row blocks this wave copies
  const char* seg1 = w_side ? tg.w_img + (int64_t)(n_tile_in_target * 16 + blk0) * tg.w_blk_stride
                            : p.a_img + (int64_t)(m_tile * 16 + blk0) * p.a_blk_stride;
  const int64_t seg1_step = w_side ? tg.w_blk_stride : p.a_blk_stride;
  const char* seg2 = w_side ? tg.w2_img + (int64_t)(n_tile_in_target * 16 + blk0) * tg.w2_blk_stride
                            : tg.a2_img + (int64_t)(m_tile * 16 + blk0) * tg.a2_blk_stride;
  const int64_t seg2_step = w_side ? tg.w2_blk_stride : tg.a2_blk_stride;
  // this wave's copies of one chunk: the chunk's image of PP consecutive blocks, `step` bytes apart, into ring slot `slot`
  auto dma_from = [&](const char* gp, int64_t step, int slot) {
    char* d = lds_raw + slot * kGemmStageBytes + piece0 * 1024;
#pragma unroll
    for (int b = 0; b < PP; ++b) gemm_dma16(gp + b * step, lane_off, d + b * 1024);
  };
  auto dma = [&](int kc, int slot) {
    const bool first = kc < nk1;
    dma_from(first ? seg1 + (int64_t)kc * 1024 : seg2 + (int64_t)(kc - nk1) * 1024, first ? seg1_step : seg2_step, slot);
  };
  // waits until at most `chunks` of this wave's newest chunk copies are still in flight
  auto wait_dma = [&](int chunks) {
    if (chunks >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PP) : "memory");
    else if (chunks == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PP) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };

  f32x4 acc[4][8];                                   // (16-token block of the wave's 64, 16-feature block of the head)
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int fb = 0; fb < 8; ++fb) acc[t][fb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Ring of four chunks.  Entering iteration kc: chunk kc is in LDS for every wave and its token images and first four
  // weight images are already on their way to this wave's registers; chunks kc+1 and kc+2 are in flight.  The barrier at
  // the top makes chunk kc+1 visible and frees the slot of chunk kc-1 for chunk kc+3, so the first images of the next
  // chunk can be read at the tail of this iteration and no wave starts a chunk by waiting for LDS.
  const int n_pre = nk < 3 ? nk : 3;
  for (int cc = 0; cc < n_pre; ++cc) dma(cc, cc);
  wait_dma(n_pre - 1);
  __syncthreads();
  const int w_off = (fh * 8) * 1024 + lane * 16;            // weight blocks fh*8..+7 of a slot
  const int a_off = 16384 + (tq * 4) * 1024 + lane * 16;    // this wave's token blocks
  bf16x8 wa[4], wb[4], xc[4], xn[4];                        // weight blocks 0..3 / 4..7, token images of this / the next chunk
  auto read_w = [&](int slot, int half, bf16x8 (&w4)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) w4[i] = *(const bf16x8*)(lds_raw + slot * kGemmStageBytes + w_off + (half * 4 + i) * 1024);
  };
  auto read_x = [&](int slot, bf16x8 (&x4)[4]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) x4[t] = *(const bf16x8*)(lds_raw + slot * kGemmStageBytes + a_off + t * 1024);
  };
  auto mfmas = [&](int half, const bf16x8 (&w4)[4], const bf16x8 (&x4)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        if constexpr (EPI == kEpiVImg) acc[t][half * 4 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x4[t], w4[i], acc[t][half * 4 + i], 0, 0, 0);
        else acc[t][half * 4 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w4[i], x4[t], acc[t][half * 4 + i], 0, 0, 0);
      }
  };
  if (head_live) {
    read_x(0, xc);
    read_w(0, 0, wa);
  }
  int slot = 0;
  // source of the next chunk to copy (chunk kc + 3 in the steady loop): a running pointer inside its K segment
  const char* g_next = nullptr;
  int64_t step_next = seg1_step;
  int left_next = 0;  // chunks left in the segment g_next walks, this one included
  if (nk > 3) {
    const bool first = 3 < nk1;
    g_next = first ? seg1 + 3 * 1024 : seg2 + (int64_t)(3 - nk1) * 1024;
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
      read_w(slot, 1, wb);
      mfmas(0, wa, xc);
    }
    // the copies of chunk kc+3 are issued under the first half's MFMAs, not in front of them: their address
    // arithmetic is a scalar chain every wave of the workgroup would otherwise run at the same time, right after
    // the barrier, with the MFMA pipe idle
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (more3()) {
      dma_from(g_next, step_next, (slot + 3) & 3);
      g_next += 1024;
      if (--left_next == 0) {
        g_next = seg2;
        step_next = seg2_step;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (head_live) {
      if constexpr (more1()) {
        read_x(next, xn);
        read_w(next, 0, wa);
      }
      mfmas(1, wb, xc);
      if constexpr (more1()) {
#pragma unroll
        for (int t = 0; t < 4; ++t) xc[t] = xn[t];
      }
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
  for (int t = 0; t < 4; ++t)
    asm volatile("s_nop 15\n\ts_nop 15"
                 : "+v"(acc[t][0]), "+v"(acc[t][1]), "+v"(acc[t][2]), "+v"(acc[t][3]), "+v"(acc[t][4]), "+v"(acc[t][5]),
                   "+v"(acc[t][6]), "+v"(acc[t][7])::"memory");
  if (!head_live) return;

  const float* bias = tg.bias ? tg.bias + head * 128 : nullptr;
  const int tok0 = m_tile * kGemmTile + tq * 64;     // the wave's 64 tokens: one K/V tile
  const int tile = m_tile * 4 + tq;
  if (tok0 >= p.M) return;                           // a tile past the last token: nothing to write

  if constexpr (EPI == kEpiVImg) {
    // lane (g, c) = feature 16*fb + c of the head, registers = tokens 4*g + i of a 16-token block: the V image
    // (half, db = fb) wants, in that same lane, the tokens 16*(j/4) + 4*g + j%4 of its 32: blocks 2*half and 2*half + 1
    char* rec = tg.out + (int64_t)head * tg.out_head_stride + (int64_t)tile * tg.out_blk_stride;
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int fb = 0; fb < 8; ++fb) {
        const float bv = bias ? bias[16 * fb + c] : 0.f;
        bf16x8 img;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int token = tok0 + 32 * half + v_image_key(g, j);
          img[j] = token < p.M ? (__bf16)(acc[2 * half + (j >> 2)][fb][j & 3] + bv) : (__bf16)0.0f;
        }
        *(bf16x8*)(rec + ((half * 8 + fb) * 64 + lane) * 16) = img;
      }
  } else {
    // lane (g, c) = token 16*t + c; its accumulators (t, fb) are elements 32*ks + 8*g + j of the head row with
    // fb = 2*ks + j/4, i = j%4 (the weight-row permutation, see pack_rows_kernel): x[8*ks + j]
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int token = tok0 + 16 * t + c;
      const bool valid = token < p.M;
      float x[32];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j) x[ks * 8 + j] = valid ? acc[t][2 * ks + (j >> 2)][j & 3] * tg.out_scale : 0.f;
      if (bias) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const f32x4 b0 = *(const f32x4*)(bias + 32 * ks + 8 * g), b1 = *(const f32x4*)(bias + 32 * ks + 8 * g + 4);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            x[ks * 8 + j] += valid ? b0[j] : 0.f;
            x[ks * 8 + 4 + j] += valid ? b1[j] : 0.f;
          }
        }
      }
      if constexpr (EPI == kEpiKImg) {
        const RowTransform tf{tg.norm_w, tg.norm_eps, tg.rope_mode, tg.cos_t, tg.sin_t};
        norm_rope_quarter(x, tf, valid ? token : 0, valid, g);
        // kept for the tile-wide reductions below
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[t][2 * ks + (j >> 2)][j & 3] = x[ks * 8 + j];
      } else if constexpr (EPI == kEpiAImg) {
        // operand images of these GEMMs: [16-token block][k-step], this lane's piece ks at its own place in image ks
        char* rec = tg.out + (int64_t)head * tg.out_head_stride + (int64_t)(m_tile * 16 + tq * 4 + t) * tg.out_blk_stride;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          bf16x8 v;
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = (__bf16)x[ks * 8 + j];
          *(bf16x8*)(rec + (ks * 64 + lane) * 16) = v;
        }
      } else {
        // row-major bf16 rows: y = residual + gate[row_index] * (acc*scale + bias); 16-byte pieces per lane
        if (!valid) continue;
        __bf16* orow = (__bf16*)tg.out + (int64_t)token * tg.out_row_stride + (int64_t)head * tg.out_head_elems;
        const __bf16* res = tg.residual ? (const __bf16*)tg.residual + (int64_t)token * tg.res_row_stride + head * 128 : nullptr;
        const __bf16* gate = tg.gate ? (const __bf16*)tg.gate + (int64_t)(tg.row_index ? tg.row_index[token] : 0) * tg.gate_row_stride + head * 128
                                     : nullptr;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const int d0 = 32 * ks + 8 * g;
          bf16x8 o, gv, rv;
          if (gate) gv = *(const bf16x8*)(gate + d0);
          if (res) rv = *(const bf16x8*)(res + d0);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            float v = x[ks * 8 + j];
            if (gate) v *= (float)gv[j];
            if (res) v += (float)rv[j];
            o[j] = (__bf16)v;
          }
          *(bf16x8*)(orow + d0) = o;
        }
      }
    }
    if constexpr (EPI == kEpiKImg) {
      // the wave's 64 tokens are one K tile: largest row norm, fp8 scale, then every piece at its place in the tile
      float nmax = 0.f, amax = 0.f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        float ssq = 0.f;
#pragma unroll
        for (int fb = 0; fb < 8; ++fb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ssq += acc[t][fb][i] * acc[t][fb][i];
            amax = fmaxf(amax, fabsf(acc[t][fb][i]));
          }
        nmax = fmaxf(nmax, wave_sum_groups(ssq));
      }
      if (tg.norm_max) {
        nmax = sqrtf(wave_max(nmax));
        if (lane == 0) raise_max(tg.norm_max + head, nmax);
      }
      char* rec = tg.out + (int64_t)head * tg.out_head_stride + (int64_t)tile * tg.out_blk_stride;
      if (!tg.fp8) {
        // K tile image (half, ks, kb2) of 16-token block t = 2*half + kb2: this lane's piece ks at its own place
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) {
            bf16x8 v;
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = (__bf16)acc[t][2 * ks + (j >> 2)][j & 3];
            *(bf16x8*)(rec + ((((t >> 1) * 4 + ks) * 2 + (t & 1)) * 64 + lane) * 16) = v;
          }
      } else {
        amax = wave_max(amax);
        const float scale = fp8_block_scale(amax, tg.fp8_pow2 != 0);
        const float inv = 1.0f / scale;
        if (lane == 0) tg.scale_out[(int64_t)head * tg.scale_head_stride + tile] = scale;
        // fp8 K tile: key block t is 2 KiB, chunk c2 of a lane holds its pieces ks = 2*c2 and 2*c2 + 1
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int c2 = 0; c2 < 2; ++c2) {
            float lo[8], hi[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              lo[j] = acc[t][4 * c2 + (j >> 2)][j & 3];
              hi[j] = acc[t][4 * c2 + 2 + (j >> 2)][j & 3];
            }
            const i32x2 q0 = quant_fp8_piece(lo, inv), q1 = quant_fp8_piece(hi, inv);
            *(i32x4*)(rec + ((t * 2 + c2) * 64 + lane) * 16) = i32x4{q0[0], q0[1], q1[0], q1[1]};
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
  int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (p.queue_next) {
    // tiles from per-XCD work queues (see fetch_unit): the launch holds spare workgroups, and an XCD that is through
    // with its run early takes tiles off the slower ones
    __shared__ int fetched_tile;
    if (threadIdx.x == 0) fetched_tile = fetch_unit(p.queue_next, blockIdx.x & (kQueues - 1), total);
    __syncthreads();
    lin = __builtin_amdgcn_readfirstlane(fetched_tile);
    if (lin < 0) return;
  }
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
    case kEpiRows: gemm_tile<kEpiRows>(p, tg, m_tile, n_tile, lds_raw); break;
    case kEpiKImg: gemm_tile<kEpiKImg>(p, tg, m_tile, n_tile, lds_raw); break;
    case kEpiAImg: gemm_tile<kEpiAImg>(p, tg, m_tile, n_tile, lds_raw); break;
    default: gemm_tile<kEpiVImg>(p, tg, m_tile, n_tile, lds_raw); break;
  }
}

hipError_t launch_gemm(const GemmParams& p, hipStream_t st) {
  const int total = p.m_tiles * p.n_tiles;
  // with work queues: an eighth more workgroups than tiles, the spare ones for the XCDs that finish early
  const int wgs = p.queue_next ? total + (total / 8 > kQueues ? total / 8 : kQueues) : total;
  hipLaunchKernelGGL(gemm_kernel<kGemmWaves>, dim3((wgs + 7) / 8 * 8), dim3(64 * kGemmWaves), 0, st, p);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Rows -> operand images, optionally through the AdaLN modulation of the block:
//   y = norm(x) * (1 + scale[row_index]) + shift[row_index]
// with norm = LayerNorm without affine parameters, RMSNorm without weight, or nothing, statistics in fp32.
// One wave per row: lane l holds the 16-byte pieces l, l + 64, ... of the row.  Piece pc (elements 8*pc .. +7) of row r
// belongs to image (16-row block r/16, k-step pc/4), lane 16*(pc%4) + r%16: byte ((r/16)*(K/32) + pc/4)*1024 +
// (16*(pc%4) + r%16)*16.
// `head_perm`: the rows are weight rows (output features) and are stored permuted inside each 128-row head
// (see gemm_tile): image row 16*fb + 4*g + i takes source row 32*(fb/2) + 8*g + 4*(fb%2) + i.
constexpr int kPackMaxPieces = 8;  // 16-byte pieces per lane: rows of up to 64 * 8 * 8 = 4096 elements

constexpr int kPackRows = 8;                                        // rows (waves) of a workgroup
constexpr int kPackPitch = kPackMaxPieces * 64 * 16 + 16;           // bytes between the rows staged in LDS (+16: no bank conflicts)

template <int NORM>
__global__ __launch_bounds__(64 * kPackRows) void pack_rows_kernel(PackParams p) {
  // the rows of the workgroup, as bf16 pieces, before they go out: in an image a row's pieces lie 256 bytes apart and
  // the same piece of 16 consecutive rows side by side, so whole cache lines only come from several rows together
  __shared__ __attribute__((aligned(16))) char stage[kPackRows * kPackPitch];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = blockIdx.x * kPackRows + wave;     // destination row (rows_padded is a multiple of 16: always inside)
  int src = row;
  if (p.head_perm) {
    const int in_head = row & 127, fb = in_head >> 4, g = (in_head >> 2) & 3, i = in_head & 3;
    src = (row & ~127) + 32 * (fb >> 1) + 8 * g + 4 * (fb & 1) + i;
  }
  const bool valid = src < p.rows;
  const int pieces = p.K / 8;                        // 16-byte pieces per row
  float v[kPackMaxPieces][8];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < kPackMaxPieces; ++c) {
    const int pc = lane + 64 * c;
    bf16x8 t = {};
    if (valid && pc < pieces) t = *(const bf16x8*)((const __bf16*)p.x + (int64_t)src * p.row_stride + 8 * pc);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      v[c][j] = (float)t[j];
      sum += v[c][j];
    }
  }
  if constexpr (NORM != kNormNone) {
    // Two passes over the row held in registers: the mean first, then the sum of squared distances from it.  The
    // one-pass form E[x^2] - mean^2 cancels when a row's mean is large against its spread.
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o, 64);
    const float inv_k = 1.0f / (float)p.K;
    const float mean = NORM == kNormLayer ? sum * inv_k : 0.f;
    float ssq = 0.f;
#pragma unroll
    for (int c = 0; c < kPackMaxPieces; ++c) {
      if (lane + 64 * c >= pieces) continue;  // pieces past the row's end hold zeros, not elements
#pragma unroll
      for (int j = 0; j < 8; ++j) ssq += (v[c][j] - mean) * (v[c][j] - mean);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) ssq += __shfl_xor(ssq, o, 64);
    // a constant row with eps == 0 comes out as zeros (plus shift) instead of 0 * inf
    const float ve = ssq * inv_k + p.eps;
    const float rs = ve > 0.f ? rsqrtf(ve) : 0.f;
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
#pragma unroll
  for (int c = 0; c < kPackMaxPieces; ++c) {
    const int pc = lane + 64 * c;
    if (pc >= pieces) continue;
    bf16x8 t;
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = (__bf16)v[c][j];
    *(bf16x8*)(stage + wave * kPackPitch + pc * 16) = t;
  }
  __syncthreads();
  // the workgroup's 8 rows are one half of a 16-row block: piece pc of the 8 rows is 128 contiguous bytes of its image
  const int row0 = blockIdx.x * kPackRows;
  char* ob = p.out + (int64_t)(row0 >> 4) * p.out_blk_stride + (row0 & 15) * 16;
  for (int q = threadIdx.x; q < kPackRows * pieces; q += 64 * kPackRows) {
    const int rr = q & (kPackRows - 1), pc = q / kPackRows;
    const bf16x8 t = *(const bf16x8*)(stage + rr * kPackPitch + pc * 16);
    *(bf16x8*)(ob + ((int64_t)(pc >> 2) * 64 + 16 * (pc & 3) + rr) * 16) = t;
  }
}

hipError_t launch_pack_rows(const PackParams& p, hipStream_t st) {
  const dim3 grid(p.rows_padded / kPackRows), block(64 * kPackRows);
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
