// Host-side structures shared by the C-ABI translation unit and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "pkh3_common.h"

namespace pkh3 {

// Block-sparse work split: a workgroup covers kSparseRows consecutive 64-query row-blocks (a wave pair each) and its
// plan holds 1 + kSparseRows tile lists (the tiles all its row-blocks keep, then one list per row-block).
constexpr int kSparseRows = 4;
constexpr int kSparseLists = 1 + kSparseRows;

// Long dense calls may end on workgroups that share a unit's key tiles and merge their partial results through global
// scratch: one wave's partial result (O^T 128 x 32, row sums, row maxima, fp32), and the most such workgroups a call
// is planned with (two rounds of workgroups on a 256-CU part; a call that would need more ends on whole workgroups).
constexpr int kPartialBytes = 64 * 64 * 4 + 4 * 64 * 4;
constexpr int kMaxPartWorkgroups = 512;
constexpr int kSections = 3;     // sections of a long dense launch
constexpr int kQueueSlots = 64;  // ints set aside for their positions, in front of the arrival counters
constexpr int kShortMaxTiles = 16;  // dense calls with at most this many key tiles run the short-key kernel

// Where each intermediate lives inside the caller's workspace (byte offsets, 256-aligned).
struct WsPlan {
  int nQ64;      // 64-query blocks, padded to a multiple of 4 (one workgroup = 4 waves x 64 queries)
  int nKt;       // 64-key tiles
  int kvTileBytes;  // bytes of one [K tile | V tile] record
  size_t kv_off, kscale_off, cnt_off, idx_off, plan_off, plan_cnt_off, kmax_off, split_off, split_cnt_off, total;
  size_t split_bytes;  // bytes at split_off: partial results of the long dense form's paired workgroups
};

// One side (Q or K) of the normalise + rotate + lay-out pass.
struct QkPrologueParams {
  const void* x;            // bf16 [B,S,H,D] strided
  int64_t sb, ss, sh;
  int B, H, S;
  int nBlk64;               // 64-row blocks to write (>= ceil(S/64); rows past the end are zero)
  const float* norm_w;      // [D] or null
  float eps;
  int rope_mode;
  const float* cos_t;       // [S, D/2] or null
  const float* sin_t;
  const int* gather_idx;    // [B, S] compacted row -> source row, or null
  const int* row_cnt;       // [B] rows that exist after compaction, or null (= S)
  char* out;                // images
  int64_t out_bh_stride;    // bytes between consecutive (b,h)
  int out_blk_stride;       // bytes between consecutive 64-row blocks
  float* scale_out;         // fp8: [B*H, nBlk64] dequantisation scales, else null
  int fp8;
  int fp8_pow2;             // fp8: block scales rounded up to a power of two
  unsigned* norm_max;       // [B*H] float bits: max row norm after norm+rotation (atomic max), or null
};

struct VPrologueParams {
  const void* v;
  int64_t sb, ss, sh;
  int B, H, S, nKt;
  const int* gather_idx;
  const int* row_cnt;
  char* out;                // points at the V part of tile 0
  int64_t out_bh_stride;
  int out_tile_stride;
  unsigned* zero_init;      // [B*H] words this launch clears (the K launch after it max-reduces into them)
};

struct FwdParams {
  const void* q;            // bf16 [B,Sq,H,D] strided; norm + rotation (+ fp8 quantisation) happen at load
  int64_t q_sb, q_ss, q_sh;
  const float* q_norm_w;    // RMSNorm weight of the Q side or null
  float q_eps;
  int q_rope_mode;
  const float* q_cos;
  const float* q_sin;
  const char* kv;           // [K tile | V tile] records
  int64_t kv_bh_stride;
  int kv_tile_stride;
  const int* row_cnt;       // [B] valid keys after compaction, or null (= Sk)
  void* o;
  int64_t o_sb, o_ss, o_sh;
  int o_images;             // write O as 16-row operand images [row block][H*4 k-steps] instead of [B, Sq, H, D] rows
  int64_t o_img_blk_stride; // bytes between consecutive 16-row blocks of those images
  int B, H, Sq, Sk;
  int nQ64, nKt;
  float c;                  // softmax_scale * log2(e)
  const int* plan;          // block-sparse: per workgroup kSparseLists tile lists nKt ints apart, or null
  const int* plan_cnt;      // [nQ64/kSparseRows][kSparseLists] entries per list
  int plan_stride;          // ints between consecutive workgroups' lists (kSparseLists * nKt)
  const float* kscale;      // [B*H, nKt] fp8 dequantisation scales of the K tiles
  const float* kmax;        // [B*H] largest K' row norm
  int fp8;
  int fp8_pow2;         // fp8: the block scales are powers of two and ride in the scaled MFMA's operands
  int long_key_kernel;  // only the plain long-key form (no short-key form, no shared last round)
  // scratch of the long dense form's shared units (see launch_fp): partial results, and arrival counters (one per
  // wave of a unit of the call's last round)
  float* split_scratch;
  size_t split_scratch_bytes;
  int* split_cnt;           // arrival counters; the kQueueSlots ints in front of them belong to the work queues
  int* queue_next;          // [kQueues] next unit of each work queue (= split_cnt - kQueueSlots), or null: fixed map
  // filled per launch: the sections of the launch.  A unit is one workgroup's block of queries; section i covers
  // sec_units[i] units after those of the sections before it, sec_parts[i] workgroups per unit, in sec_blocks[i]
  // workgroup indices (a multiple of 8)
  int sec_units[kSections], sec_parts[kSections], sec_blocks[kSections];
};

// ---- projection GEMMs (pkh3_gemm.hip) -------------------------------------------------------------------
// what a target's epilogue writes: row-major rows, the attention kernel's K tiles (norm, rotation, fp8), its V tiles,
// or bf16 operand images of these GEMMs themselves (the LoRA down-projection feeding the second K segment)
enum { kEpiRows = 0, kEpiKImg = 1, kEpiVImg = 2, kEpiAImg = 3 };
enum { kNormNone = 0, kNormLayer = 1, kNormRms = 2 };    // row normalisation of the pack / modulation pass

// One output of a GEMM launch: a run of `n` features (whole 128-feature heads) with its own weights and epilogue.
struct GemmTarget {
  int epi;                 // kEpi*
  int n;                   // features of this target (multiple of 128)
  int n_tiles;             // 256-feature workgroup tiles: ceil(n / 256)
  const char* w_img;       // packed weights [feature block][k-step], head-permuted rows unless epi == kEpiVImg
  int64_t w_blk_stride;    // bytes between consecutive 16-feature blocks
  const float* bias;       // [n] fp32 in original feature order, or null
  float out_scale;         // accumulator * out_scale (+ bias)
  // second K segment (LoRA): activations from the down-projected rows of this target, weights from B
  const char* a2_img;
  int64_t a2_blk_stride;
  const char* w2_img;
  int64_t w2_blk_stride;
  int nk2;                 // 32-wide k-chunks of the second segment (0 = none)
  // output
  char* out;
  int64_t out_head_stride; // image epilogues: bytes between heads
  int64_t out_blk_stride;  // kEpiKImg / kEpiVImg: bytes between 64-token tiles; kEpiAImg: between 16-token blocks
  int64_t out_row_stride;  // kEpiRows: elements between token rows
  int out_head_elems;      // kEpiRows: elements between heads
  // kEpiKImg
  const float* norm_w;
  float norm_eps;
  int rope_mode;
  const float* cos_t;
  const float* sin_t;
  unsigned* norm_max;      // [heads] float bits, atomic max of the row norms, or null
  int fp8;
  int fp8_pow2;            // fp8: block scales rounded up to a power of two
  float* scale_out;        // fp8: [heads][scale_head_stride] dequantisation scales
  int scale_head_stride;
  // kEpiRows: y = residual + gate[row_index[token]] * (acc * out_scale + bias)
  const void* gate;        // bf16 [rows, gate_row_stride] or null
  int64_t gate_row_stride;
  const int* row_index;    // [M] or null (row 0)
  const void* residual;    // bf16 [M, res_row_stride] or null
  int64_t res_row_stride;
};

struct GemmParams {
  const char* a_img;       // activations [token block][k-step]
  int64_t a_blk_stride;    // bytes between consecutive 16-token blocks
  int nk1;                 // 32-wide k-chunks of the first segment
  int M;                   // tokens
  int m_tiles, n_tiles;    // 256 x 256 workgroup tiles
  int n_targets;
  GemmTarget tg[3];
  int* queue_next;         // [kQueues] zeroed positions of the per-XCD work queues the tiles are taken from, or null: fixed map
};

// rows (activations or weights) -> operand images, optionally normalised and modulated
struct PackParams {
  const void* x;           // bf16 [rows, row_stride]
  int64_t row_stride;      // elements
  int rows, rows_padded;   // rows that exist / image rows to write (multiple of 16; the rest is zero)
  int K;                   // elements per row (multiple of 16, <= 4096)
  int head_perm;
  int norm;                // kNorm*
  float eps;
  const void* shift;       // bf16 [table rows, table_stride] or null
  const void* scale;
  int64_t table_stride;
  const int* row_index;    // [rows] table row of each row, or null (row 0)
  char* out;
  int64_t out_blk_stride;  // bytes between consecutive 16-row blocks
};

hipError_t launch_gemm(const GemmParams& p, hipStream_t st);
hipError_t launch_pack_rows(const PackParams& p, hipStream_t st);
hipError_t launch_fill_zero(unsigned* p, int n, hipStream_t st);

hipError_t launch_mask_compact(const uint8_t* mask, int B, int Sk, int* idx, int* cnt, hipStream_t st);
hipError_t launch_qk_prologue(const QkPrologueParams& p, hipStream_t st);
hipError_t launch_v_prologue(const VPrologueParams& p, hipStream_t st);
hipError_t launch_attn_fwd(const FwdParams& p, hipStream_t st);
hipError_t device_cu_count(int* out);  // CUs of the current device (cached per device after the first call)
hipError_t launch_sparse_plan(const int* row_ptr, const int* col_idx, int nRow64, int nQ64, int nKt, int* plan,
                              int plan_stride, int* plan_cnt, hipStream_t st);
hipError_t launch_rope_tables(const double* pos, int S, const int* axis_dims, double theta, float* cos_out,
                              float* sin_out, hipStream_t st);

}  // namespace pkh3
