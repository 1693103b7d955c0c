/*
 * pkh3_attn.h -- C ABI of libpkh3attn.so, the gfx950 (MI355X) attention engine for the
 * Pika H3 Flex video+audio DiT.
 *
 * What each entry point replaces in the reference (paths relative to the reference checkout):
 *
 *   The reference holds no attention code and no FFI of its own.  Its transformer is the
 *   un-vendored `diffusers.MiniMaxH3Transformer3DModel` (src/pika_h3/core/loader.py:11-18) which
 *   H3DiffusionWrapper calls once per denoising step (src/pika_h3/core/wrapper.py:248) with the
 *   packed-sequence keyword tensors assembled at src/pika_h3/core/wrapper.py:192-204.  Inside each
 *   block, the attention module owns the sub-layers `to_q/to_k/to_v/to_out.0`
 *   (src/pika_h3/core/loader.py:9).  These entry points are what an attention processor attached to
 *   that module binds instead of torch's scaled_dot_product_attention:
 *
 *     pkh3_attn_fwd            the per-block attention between `to_v` and `to_out.0`:
 *                              QK-RMSNorm -> 3-axis RoPE from position_ids
 *                              (src/pika_h3/core/packing.py:126-135) -> softmax(QK^T * scale) V
 *     pkh3_kv_prepare          the K/V side of that call alone, for keys and values several calls share
 *     pkh3_workspace_bytes     sizing of the scratch the call needs (caller-owned, e.g. torch.empty)
 *     pkh3_rope_tables         cos/sin tables from the [S,3] float64 position grid the layout
 *                              builder returns (src/pika_h3/core/packing.py:199, :128)
 *     pkh3_last_error / pkh3_version / pkh3_strerror   diagnostics
 *
 * Conventions
 *   - plain pointers and sizes only; every buffer is owned by the caller and lives in device
 *     memory (HBM) unless stated; the library allocates nothing.
 *   - all work is enqueued on `stream` (a hipStream_t passed as void*); no call declared in this header
 *     synchronises (the benchmark hook in pkh3_attn_bench.h does, and is kept apart for that reason).
 *   - strides are in ELEMENTS; the innermost (head-dim) stride is 1 and D must be 128.
 *   - return value 0 = success, negative = PKH3_E* below.  Arguments are validated on the host
 *     before any HIP call, so argument errors are reported without a GPU.
 */
#ifndef PKH3_ATTN_H
#define PKH3_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PKH3_VERSION 107

enum {
  PKH3_OK = 0,
  PKH3_ENULL = -1,        /* a required pointer is NULL */
  PKH3_ESHAPE = -2,       /* B/H/Sq/Sk out of range */
  PKH3_EHEADDIM = -3,     /* D != 128 */
  PKH3_ESTRIDE = -4,      /* stride not a multiple of 8 elements (16-byte rows) or negative */
  PKH3_EALIGN = -5,       /* base pointer not 16-byte aligned */
  PKH3_EWORKSPACE = -6,   /* workspace missing, misaligned (256 B) or too small */
  PKH3_EUNSUPPORTED = -7, /* combination of options that is not implemented */
  PKH3_EHIP = -8,         /* a HIP runtime call failed; see pkh3_last_error() */
  PKH3_EARG = -9          /* other invalid argument (flags, scale, eps) */
};

/* rope_mode */
enum {
  PKH3_ROPE_NONE = 0,
  PKH3_ROPE_INTERLEAVED = 1, /* pairs (x[2i], x[2i+1]) rotate by angle i */
  PKH3_ROPE_HALF = 2         /* pairs (x[i], x[i+D/2]) rotate by angle i  (rotate_half) */
};

/* flags */
enum {
  PKH3_FLAG_FP8_QK = 1u << 0, /* quantise normed+roped Q and K to fp8 e4m3 (OCP) with one absmax scale
                                 per (batch, head, 64-row block); P.V stays bf16 with fp32 accumulation */
  PKH3_FLAG_KV_PREPARED = 1u << 2, /* K and V already lie in `workspace` as the attention kernel reads them, written
                                 there by pkh3_qkv_proj or pkh3_kv_prepare with the same B, H, Sk and K-side options:
                                 the call skips its own K/V pass (key-mask compaction included; `key_mask` must still
                                 be non-NULL when the keys were prepared with one); `k` and `v` are not read and may
                                 be NULL */
  PKH3_FLAG_O_IMAGES = 1u << 3, /* `o` is not a [B, Sq, H, D] tensor but the operand-image buffer pkh3_out_proj reads
                                 (what pkh3_pack_rows would make of the [Sq, H*D] output: pkh3_packed_bytes(Sq, H*D)
                                 bytes, 16-byte aligned): the kernel's epilogue writes the images itself and the
                                 separate packing pass disappears.  B must be 1; o_sb, o_ss, o_sh are not read.  Rows
                                 of the buffer past ceil(Sq/32)*32 are left as they are (pkh3_out_proj never uses
                                 what it computes from them) */
  PKH3_FLAG_FP8_POW2_SCALES = 1u << 4, /* with PKH3_FLAG_FP8_QK: another quantisation rule, for speed.  Every block
                                 scale is the smallest power of two that is at least absmax / 448 (both formed in
                                 float32), and Q is multiplied by softmax_scale * log2(e) before it is quantised instead
                                 of its logits afterwards.  The matrix instruction then applies the scales itself and
                                 the softmax needs no multiply per logit.  A K-side option too: pkh3_kv_prepare,
                                 pkh3_qkv_proj and the calls on their keys must agree on it.  At most one binade of
                                 the e4m3 range is given up; the error stays that of an e4m3 rounding (relative step
                                 2^-4) */
  PKH3_FLAG_LONG_KEY_KERNEL = 1u << 1 /* dense calls with at most 16 key tiles (Sk <= 1024) normally run a
                                 short-key form of the kernel (small workgroups, three per CU), and long dense
                                 calls share the query tiles of a thinly filled last round of workgroups out
                                 among several workgroups each; this flag selects the plain long-key form,
                                 one workgroup per query tile, for all of them.  Same results to the tolerance
                                 of the path; meant for tests and measurements */
};

typedef struct pkh3_attn_args {
  /* bf16 tensors, logical shape [B, S, H, D], addressed as base + b*sb + s*ss + h*sh + d */
  const void* q;
  const void* k;
  const void* v;
  void* o;
  int64_t q_sb, q_ss, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  int32_t B, H, Sq, Sk, D;
  float softmax_scale; /* <= 0 selects 1/sqrt(D) */
  /* QK-RMSNorm over the head dim: x * rsqrt(mean(x^2) + eps) * w.  fp32 [D]; NULL = no norm on that side */
  const float* q_norm_w;
  const float* k_norm_w;
  float norm_eps;
  /* rotary tables, fp32 [Sq, D/2] and [Sk, D/2] (row = token, column = pair index) */
  int32_t rope_mode;
  const float* q_rope_cos;
  const float* q_rope_sin;
  const float* k_rope_cos;
  const float* k_rope_sin;
  /* key padding mask, uint8 [B, Sk], non-zero = attend; NULL = all keys valid.  A query row whose
     every key is masked gets an all-zero output row. */
  const uint8_t* key_mask;
  /* block-sparse map over 64x64 (query x key) tiles in CSR form, shared by all batches and heads:
     blk_row_ptr int32 [ceil(Sq/64)+1], blk_col_idx int32 [blk_row_ptr[last]].  NULL = dense.  Rows
     with no tile get an all-zero output.
     Preconditions, NOT checked (the arrays live in device memory and are read by a kernel only):
     blk_row_ptr[0] = 0, blk_row_ptr non-decreasing, every value at most the number of int32 entries
     allocated behind blk_col_idx; columns in [0, ceil(Sk/64)), each at most once per row (any order;
     the library sorts).  What a violation does: a column outside the range is ignored, a repeated
     column counts once, a row whose end lies before its start is treated as empty; blk_row_ptr values
     beyond the blk_col_idx allocation make the planning kernel read out of bounds. */
  const int32_t* blk_row_ptr;
  const int32_t* blk_col_idx;
  uint32_t flags;
  /* scratch, 256-byte aligned, at least pkh3_workspace_bytes() long.  It must stay alive until the stream has
     run the call.  Every call writes in it (behind the keys, also with PKH3_FLAG_KV_PREPARED: block-sparse plans,
     work-queue positions, arrival counters and partial results of workgroups that share a query tile), so
     calls that may overlap on one GPU -- different streams -- need a workspace each; calls on one stream are
     ordered and may share one */
  void* workspace;
  size_t workspace_bytes;
} pkh3_attn_args;

/* Bytes of scratch pkh3_attn_fwd needs for these shapes/options (0 on invalid arguments).
   Replaces nothing in the reference: torch SDPA sizes its own scratch. */
size_t pkh3_workspace_bytes(const pkh3_attn_args* a);

/* One attention call: the arithmetic of the DiT block's attention between the q/k/v projections and
   the output projection (module at src/pika_h3/core/loader.py:9; call site src/pika_h3/core/wrapper.py:248). */
int pkh3_attn_fwd(const pkh3_attn_args* a, void* stream);

/* The K/V side of pkh3_attn_fwd on its own: key-mask compaction, K through QK-RMSNorm, rotation and (with
   PKH3_FLAG_FP8_QK) quantisation, K and V into `a->workspace` in the layout the attention kernel reads.  The
   attention calls that follow pass the same B, H, Sk, K-side options (k_norm_w, norm_eps, rope_mode, k tables,
   key_mask, PKH3_FLAG_FP8_QK) and workspace with PKH3_FLAG_KV_PREPARED added, and any q, o, Sq and block map:
   keys and values that several calls share are prepared once -- the text keys of a block's cross-attention do not
   change over the denoising steps of a clip (src/pika_h3/pipeline.py:13 runs the model six times on one prompt).
   `q` and `o` of `a` are not looked at.  The K/V side occupies the head of the workspace and its size does not
   depend on Sq or the block map; the later calls still need pkh3_workspace_bytes() of their own arguments. */
int pkh3_kv_prepare(const pkh3_attn_args* a, void* stream);

/* The same call for callers that cannot allocate device memory or pass a workspace (code under HIP graph
   capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
   `workspace` / `workspace_bytes` of `a` are ignored: the scratch is an array built into the library, one
   copy per GPU, PKH3_NOALLOC_SCRATCH_BYTES long, held until the process ends.  The call allocates and frees
   nothing.  Calls whose pkh3_workspace_bytes() exceeds that size are rejected with PKH3_EWORKSPACE.  Every
   call on one GPU shares that GPU's array (each call rewrites all of it that it reads, so nothing needs
   clearing between calls), hence two such calls that may overlap on one GPU -- different streams, or one
   graph launched twice at once -- race; calls on one stream are ordered and safe.  Same kernels, same
   results as pkh3_attn_fwd. */
#define PKH3_NOALLOC_SCRATCH_BYTES (64u << 20)
int pkh3_attn_fwd_noalloc(const pkh3_attn_args* a, void* stream);

/* Set-up of pkh3_attn_fwd_noalloc for the CURRENT device: looks up the address of that device's copy of the
   built-in array and the device's CU count and keeps both.  The first pkh3_attn_fwd_noalloc call on a device does
   the same by itself, but these look-ups are not stream operations and a stream capture in progress may refuse
   them: a caller that captures pkh3_attn_fwd_noalloc into a HIP graph calls this once per device beforehand (or
   makes one ordinary call first).  Allocates nothing, launches nothing.  Like the call it serves it has no
   counterpart in the reference. */
int pkh3_noalloc_init(void);

/* Rotary tables from the packed layout's position grid (src/pika_h3/core/packing.py:128 position_ids
   [S,3] float64, device memory).  axis_dims[3] are the head-dim slices per (t,h,w) axis (sum = D,
   each even); pair p of axis a rotates by pos[a] * theta^(-2*i/axis_dims[a]) with i the pair's index
   inside its axis slice.  Writes cos/sin fp32 [S, D/2]. */
int pkh3_rope_tables(const double* position_ids, int32_t S, const int32_t axis_dims[3], double theta,
                     float* cos_out, float* sin_out, void* stream);

/* ---------------------------------------------------------------------------------------------------
 * Projections around the attention call: the `to_q / to_k / to_v / to_out.0` linear layers of the
 * attention module with their LoRA adapters (target list src/pika_h3/core/loader.py:9, rank/alpha
 * injection src/pika_h3/core/loader.py:20-49, applied at src/pika_h3/pipeline.py:105-107) and the AdaLN
 * modulation that feeds them (patches/0001-h3-adaln-fp32.patch:34-40: norm(x) * (1 + scale[idx]) +
 * shift[idx], rows gathered by `timestep_indices`, src/pika_h3/core/wrapper.py:182-190,196-197).
 *
 * Matrix operands are kept as "operand images": 1 KiB blocks of 16 rows x 32 contraction elements in
 * the register order of the gfx950 16x16x32 MFMA.  Weights are packed once (pkh3_pack_weight) when
 * they are loaded; activations are packed by the kernel that produces them (pkh3_adaln_modulate) or
 * by pkh3_pack_rows.  A packed buffer for [rows, K] takes pkh3_packed_bytes(rows, K) bytes, 256-byte
 * aligned; rows are padded to a multiple of 256 with zeros.  K must be a multiple of 32 and <= 4096.
 */
enum { PKH3_NORM_NONE = 0, PKH3_NORM_LAYER = 1 /* (x - mean) * rsqrt(var + eps), no affine */,
       PKH3_NORM_RMS = 2 /* x * rsqrt(mean(x^2) + eps), no weight */ };

#define PKH3_LORA_RANK 128 /* the adapters' rank (src/pika_h3/pipeline.py:34 via the manifest); other ranks: PKH3_EUNSUPPORTED */

size_t pkh3_packed_bytes(int32_t rows, int32_t K);

/* W bf16 [N, K] (row = output feature, `row_stride` elements between rows; torch Linear.weight) -> images.
   N must be a multiple of 128.  head_perm = 1 stores the rows of every 128-feature head in the order the
   row-per-lane epilogues need (Q, K, to_out.0, LoRA A and the B matrices that go with them); head_perm = 0
   for a V projection and its LoRA B, whose epilogue holds one feature per lane. */
int pkh3_pack_weight(const void* w, int64_t row_stride, int32_t N, int32_t K, int32_t head_perm, void* out,
                     void* stream);

/* x bf16 [S, K] row-major (`row_stride` elements between rows) -> images of the activations. */
int pkh3_pack_rows(const void* x, int64_t row_stride, int32_t S, int32_t K, void* out, void* stream);

/* AdaLN modulation fused with the packing: out = images of norm(x) * (1 + scale[row_index[s]]) +
   shift[row_index[s]], statistics and arithmetic in fp32, one rounding to bf16.  shift / scale: bf16
   [table rows, table_stride] (either may be NULL: no such term); row_index int32 [S] or NULL (table row
   0 for every token).  Replaces the modulation of patches/0001-h3-adaln-fp32.patch:34-40. */
int pkh3_adaln_modulate(const void* x, int64_t row_stride, int32_t S, int32_t K, int32_t norm_kind, float eps,
                        const void* shift, const void* scale, int64_t table_stride, const int32_t* row_index,
                        void* out, void* stream);

/* One linear layer with its adapter: y = x W^T + bias + lora_scale * (x A^T) B^T. */
typedef struct pkh3_linear {
  const void* w_img;       /* pkh3_pack_weight(W [N, K]) */
  const float* bias;       /* fp32 [N] or NULL */
  const void* lora_a_img;  /* pkh3_pack_weight(A [PKH3_LORA_RANK, K], head_perm = 1) or NULL: no adapter */
  const void* lora_b_img;  /* pkh3_pack_weight(B [N, PKH3_LORA_RANK], head_perm as for w_img) */
  float lora_scale;        /* lora_alpha / rank */
} pkh3_linear;

typedef struct pkh3_qkv_args {
  const void* x_img;       /* activations [S, K] as images */
  int32_t S, K;            /* tokens, hidden size */
  pkh3_linear q, k, v;     /* N = H * 128 each; q and k packed with head_perm = 1, v with head_perm = 0 */
  void* lora_workspace;    /* scratch for the down-projected rows: pkh3_packed_bytes(S, 3 * PKH3_LORA_RANK); may be
                              NULL when no projection has an adapter.  When q, k and v all have one, with equal
                              lora_scale, and k.lora_a_img / v.lora_a_img lie 8 / 16 blocks of 16 rows (K/32 KiB each)
                              behind q.lora_a_img in one allocation of at least 32 such blocks, the three
                              down-projections run as one launch target (fewer, fuller workgroups; same results) */
  size_t lora_workspace_bytes;
} pkh3_qkv_args;

/* to_q / to_k / to_v of one self-attention call in one launch (plus one for the adapters' down-projection).
   `attn` describes the attention call that follows (B = 1, Sq = Sk = S, no key mask): Q is written as bf16 to
   attn->q with attn's strides; K goes through QK-RMSNorm (attn->k_norm_w, norm_eps), rotation (attn->rope_mode,
   k_rope_cos / k_rope_sin) and, with PKH3_FLAG_FP8_QK, quantisation, and K and V are written into attn->workspace
   in the layout the attention kernel reads.  Then call pkh3_attn_fwd(attn) with PKH3_FLAG_KV_PREPARED added.
   attn->k, attn->v and attn->o are not touched by this call. */
int pkh3_qkv_proj(const pkh3_qkv_args* p, const pkh3_attn_args* attn, void* stream);

typedef struct pkh3_out_args {
  const void* o_img;       /* attention output [S, K] as images (pkh3_pack_rows of O viewed as [S, H*128]) */
  int32_t S, K, N;
  pkh3_linear proj;        /* packed with head_perm = 1 */
  const void* gate;        /* bf16 [table rows, gate_stride] or NULL; row_index int32 [S] or NULL (row 0) */
  int64_t gate_stride;
  const int32_t* row_index;
  const void* residual;    /* bf16 [S, residual_stride] or NULL */
  int64_t residual_stride;
  void* y;                 /* bf16 [S, y_stride]: residual + gate[row_index] * (o W^T + bias + adapter) */
  int64_t y_stride;
  void* lora_workspace;    /* pkh3_packed_bytes(S, PKH3_LORA_RANK) when proj has an adapter */
  size_t lora_workspace_bytes;
} pkh3_out_args;

/* to_out.0 with its adapter and the gated residual update of the block around it. */
int pkh3_out_proj(const pkh3_out_args* p, void* stream);

int pkh3_version(void);
const char* pkh3_strerror(int code);
/* Message of the last failing call on this thread ("" if none). */
const char* pkh3_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
