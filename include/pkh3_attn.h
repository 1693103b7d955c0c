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

#define PKH3_VERSION 101

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
  PKH3_FLAG_LONG_KEY_KERNEL = 1u << 1 /* dense calls with at most 16 key tiles (Sk <= 1024) normally run a
                                 short-key form of the kernel (small workgroups, three per CU); this flag
                                 selects the long-key form for them too.  Same results to the tolerance of the
                                 path; meant for tests and measurements */
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
     blk_row_ptr int32 [ceil(Sq/64)+1], blk_col_idx int32 [blk_row_ptr[last]], columns strictly
     ascending within a row.  NULL = dense.  Rows with no tile get an all-zero output. */
  const int32_t* blk_row_ptr;
  const int32_t* blk_col_idx;
  uint32_t flags;
  /* scratch, 256-byte aligned, at least pkh3_workspace_bytes() long */
  void* workspace;
  size_t workspace_bytes;
} pkh3_attn_args;

/* Bytes of scratch pkh3_attn_fwd needs for these shapes/options (0 on invalid arguments).
   Replaces nothing in the reference: torch SDPA sizes its own scratch. */
size_t pkh3_workspace_bytes(const pkh3_attn_args* a);

/* One attention call: the arithmetic of the DiT block's attention between the q/k/v projections and
   the output projection (module at src/pika_h3/core/loader.py:9; call site src/pika_h3/core/wrapper.py:248). */
int pkh3_attn_fwd(const pkh3_attn_args* a, void* stream);

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

/* Rotary tables from the packed layout's position grid (src/pika_h3/core/packing.py:128 position_ids
   [S,3] float64, device memory).  axis_dims[3] are the head-dim slices per (t,h,w) axis (sum = D,
   each even); pair p of axis a rotates by pos[a] * theta^(-2*i/axis_dims[a]) with i the pair's index
   inside its axis slice.  Writes cos/sin fp32 [S, D/2]. */
int pkh3_rope_tables(const double* position_ids, int32_t S, const int32_t axis_dims[3], double theta,
                     float* cos_out, float* sin_out, void* stream);

int pkh3_version(void);
const char* pkh3_strerror(int code);
/* Message of the last failing call on this thread ("" if none). */
const char* pkh3_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
