// C ABI of libpkh3attn.so: argument validation (host only, before any HIP call), workspace
// planning, and the sequence of launches that makes up one attention call.
#include "../../include/pkh3_attn.h"

#include <math.h>

#include <mutex>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "pkh3_common.h"
#include "pkh3_internal.h"

using namespace pkh3;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

bool misaligned16(const void* p) { return ((uintptr_t)p & 15u) != 0; }

int check_tensor(const char* name, const void* ptr, int64_t sb, int64_t ss, int64_t sh, int B, int H) {
  if (!ptr) return fail(PKH3_ENULL, "%s is NULL", name);
  if (misaligned16(ptr)) return fail(PKH3_EALIGN, "%s is not 16-byte aligned", name);
  if (sb < 0 || ss < 0 || sh < 0) return fail(PKH3_ESTRIDE, "%s: negative stride", name);
  if ((ss % 8) || (sh % 8) || (B > 1 && (sb % 8)))
    return fail(PKH3_ESTRIDE, "%s: strides must be multiples of 8 elements (16-byte rows), got (%lld, %lld, %lld)", name,
                (long long)sb, (long long)ss, (long long)sh);
  if (H > 1 && sh == 0) return fail(PKH3_ESTRIDE, "%s: head stride is 0", name);
  return PKH3_OK;
}

// Validation shared by pkh3_workspace_bytes (shapes/options only), pkh3_attn_fwd (everything) and
// pkh3_attn_fwd_noalloc (everything but the caller's workspace, which it does not use).
int validate(const pkh3_attn_args* a, bool pointers, bool caller_workspace = true, bool need_kv = true, bool need_qo = true) {
  if (!a) return fail(PKH3_ENULL, "args is NULL");
  if (a->D != kD) return fail(PKH3_EHEADDIM, "head dim must be 128, got %d", a->D);
  if (a->B < 1 || a->H < 1 || a->Sq < 1 || a->Sk < 1) return fail(PKH3_ESHAPE, "B, H, Sq, Sk must be >= 1");
  if (a->B > 65535 || a->H > 65535) return fail(PKH3_ESHAPE, "B and H must be <= 65535");
  if (a->Sq > (1 << 24) || a->Sk > (1 << 24)) return fail(PKH3_ESHAPE, "Sq and Sk must be <= 2^24");
  // workgroup counts and tile indices are 32-bit: at most 2^30 blocks of 32 queries per call
  if ((int64_t)a->B * a->H * ((a->Sq + 31) / 32) > (1ll << 30))
    return fail(PKH3_ESHAPE, "B * H * ceil(Sq / 32) must be <= 2^30");
  if (a->flags & ~(uint32_t)(PKH3_FLAG_FP8_QK | PKH3_FLAG_LONG_KEY_KERNEL | PKH3_FLAG_KV_PREPARED | PKH3_FLAG_O_IMAGES |
                             PKH3_FLAG_FP8_POW2_SCALES))
    return fail(PKH3_EARG, "unknown flag bits 0x%x", a->flags);
  if ((a->flags & PKH3_FLAG_FP8_POW2_SCALES) && !(a->flags & PKH3_FLAG_FP8_QK))
    return fail(PKH3_EARG, "PKH3_FLAG_FP8_POW2_SCALES is an option of PKH3_FLAG_FP8_QK");
  if ((a->flags & PKH3_FLAG_O_IMAGES) && a->B != 1)
    return fail(PKH3_EUNSUPPORTED, "output as operand images (PKH3_FLAG_O_IMAGES) means one document: B = 1");
  if (a->rope_mode < PKH3_ROPE_NONE || a->rope_mode > PKH3_ROPE_HALF) return fail(PKH3_EARG, "bad rope_mode %d", a->rope_mode);
  if (!(a->softmax_scale == a->softmax_scale) || isinf(a->softmax_scale)) return fail(PKH3_EARG, "softmax_scale is not finite");
  if ((a->q_norm_w || a->k_norm_w) && !(a->norm_eps >= 0.f)) return fail(PKH3_EARG, "norm_eps must be >= 0");
  if ((a->blk_row_ptr == nullptr) != (a->blk_col_idx == nullptr))
    return fail(PKH3_ENULL, "blk_row_ptr and blk_col_idx must be given together");
  if (a->blk_row_ptr && a->key_mask) return fail(PKH3_EUNSUPPORTED, "block-sparse map together with a key mask is not supported");
  if ((a->flags & PKH3_FLAG_FP8_QK) && a->key_mask)
    return fail(PKH3_EUNSUPPORTED, "fp8 QK^T together with a key mask is not supported");
  if (!pointers) return PKH3_OK;
  int rc = PKH3_OK;
  if (need_qo && (rc = check_tensor("q", a->q, a->q_sb, a->q_ss, a->q_sh, a->B, a->H))) return rc;
  if (need_kv && !(a->flags & PKH3_FLAG_KV_PREPARED)) {
    if ((rc = check_tensor("k", a->k, a->k_sb, a->k_ss, a->k_sh, a->B, a->H))) return rc;
    if ((rc = check_tensor("v", a->v, a->v_sb, a->v_ss, a->v_sh, a->B, a->H))) return rc;
  }
  if (!need_qo) {
    // the K/V side alone: q and o are not looked at
  } else if (a->flags & PKH3_FLAG_O_IMAGES) {
    if (!a->o) return fail(PKH3_ENULL, "o is NULL");
    if (misaligned16(a->o)) return fail(PKH3_EALIGN, "o is not 16-byte aligned");
  } else if ((rc = check_tensor("o", a->o, a->o_sb, a->o_ss, a->o_sh, a->B, a->H))) {
    return rc;
  }
  if (a->rope_mode != PKH3_ROPE_NONE) {
    if (!a->q_rope_cos || !a->q_rope_sin || !a->k_rope_cos || !a->k_rope_sin)
      return fail(PKH3_ENULL, "rope_mode set but a cos/sin table is NULL");
    if (misaligned16(a->q_rope_cos) || misaligned16(a->q_rope_sin) || misaligned16(a->k_rope_cos) || misaligned16(a->k_rope_sin))
      return fail(PKH3_EALIGN, "rope tables must be 16-byte aligned");
  }
  if ((a->q_norm_w && misaligned16(a->q_norm_w)) || (a->k_norm_w && misaligned16(a->k_norm_w)))
    return fail(PKH3_EALIGN, "norm weights must be 16-byte aligned");
  if (!caller_workspace) return PKH3_OK;
  if (!a->workspace) return fail(PKH3_EWORKSPACE, "workspace is NULL");
  if ((uintptr_t)a->workspace & 255u) return fail(PKH3_EWORKSPACE, "workspace is not 256-byte aligned");
  return PKH3_OK;
}

WsPlan plan(const pkh3_attn_args* a, bool part_scratch = true) {
  WsPlan w{};
  const bool fp8 = a->flags & PKH3_FLAG_FP8_QK;
  w.nQ64 = (int)align_up((size_t)(a->Sq + 63) / 64, 4);
  w.nKt = (a->Sk + 63) / 64;
  w.kvTileBytes = (fp8 ? kK8TileBytes : kKTileBytes) + kVTileBytes;
  const size_t bh = (size_t)a->B * a->H;
  size_t off = 0;
  w.kv_off = off;     off = align_up(off + bh * w.nKt * (size_t)w.kvTileBytes, 256);
  w.kscale_off = off; if (fp8) off = align_up(off + bh * w.nKt * sizeof(float), 256);
  w.cnt_off = off;    if (a->key_mask) off = align_up(off + (size_t)a->B * sizeof(int), 256);
  w.idx_off = off;    if (a->key_mask) off = align_up(off + (size_t)a->B * a->Sk * sizeof(int), 256);
  // behind the maxima: the positions of the work queues of the fused q/k/v projection
  w.kmax_off = off;   off = align_up(off + bh * sizeof(float) + kQueues * sizeof(int), 256);
  // everything above is the K/V side and depends on B, H, Sk and the K-side options only (pkh3_kv_prepare);
  // what follows depends on the queries of the call
  w.plan_off = off;   if (a->blk_row_ptr) off = align_up(off + (size_t)(w.nQ64 / kSparseRows) * kSparseLists * w.nKt * sizeof(int), 256);
  w.plan_cnt_off = off; if (a->blk_row_ptr) off = align_up(off + (size_t)(w.nQ64 / kSparseRows) * kSparseLists * sizeof(int), 256);
  // long dense calls: partial results and arrival counters of the workgroups that may share out the units of the
  // call's last round (none for short-key calls and for calls too small to fill a round of workgroups on any device;
  // `part_scratch` false: none at all, the call then ends on whole workgroups)
  const size_t tiles384 = bh * (((size_t)w.nQ64 * 2 + 11) / 12);
  const size_t part_wgs = (!part_scratch || a->blk_row_ptr || w.nKt <= kShortMaxTiles || tiles384 < 64) ? 0
                          : (tiles384 * 8 < (size_t)kMaxPartWorkgroups ? tiles384 * 8 : (size_t)kMaxPartWorkgroups);
  w.split_bytes = part_wgs * 12 * (size_t)kPartialBytes;
  w.split_off = off;  off = align_up(off + w.split_bytes, 256);
  // positions of the work queues of a long dense call, then the arrival counters
  w.split_cnt_off = off; off = align_up(off + (kQueueSlots + part_wgs * 12) * sizeof(int), 256);
  w.total = off;
  return w;
}

struct Launch {
  WsPlan w;
  char* ws;  // scratch of this call: the caller's workspace, or the library's static array
  QkPrologueParams kp;
  VPrologueParams vp;
  FwdParams f;
  int* cnt;
  int* idx;
};

void build(const pkh3_attn_args* a, void* workspace, Launch& L, bool part_scratch = true) {
  const bool fp8 = a->flags & PKH3_FLAG_FP8_QK;
  L.w = plan(a, part_scratch);
  L.ws = (char*)workspace;
  char* ws = L.ws;
  L.cnt = a->key_mask ? (int*)(ws + L.w.cnt_off) : nullptr;
  L.idx = a->key_mask ? (int*)(ws + L.w.idx_off) : nullptr;
  const int kBytes = fp8 ? kK8TileBytes : kKTileBytes;

  QkPrologueParams& k = L.kp;
  k = QkPrologueParams{};
  k.x = a->k; k.sb = a->k_sb; k.ss = a->k_ss; k.sh = a->k_sh;
  k.B = a->B; k.H = a->H; k.S = a->Sk; k.nBlk64 = L.w.nKt;
  k.norm_w = a->k_norm_w; k.eps = a->norm_eps; k.rope_mode = a->rope_mode;
  k.cos_t = a->k_rope_cos; k.sin_t = a->k_rope_sin;
  k.gather_idx = L.idx; k.row_cnt = L.cnt;
  k.out = ws + L.w.kv_off; k.out_bh_stride = (int64_t)L.w.nKt * L.w.kvTileBytes; k.out_blk_stride = L.w.kvTileBytes;
  k.scale_out = fp8 ? (float*)(ws + L.w.kscale_off) : nullptr; k.fp8 = fp8;
  k.fp8_pow2 = (a->flags & PKH3_FLAG_FP8_POW2_SCALES) ? 1 : 0;
  k.norm_max = (unsigned*)(ws + L.w.kmax_off);

  VPrologueParams& v = L.vp;
  v = VPrologueParams{};
  v.v = a->v; v.sb = a->v_sb; v.ss = a->v_ss; v.sh = a->v_sh;
  v.B = a->B; v.H = a->H; v.S = a->Sk; v.nKt = L.w.nKt;
  v.gather_idx = L.idx; v.row_cnt = L.cnt;
  v.out = ws + L.w.kv_off + kBytes; v.out_bh_stride = k.out_bh_stride; v.out_tile_stride = L.w.kvTileBytes;
  v.zero_init = (unsigned*)(ws + L.w.kmax_off);

  FwdParams& f = L.f;
  f = FwdParams{};
  f.q = a->q; f.q_sb = a->q_sb; f.q_ss = a->q_ss; f.q_sh = a->q_sh;
  f.q_norm_w = a->q_norm_w; f.q_eps = a->norm_eps; f.q_rope_mode = a->rope_mode;
  f.q_cos = a->q_rope_cos; f.q_sin = a->q_rope_sin;
  f.kv = ws + L.w.kv_off; f.kv_bh_stride = k.out_bh_stride; f.kv_tile_stride = L.w.kvTileBytes;
  f.row_cnt = L.cnt;
  f.o = a->o; f.o_sb = a->o_sb; f.o_ss = a->o_ss; f.o_sh = a->o_sh;
  // output as the operand images of the out-projection GEMM: [16-row block][(H*128)/32 k-steps] of 1 KiB
  f.o_images = (a->flags & PKH3_FLAG_O_IMAGES) ? 1 : 0;
  f.o_img_blk_stride = (int64_t)a->H * (kD / 32) * 1024;
  f.B = a->B; f.H = a->H; f.Sq = a->Sq; f.Sk = a->Sk; f.nQ64 = L.w.nQ64; f.nKt = L.w.nKt;
  const float scale = a->softmax_scale > 0.f ? a->softmax_scale : 1.0f / sqrtf((float)kD);
  f.c = scale * kLog2e;
  f.plan = a->blk_row_ptr ? (const int*)(ws + L.w.plan_off) : nullptr;
  f.plan_cnt = a->blk_row_ptr ? (const int*)(ws + L.w.plan_cnt_off) : nullptr;
  f.plan_stride = kSparseLists * L.w.nKt;
  f.kscale = k.scale_out; f.fp8 = fp8; f.fp8_pow2 = k.fp8_pow2; f.long_key_kernel = (a->flags & PKH3_FLAG_LONG_KEY_KERNEL) ? 1 : 0;
  f.kmax = (const float*)(ws + L.w.kmax_off);
  f.split_scratch = L.w.split_bytes ? (float*)(ws + L.w.split_off) : nullptr;
  f.split_scratch_bytes = L.w.split_bytes;
  f.split_cnt = (int*)(ws + L.w.split_cnt_off) + kQueueSlots;
  f.queue_next = (int*)(ws + L.w.split_cnt_off);
}

int hip_fail(hipError_t e, const char* what) {
  return fail(PKH3_EHIP, "%s: %s", what, hipGetErrorString(e));
}

// The K/V side of a call: key-mask compaction, then V and K into the workspace in the attention kernel's layout.
int run_kv_side(const pkh3_attn_args* a, const Launch& L, hipStream_t st) {
  hipError_t e;
  if (a->key_mask) {
    if ((e = launch_mask_compact(a->key_mask, a->B, a->Sk, L.idx, L.cnt, st)) != hipSuccess) return hip_fail(e, "mask_compact");
  }
  // V first: it also clears the per-head slots the K pass max-reduces its row norms into
  if ((e = launch_v_prologue(L.vp, st)) != hipSuccess) return hip_fail(e, "v prologue");
  if ((e = launch_qk_prologue(L.kp, st)) != hipSuccess) return hip_fail(e, "k prologue");
  return PKH3_OK;
}

int run_prologue(const pkh3_attn_args* a, const Launch& L, hipStream_t st) {
  hipError_t e;
  if (a->blk_row_ptr) {
    char* ws = L.ws;
    if ((e = launch_sparse_plan(a->blk_row_ptr, a->blk_col_idx, (a->Sq + 63) / 64, L.w.nQ64, L.w.nKt, (int*)(ws + L.w.plan_off),
                                kSparseLists * L.w.nKt, (int*)(ws + L.w.plan_cnt_off), st)) != hipSuccess)
      return hip_fail(e, "sparse plan");
  }
  // prepared: pkh3_qkv_proj or pkh3_kv_prepare wrote K, V, the scales, the row-norm maxima and the compacted key list
  if (a->flags & PKH3_FLAG_KV_PREPARED) return PKH3_OK;
  return run_kv_side(a, L, st);
}

// ---- helpers of the projection entry points
size_t padded_rows(int32_t rows) { return ((size_t)rows + 255) / 256 * 256; }

int check_pack(const char* what, const void* x, int64_t row_stride, int32_t rows, int32_t K, const void* out) {
  if (!x || !out) return fail(PKH3_ENULL, "%s: NULL pointer", what);
  if (misaligned16(x)) return fail(PKH3_EALIGN, "%s: source is not 16-byte aligned", what);
  if ((uintptr_t)out & 255u) return fail(PKH3_EALIGN, "%s: destination is not 256-byte aligned", what);
  if (rows < 1) return fail(PKH3_ESHAPE, "%s: rows must be >= 1", what);
  if (K < 32 || (K % 32) || K > 4096) return fail(PKH3_ESHAPE, "%s: K must be a multiple of 32 in [32, 4096], got %d", what, K);
  if (row_stride < K || (row_stride % 8)) return fail(PKH3_ESTRIDE, "%s: row_stride must be >= K and a multiple of 8 elements", what);
  return PKH3_OK;
}

int run_pack(const void* x, int64_t row_stride, int32_t rows, int32_t K, int head_perm, int norm, float eps, const void* shift,
             const void* scale, int64_t table_stride, const int32_t* row_index, void* out, void* stream) {
  PackParams p{};
  p.x = x; p.row_stride = row_stride; p.rows = rows; p.rows_padded = (int)padded_rows(rows); p.K = K;
  p.head_perm = head_perm; p.norm = norm; p.eps = eps; p.shift = shift; p.scale = scale; p.table_stride = table_stride;
  p.row_index = row_index; p.out = (char*)out; p.out_blk_stride = (int64_t)(K / 32) * 1024;
  hipError_t e = launch_pack_rows(p, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "pack_rows");
  g_err[0] = 0;
  return PKH3_OK;
}

int check_linear(const char* name, const pkh3_linear* l) {
  if (!l->w_img || misaligned16(l->w_img)) return fail(PKH3_ENULL, "%s: w_img is NULL or misaligned", name);
  if (l->bias && misaligned16(l->bias)) return fail(PKH3_EALIGN, "%s: bias is not 16-byte aligned", name);
  if ((l->lora_a_img == nullptr) != (l->lora_b_img == nullptr))
    return fail(PKH3_ENULL, "%s: lora_a_img and lora_b_img must be given together", name);
  if (l->lora_a_img && (misaligned16(l->lora_a_img) || misaligned16(l->lora_b_img)))
    return fail(PKH3_EALIGN, "%s: adapter images are not 16-byte aligned", name);
  if (l->lora_a_img && !(l->lora_scale == l->lora_scale)) return fail(PKH3_EARG, "%s: lora_scale is not a number", name);
  return PKH3_OK;
}

// Scratch of pkh3_attn_fwd_noalloc: one array per GPU the library is loaded on, held until the process ends.
// In host code the array's name is only a handle; each device's copy has its own address, looked up once per
// device (with that device current) and used from then on wherever the memory itself is meant.
static __device__ __align__(256) unsigned char scratch[PKH3_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return fail(PKH3_EARG, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (!ptr || ((uintptr_t)ptr & 255u)) return fail(PKH3_EHIP, "built-in scratch buffer has an unusable address");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return PKH3_OK;
}

}  // namespace

namespace pkh3 {

// Everything of an attention call except the attention launch itself: validation, workspace planning and the
// prologue kernels; `out` receives the parameters the attention launch takes.  For the measurement library
// (pkh3_bench.hip), which times that launch alone.
int prepare_call(const pkh3_attn_args* a, hipStream_t st, FwdParams* out) {
  int rc = validate(a, true);
  if (rc) return rc;
  Launch L;
  build(a, a->workspace, L);
  if (a->workspace_bytes < L.w.total)
    return fail(PKH3_EWORKSPACE, "workspace too small: %zu < %zu bytes", a->workspace_bytes, L.w.total);
  if ((rc = run_prologue(a, L, st))) return rc;
  *out = L.f;
  g_err[0] = 0;
  return PKH3_OK;
}

int report_error(int code, const char* text) { return fail(code, "%s", text); }

}  // namespace pkh3

extern "C" {

int pkh3_version(void) { return PKH3_VERSION; }

const char* pkh3_last_error(void) { return g_err; }

const char* pkh3_strerror(int code) {
  switch (code) {
    case PKH3_OK: return "ok";
    case PKH3_ENULL: return "required pointer is NULL";
    case PKH3_ESHAPE: return "shape out of range";
    case PKH3_EHEADDIM: return "head dim must be 128";
    case PKH3_ESTRIDE: return "bad stride";
    case PKH3_EALIGN: return "pointer not 16-byte aligned";
    case PKH3_EWORKSPACE: return "workspace missing, misaligned or too small";
    case PKH3_EUNSUPPORTED: return "unsupported combination of options";
    case PKH3_EHIP: return "HIP runtime error";
    case PKH3_EARG: return "invalid argument";
    default: return "unknown error code";
  }
}

size_t pkh3_workspace_bytes(const pkh3_attn_args* a) {
  if (validate(a, false) != PKH3_OK) return 0;
  return plan(a).total;
}

int pkh3_attn_fwd(const pkh3_attn_args* a, void* stream) {
  int rc = validate(a, true);
  if (rc) return rc;
  Launch L;
  build(a, a->workspace, L);
  if (a->workspace_bytes < L.w.total)
    return fail(PKH3_EWORKSPACE, "workspace too small: %zu < %zu bytes", a->workspace_bytes, L.w.total);
  hipStream_t st = (hipStream_t)stream;
  if ((rc = run_prologue(a, L, st))) return rc;
  hipError_t e = launch_attn_fwd(L.f, st);
  if (e != hipSuccess) return hip_fail(e, "attn_fwd");
  g_err[0] = 0;
  return PKH3_OK;
}

int pkh3_kv_prepare(const pkh3_attn_args* a, void* stream) {
  int rc = validate(a, true, true, /*need_kv=*/true, /*need_qo=*/false);
  if (rc) return rc;
  if (a->flags & PKH3_FLAG_KV_PREPARED) return fail(PKH3_EARG, "kv_prepare: PKH3_FLAG_KV_PREPARED belongs to the calls that follow");
  Launch L;
  build(a, a->workspace, L);
  if (a->workspace_bytes < L.w.total)
    return fail(PKH3_EWORKSPACE, "workspace too small: %zu < %zu bytes", a->workspace_bytes, L.w.total);
  if ((rc = run_kv_side(a, L, (hipStream_t)stream))) return rc;
  g_err[0] = 0;
  return PKH3_OK;
}

int pkh3_noalloc_init(void) {
  void* ptr = nullptr;
  int rc = static_scratch(&ptr);
  if (rc) return rc;
  int cus = 0;
  hipError_t e = device_cu_count(&cus);
  if (e != hipSuccess) return hip_fail(e, "device properties");
  g_err[0] = 0;
  return PKH3_OK;
}

int pkh3_attn_fwd_noalloc(const pkh3_attn_args* a, void* stream) {
  int rc = validate(a, true, /*caller_workspace=*/false);
  if (rc) return rc;
  if (a->flags & PKH3_FLAG_KV_PREPARED)
    return fail(PKH3_EUNSUPPORTED, "pkh3_attn_fwd_noalloc: prepared K/V live in a caller workspace, which this call does not take");
  // the scratch of the shared last round (a matter of speed only) is left out when the built-in buffer cannot hold it
  const bool part_scratch = plan(a, true).total <= (size_t)PKH3_NOALLOC_SCRATCH_BYTES;
  const size_t need = plan(a, part_scratch).total;
  if (need > (size_t)PKH3_NOALLOC_SCRATCH_BYTES)
    return fail(PKH3_EWORKSPACE,
                "pkh3_attn_fwd_noalloc: this call needs %zu bytes of scratch, the built-in buffer holds %zu; use "
                "pkh3_attn_fwd with a caller-owned workspace",
                need, (size_t)PKH3_NOALLOC_SCRATCH_BYTES);
  void* ptr = nullptr;  // this device's copy of the built-in scratch array
  if ((rc = static_scratch(&ptr))) return rc;
  Launch L;
  build(a, ptr, L, part_scratch);
  hipStream_t st = (hipStream_t)stream;
  if ((rc = run_prologue(a, L, st))) return rc;
  hipError_t e = launch_attn_fwd(L.f, st);
  if (e != hipSuccess) return hip_fail(e, "attn_fwd");
  g_err[0] = 0;
  return PKH3_OK;
}

int pkh3_rope_tables(const double* position_ids, int32_t S, const int32_t axis_dims[3], double theta, float* cos_out,
                     float* sin_out, void* stream) {
  if (!position_ids || !axis_dims || !cos_out || !sin_out) return fail(PKH3_ENULL, "rope_tables: NULL argument");
  if (S < 1) return fail(PKH3_ESHAPE, "rope_tables: S must be >= 1");
  int sum = 0;
  for (int i = 0; i < 3; ++i) {
    if (axis_dims[i] < 0 || (axis_dims[i] & 1)) return fail(PKH3_EARG, "rope_tables: axis dims must be even and >= 0");
    sum += axis_dims[i];
  }
  if (sum != kD) return fail(PKH3_EARG, "rope_tables: axis dims must sum to 128, got %d", sum);
  if (!(theta > 1.0)) return fail(PKH3_EARG, "rope_tables: theta must be > 1");
  hipError_t e = launch_rope_tables(position_ids, S, axis_dims, theta, cos_out, sin_out, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "rope_tables");
  g_err[0] = 0;
  return PKH3_OK;
}

// ---- projections ------------------------------------------------------------------------------------------

size_t pkh3_packed_bytes(int32_t rows, int32_t K) {
  if (rows < 1 || K < 32 || (K % 32) || K > 4096) return 0;
  return padded_rows(rows) * (size_t)K * 2;
}

int pkh3_pack_weight(const void* w, int64_t row_stride, int32_t N, int32_t K, int32_t head_perm, void* out, void* stream) {
  int rc = check_pack("pack_weight", w, row_stride, N, K, out);
  if (rc) return rc;
  if (N % 128) return fail(PKH3_ESHAPE, "pack_weight: N must be a multiple of 128 (whole heads), got %d", N);
  return run_pack(w, row_stride, N, K, head_perm ? 1 : 0, kNormNone, 0.f, nullptr, nullptr, 0, nullptr, out, stream);
}

int pkh3_pack_rows(const void* x, int64_t row_stride, int32_t S, int32_t K, void* out, void* stream) {
  int rc = check_pack("pack_rows", x, row_stride, S, K, out);
  if (rc) return rc;
  return run_pack(x, row_stride, S, K, 0, kNormNone, 0.f, nullptr, nullptr, 0, nullptr, out, stream);
}

int pkh3_adaln_modulate(const void* x, int64_t row_stride, int32_t S, int32_t K, int32_t norm_kind, float eps,
                        const void* shift, const void* scale, int64_t table_stride, const int32_t* row_index, void* out,
                        void* stream) {
  int rc = check_pack("adaln_modulate", x, row_stride, S, K, out);
  if (rc) return rc;
  if (norm_kind < PKH3_NORM_NONE || norm_kind > PKH3_NORM_RMS) return fail(PKH3_EARG, "adaln_modulate: bad norm_kind %d", norm_kind);
  if (norm_kind != PKH3_NORM_NONE && !(eps >= 0.f)) return fail(PKH3_EARG, "adaln_modulate: eps must be >= 0");
  if (norm_kind == PKH3_NORM_NONE && (shift || scale))
    return fail(PKH3_EUNSUPPORTED, "adaln_modulate: shift/scale without a norm is not implemented");
  if ((shift && misaligned16(shift)) || (scale && misaligned16(scale)))
    return fail(PKH3_EALIGN, "adaln_modulate: shift/scale tables must be 16-byte aligned");
  if ((shift || scale) && (table_stride < K || (table_stride % 8)))
    return fail(PKH3_ESTRIDE, "adaln_modulate: table_stride must be >= K and a multiple of 8 elements");
  return run_pack(x, row_stride, S, K, 0, norm_kind, eps, shift, scale, table_stride, row_index, out, stream);
}

int pkh3_qkv_proj(const pkh3_qkv_args* p, const pkh3_attn_args* a, void* stream) {
  if (!p) return fail(PKH3_ENULL, "qkv_proj: args is NULL");
  int rc = validate(a, true, true, /*need_kv=*/false);
  if (rc) return rc;
  if (a->B != 1 || a->Sq != a->Sk || a->key_mask)
    return fail(PKH3_EUNSUPPORTED, "qkv_proj: one self-attention document only (B = 1, Sq = Sk, no key mask)");
  if (p->S != a->Sq) return fail(PKH3_ESHAPE, "qkv_proj: S = %d but the attention call has Sq = %d", p->S, a->Sq);
  if (p->K < 32 || (p->K % 32) || p->K > 4096) return fail(PKH3_ESHAPE, "qkv_proj: K must be a multiple of 32 in [32, 4096], got %d", p->K);
  if (!p->x_img || misaligned16(p->x_img)) return fail(PKH3_ENULL, "qkv_proj: x_img is NULL or misaligned");
  if (a->q_sh > INT32_MAX) return fail(PKH3_ESTRIDE, "qkv_proj: q head stride too large");
  const pkh3_linear* lin[3] = {&p->q, &p->k, &p->v};
  const char* names[3] = {"q", "k", "v"};
  bool any_lora = false;
  for (int t = 0; t < 3; ++t) {
    if ((rc = check_linear(names[t], lin[t]))) return rc;
    any_lora |= lin[t]->lora_a_img != nullptr;
  }
  const size_t lora_need = any_lora ? pkh3_packed_bytes(p->S, 3 * PKH3_LORA_RANK) : 0;
  if (any_lora && (!p->lora_workspace || ((uintptr_t)p->lora_workspace & 255u) || p->lora_workspace_bytes < lora_need))
    return fail(PKH3_EWORKSPACE, "qkv_proj: lora_workspace missing, misaligned (256 B) or smaller than %zu bytes", lora_need);
  Launch L;
  build(a, a->workspace, L);
  if (a->workspace_bytes < L.w.total)
    return fail(PKH3_EWORKSPACE, "workspace too small: %zu < %zu bytes", a->workspace_bytes, L.w.total);
  hipStream_t st = (hipStream_t)stream;
  hipError_t e;
  const int H = a->H, N = H * kD;
  const bool fp8 = a->flags & PKH3_FLAG_FP8_QK;
  const int64_t w_blk = (int64_t)(p->K / 32) * 1024;       // bytes of one 16-row block of images over K
  const int64_t b_blk = (int64_t)(PKH3_LORA_RANK / 32) * 1024;
  const int64_t xa_blk = 3 * b_blk;                        // down-projected rows: three targets side by side
  const int m_tiles = (int)(padded_rows(p->S) / 256);

  // the K epilogue max-reduces its row norms into per-head slots that must start at zero; so must the positions of
  // the projection's work queues behind them
  if ((e = launch_fill_zero((unsigned*)(L.ws + L.w.kmax_off), H + kQueues, st)) != hipSuccess) return hip_fail(e, "fill_zero");

  if (any_lora) {
    // x A^T for the three adapters, scaled, as the activation images of the second K segment
    GemmParams g{};
    g.a_img = (const char*)p->x_img; g.a_blk_stride = w_blk; g.nk1 = p->K / 32; g.M = p->S; g.m_tiles = m_tiles;
    // Three adapters whose A images lie one behind the other (8 blocks of 16 features each) with one scale are one
    // target of three heads: two workgroup tiles per 256 tokens instead of three half-empty ones.
    const char* a0 = (const char*)lin[0]->lora_a_img;
    const bool together = a0 && (const char*)lin[1]->lora_a_img == a0 + 8 * w_blk && (const char*)lin[2]->lora_a_img == a0 + 16 * w_blk &&
                          lin[0]->lora_scale == lin[1]->lora_scale && lin[0]->lora_scale == lin[2]->lora_scale;
    if (together) {
      GemmTarget& tg = g.tg[g.n_targets++];
      tg = GemmTarget{};
      tg.epi = kEpiAImg; tg.n = 3 * PKH3_LORA_RANK; tg.n_tiles = 2;
      tg.w_img = a0; tg.w_blk_stride = w_blk;
      tg.out_scale = lin[0]->lora_scale;
      tg.out = (char*)p->lora_workspace; tg.out_head_stride = b_blk;
      tg.out_blk_stride = xa_blk;
      tg.rope_mode = PKH3_ROPE_NONE;
      g.n_tiles += 2;
    }
    for (int t = 0; t < 3 && !together; ++t) {
      if (!lin[t]->lora_a_img) continue;
      GemmTarget& tg = g.tg[g.n_targets++];
      tg = GemmTarget{};
      tg.epi = kEpiAImg; tg.n = PKH3_LORA_RANK; tg.n_tiles = 1;
      tg.w_img = (const char*)lin[t]->lora_a_img; tg.w_blk_stride = w_blk;
      tg.out_scale = lin[t]->lora_scale;
      tg.out = (char*)p->lora_workspace + t * b_blk; tg.out_head_stride = 0;
      tg.out_blk_stride = xa_blk;
      tg.rope_mode = PKH3_ROPE_NONE;
      g.n_tiles += 1;
    }
    if ((e = launch_gemm(g, st)) != hipSuccess) return hip_fail(e, "lora down-projection");
  }

  GemmParams g{};
  g.a_img = (const char*)p->x_img; g.a_blk_stride = w_blk; g.nk1 = p->K / 32; g.M = p->S; g.m_tiles = m_tiles;
  g.n_targets = 3;
  for (int t = 0; t < 3; ++t) {
    GemmTarget& tg = g.tg[t];
    tg = GemmTarget{};
    tg.n = N; tg.n_tiles = (N + 255) / 256;
    tg.w_img = (const char*)lin[t]->w_img; tg.w_blk_stride = w_blk;
    tg.bias = lin[t]->bias; tg.out_scale = 1.0f;
    if (lin[t]->lora_a_img) {
      tg.a2_img = (const char*)p->lora_workspace + t * b_blk; tg.a2_blk_stride = xa_blk;
      tg.w2_img = (const char*)lin[t]->lora_b_img; tg.w2_blk_stride = b_blk; tg.nk2 = PKH3_LORA_RANK / 32;
    }
    g.n_tiles += tg.n_tiles;
  }
  {
    GemmTarget& q = g.tg[0];
    q.epi = kEpiRows; q.out = (char*)a->q; q.out_row_stride = a->q_ss; q.out_head_elems = (int)a->q_sh;
    GemmTarget& k = g.tg[1];
    k.epi = kEpiKImg; k.out = L.kp.out; k.out_head_stride = L.kp.out_bh_stride; k.out_blk_stride = L.kp.out_blk_stride;
    k.norm_w = a->k_norm_w; k.norm_eps = a->norm_eps; k.rope_mode = a->rope_mode; k.cos_t = a->k_rope_cos; k.sin_t = a->k_rope_sin;
    k.norm_max = L.kp.norm_max; k.fp8 = fp8; k.fp8_pow2 = L.kp.fp8_pow2; k.scale_out = L.kp.scale_out; k.scale_head_stride = L.w.nKt;
    GemmTarget& v = g.tg[2];
    v.epi = kEpiVImg; v.out = L.vp.out; v.out_head_stride = L.vp.out_bh_stride; v.out_blk_stride = L.vp.out_tile_stride;
  }
  // launches of at least two rounds of workgroups take their tiles from per-XCD work queues
  int cus = 0;
  if ((e = device_cu_count(&cus)) != hipSuccess) return hip_fail(e, "device_cu_count");
  if (cus > 0 && g.m_tiles * g.n_tiles >= 2 * cus) g.queue_next = (int*)(L.ws + L.w.kmax_off) + H;
  if ((e = launch_gemm(g, st)) != hipSuccess) return hip_fail(e, "qkv projection");
  g_err[0] = 0;
  return PKH3_OK;
}

int pkh3_out_proj(const pkh3_out_args* p, void* stream) {
  if (!p) return fail(PKH3_ENULL, "out_proj: args is NULL");
  if (p->S < 1) return fail(PKH3_ESHAPE, "out_proj: S must be >= 1");
  if (p->K < 32 || (p->K % 32) || p->K > 4096) return fail(PKH3_ESHAPE, "out_proj: K must be a multiple of 32 in [32, 4096], got %d", p->K);
  if (p->N < 128 || (p->N % 128)) return fail(PKH3_ESHAPE, "out_proj: N must be a multiple of 128, got %d", p->N);
  if (!p->o_img || misaligned16(p->o_img)) return fail(PKH3_ENULL, "out_proj: o_img is NULL or misaligned");
  if (!p->y || misaligned16(p->y)) return fail(PKH3_ENULL, "out_proj: y is NULL or misaligned");
  if (p->y_stride < p->N || (p->y_stride % 8)) return fail(PKH3_ESTRIDE, "out_proj: y_stride must be >= N and a multiple of 8 elements");
  if (p->gate && (misaligned16(p->gate) || p->gate_stride < p->N || (p->gate_stride % 8)))
    return fail(PKH3_ESTRIDE, "out_proj: gate table misaligned or gate_stride not >= N and a multiple of 8");
  if (p->residual && (misaligned16(p->residual) || p->residual_stride < p->N || (p->residual_stride % 8)))
    return fail(PKH3_ESTRIDE, "out_proj: residual misaligned or residual_stride not >= N and a multiple of 8");
  int rc = check_linear("to_out", &p->proj);
  if (rc) return rc;
  const bool lora = p->proj.lora_a_img != nullptr;
  const size_t lora_need = lora ? pkh3_packed_bytes(p->S, PKH3_LORA_RANK) : 0;
  if (lora && (!p->lora_workspace || ((uintptr_t)p->lora_workspace & 255u) || p->lora_workspace_bytes < lora_need))
    return fail(PKH3_EWORKSPACE, "out_proj: lora_workspace missing, misaligned (256 B) or smaller than %zu bytes", lora_need);
  hipStream_t st = (hipStream_t)stream;
  hipError_t e;
  const int64_t w_blk = (int64_t)(p->K / 32) * 1024;
  const int64_t b_blk = (int64_t)(PKH3_LORA_RANK / 32) * 1024;
  const int m_tiles = (int)(padded_rows(p->S) / 256);
  if (lora) {
    GemmParams g{};
    g.a_img = (const char*)p->o_img; g.a_blk_stride = w_blk; g.nk1 = p->K / 32; g.M = p->S; g.m_tiles = m_tiles;
    g.n_targets = 1; g.n_tiles = 1;
    GemmTarget& tg = g.tg[0];
    tg = GemmTarget{};
    tg.epi = kEpiAImg; tg.n = PKH3_LORA_RANK; tg.n_tiles = 1;
    tg.w_img = (const char*)p->proj.lora_a_img; tg.w_blk_stride = w_blk; tg.out_scale = p->proj.lora_scale;
    tg.out = (char*)p->lora_workspace; tg.out_blk_stride = b_blk;
    if ((e = launch_gemm(g, st)) != hipSuccess) return hip_fail(e, "lora down-projection");
  }
  GemmParams g{};
  g.a_img = (const char*)p->o_img; g.a_blk_stride = w_blk; g.nk1 = p->K / 32; g.M = p->S; g.m_tiles = m_tiles;
  g.n_targets = 1;
  GemmTarget& tg = g.tg[0];
  tg = GemmTarget{};
  tg.epi = kEpiRows; tg.n = p->N; tg.n_tiles = (p->N + 255) / 256; g.n_tiles = tg.n_tiles;
  tg.w_img = (const char*)p->proj.w_img; tg.w_blk_stride = w_blk; tg.bias = p->proj.bias; tg.out_scale = 1.0f;
  if (lora) {
    tg.a2_img = (const char*)p->lora_workspace; tg.a2_blk_stride = b_blk;
    tg.w2_img = (const char*)p->proj.lora_b_img; tg.w2_blk_stride = b_blk; tg.nk2 = PKH3_LORA_RANK / 32;
  }
  tg.out = (char*)p->y; tg.out_row_stride = p->y_stride; tg.out_head_elems = kD;
  tg.gate = p->gate; tg.gate_row_stride = p->gate_stride; tg.row_index = p->row_index;
  tg.residual = p->residual; tg.res_row_stride = p->residual_stride;
  if ((e = launch_gemm(g, st)) != hipSuccess) return hip_fail(e, "output projection");
  g_err[0] = 0;
  return PKH3_OK;
}

}  // extern "C"
