"""Tensor-level front end of the C ABI: takes torch tensors (device memory + strides), fills
``pkh3_attn_args`` and enqueues the call on torch's current HIP stream.  PyTorch is used here for
memory and streams only; all arithmetic happens in libpkh3attn.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib

HEAD_DIM = 128


@dataclass
class BlockMask:
    """64x64-tile block-sparse map in CSR form (int32, on the device), shared by batches and heads."""

    row_ptr: torch.Tensor  # [ceil(Sq/64)+1]
    col_idx: torch.Tensor  # [nnz]
    n_cols: Optional[int] = None  # key tiles of the map it was built from (checked against ceil(Sk/64) when known)

    @staticmethod
    def from_dense(tile_map: torch.Tensor, device=None) -> "BlockMask":
        """``tile_map``: bool [ceil(Sq/64), ceil(Sk/64)], True = compute that tile."""
        tm = tile_map.to("cpu", torch.bool)
        counts = tm.sum(dim=1, dtype=torch.int64)
        row_ptr = torch.zeros(tm.shape[0] + 1, dtype=torch.int32)
        row_ptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
        col_idx = tm.nonzero(as_tuple=False)[:, 1].to(torch.int32).contiguous()
        if col_idx.numel() == 0:
            col_idx = torch.zeros(1, dtype=torch.int32)
        dev = device if device is not None else tile_map.device
        return BlockMask(row_ptr.to(dev), col_idx.to(dev), int(tm.shape[1]))


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_bshd(name: str, t: torch.Tensor) -> None:
    if t.dim() != 4:
        raise ValueError(f"{name} must be [B, S, H, D], got shape {tuple(t.shape)}")
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
    if t.stride(3) != 1:
        raise ValueError(f"{name}: head-dim stride must be 1, got {t.stride(3)}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live in device memory (got {t.device}); the HIP library is the only compute path")


def _on_device(name: str, t: torch.Tensor, device) -> None:
    """Every pointer handed to the library is dereferenced by a kernel running on ``device``."""
    if t.device != device:
        raise ValueError(f"{name} must live in device memory on {device} (got {t.device})")


def _f32(name: str, t: Optional[torch.Tensor], shape, device) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must be contiguous float32 {tuple(shape)}, got {t.dtype} {tuple(t.shape)}")
    _on_device(name, t, device)
    return t


FP8_POW2 = "pow2"  # value of ``fp8_qk`` that selects power-of-two block scales (PKH3_FLAG_FP8_POW2_SCALES)


def fp8_mode(fp8_qk) -> object:
    """Normal form of the ``fp8_qk`` option: False, True (absmax / 448 scales) or ``"pow2"`` (every block scale
    the smallest power of two >= absmax / 448, softmax scale folded into Q before quantisation: faster, same e4m3
    rounding error)."""
    if isinstance(fp8_qk, str):
        if fp8_qk != FP8_POW2:
            raise ValueError(f'fp8_qk must be False, True or "{FP8_POW2}", got {fp8_qk!r}')
        return FP8_POW2
    return bool(fp8_qk)


def fill_args(
    q, k, v, out, *, q_norm_weight=None, k_norm_weight=None, norm_eps=1e-6, rope_q=None, rope_k=None,
    rope_mode=_lib.ROPE_NONE, key_mask=None, block_mask: Optional[BlockMask] = None, fp8_qk=False,
    softmax_scale: Optional[float] = None, long_key_kernel: bool = False, kv_prepared: bool = False,
    out_images: bool = False, prepared_keys: Optional[int] = None,
) -> Tuple[_lib.AttnArgs, list]:
    """Build ``pkh3_attn_args`` for these tensors.  Returns (args, keep_alive).  ``kv_prepared``: K and V
    come through the workspace, from the fused projection (``pkh3_qkv_proj``) or from ``pkh3_kv_prepare``
    (then ``prepared_keys`` is their Sk); ``k`` and ``v`` are then None.
    ``fp8_qk``: False, True or ``"pow2"`` (see :func:`fp8_mode`).
    ``out_images``: ``out`` is a uint8 operand-image buffer for ``pkh3_out_proj`` (``projections.packed_bytes(Sq,
    H*D)`` bytes) instead of a ``[B, Sq, H, D]`` tensor, and B must be 1."""
    if kv_prepared != (k is None) or (k is None) != (v is None):
        raise ValueError("k and v are None exactly when kv_prepared is set")
    for n, t in (("q", q), ("k", k), ("v", v)) + (() if out_images else (("out", out),)):
        if t is not None:
            _check_bshd(n, t)
    B, Sq, H, D = q.shape
    Sk = (Sq if prepared_keys is None else int(prepared_keys)) if k is None else k.shape[1]
    if k is not None and (tuple(k.shape) != (B, Sk, H, D) or tuple(v.shape) != (B, Sk, H, D)):
        raise ValueError(f"k/v shapes {tuple(k.shape)}/{tuple(v.shape)} do not match q {tuple(q.shape)}")
    if out_images:
        need = ((Sq + 255) // 256 * 256) * H * D * 2
        if out.dtype != torch.uint8 or not out.is_contiguous() or out.numel() < need or B != 1:
            raise ValueError(f"out_images: out must be a contiguous uint8 buffer of at least {need} bytes and B must be 1")
    elif tuple(out.shape) != (B, Sq, H, D):
        raise ValueError(f"out shape {tuple(out.shape)} != {(B, Sq, H, D)}")
    dev = q.device
    for n, t in (("k", k), ("v", v), ("out", out)):
        if t is not None:
            _on_device(n, t, dev)
    keep = [q, k, v, out]
    a = _lib.AttnArgs()
    a.q, a.o = q.data_ptr(), out.data_ptr()
    a.q_sb, a.q_ss, a.q_sh = q.stride(0), q.stride(1), q.stride(2)
    if k is not None:
        a.k, a.v = k.data_ptr(), v.data_ptr()
        a.k_sb, a.k_ss, a.k_sh = k.stride(0), k.stride(1), k.stride(2)
        a.v_sb, a.v_ss, a.v_sh = v.stride(0), v.stride(1), v.stride(2)
    if not out_images:
        a.o_sb, a.o_ss, a.o_sh = out.stride(0), out.stride(1), out.stride(2)
    a.B, a.H, a.Sq, a.Sk, a.D = B, H, Sq, Sk, D
    a.softmax_scale = float(softmax_scale) if softmax_scale is not None else 0.0
    qw = _f32("q_norm_weight", q_norm_weight, (D,), dev)
    kw = _f32("k_norm_weight", k_norm_weight, (D,), dev)
    a.q_norm_w, a.k_norm_w, a.norm_eps = _ptr(qw), _ptr(kw), float(norm_eps)
    a.rope_mode = int(rope_mode)
    if rope_mode != _lib.ROPE_NONE:
        if rope_q is None:
            raise ValueError("rope_mode set but rope_q tables missing")
        if rope_k is None:
            if Sq != Sk:
                raise ValueError("rope_k tables are required when Sq != Sk")
            rope_k = rope_q
        qc, qs = _f32("rope_q cos", rope_q[0], (Sq, D // 2), dev), _f32("rope_q sin", rope_q[1], (Sq, D // 2), dev)
        kc, ks = _f32("rope_k cos", rope_k[0], (Sk, D // 2), dev), _f32("rope_k sin", rope_k[1], (Sk, D // 2), dev)
        a.q_rope_cos, a.q_rope_sin, a.k_rope_cos, a.k_rope_sin = qc.data_ptr(), qs.data_ptr(), kc.data_ptr(), ks.data_ptr()
        keep += [qc, qs, kc, ks]
    if key_mask is not None:
        if tuple(key_mask.shape) != (B, Sk):
            raise ValueError(f"key_mask must be [B, Sk] = {(B, Sk)}, got {tuple(key_mask.shape)}")
        _on_device("key_mask", key_mask, dev)
        km = key_mask.to(torch.uint8).contiguous() if key_mask.dtype != torch.uint8 else key_mask.contiguous()
        a.key_mask = km.data_ptr()
        keep.append(km)
    if block_mask is not None:
        nrow = (Sq + 63) // 64
        if block_mask.row_ptr.dtype != torch.int32 or block_mask.col_idx.dtype != torch.int32:
            raise TypeError("block mask CSR arrays must be int32")
        if block_mask.row_ptr.numel() != nrow + 1:
            raise ValueError(f"block mask has {block_mask.row_ptr.numel() - 1} tile rows, need {nrow}")
        if block_mask.n_cols is not None and block_mask.n_cols != (Sk + 63) // 64:
            raise ValueError(f"block mask has {block_mask.n_cols} tile columns, need {(Sk + 63) // 64}")
        _on_device("block mask row_ptr", block_mask.row_ptr, dev)
        _on_device("block mask col_idx", block_mask.col_idx, dev)
        if not (block_mask.row_ptr.is_contiguous() and block_mask.col_idx.is_contiguous()):
            raise ValueError("block mask CSR arrays must be contiguous")
        a.blk_row_ptr, a.blk_col_idx = block_mask.row_ptr.data_ptr(), block_mask.col_idx.data_ptr()
        keep += [block_mask.row_ptr, block_mask.col_idx]
    fp8_qk = fp8_mode(fp8_qk)
    a.flags = ((_lib.FLAG_FP8_QK if fp8_qk else 0) | (_lib.FLAG_FP8_POW2_SCALES if fp8_qk == FP8_POW2 else 0)
               | (_lib.FLAG_LONG_KEY_KERNEL if long_key_kernel else 0)
               | (_lib.FLAG_KV_PREPARED if kv_prepared else 0) | (_lib.FLAG_O_IMAGES if out_images else 0))
    keep += [qw, kw]
    return a, keep


def workspace_bytes(args: _lib.AttnArgs) -> int:
    n = _lib.load().pkh3_workspace_bytes(C.byref(args))
    if n == 0:
        raise _lib.Pkh3Error(_lib.PKH3_EARG, _lib.load().pkh3_last_error().decode())
    return int(n)


def attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, out: Optional[torch.Tensor] = None,
    workspace=None, static_scratch: bool = False, **opts,
) -> torch.Tensor:
    """softmax(norm_rope(q) norm_rope(k)^T * scale) v over ``[B, S, H, D]`` bf16 views (any strides
    with a unit head-dim stride).  Keyword options are those of :func:`fill_args`.  ``workspace`` is a
    uint8 device tensor to use as scratch when large enough, or a callable ``(device, nbytes) -> tensor``
    that provides one; without it a fresh buffer is allocated.  ``static_scratch=True`` calls the
    entry point that allocates nothing instead (``pkh3_attn_fwd_noalloc``: scratch built into the library,
    at most ``_lib.NOALLOC_SCRATCH_BYTES``; pass ``out`` as well and the call touches no allocator at all).
    Runs asynchronously on the current stream and returns ``out`` ([B, Sq, H, D], bf16)."""
    lib = _lib.load()
    if out is None:
        if opts.get("out_images"):
            raise ValueError("out_images needs the image buffer as out")
        out = torch.empty((q.shape[0], q.shape[1], q.shape[2], q.shape[3]), dtype=torch.bfloat16, device=q.device)
    args, keep = fill_args(q, k, v, out, **opts)
    if static_scratch:
        with torch.cuda.device(q.device):
            _lib.check(lib.pkh3_attn_fwd_noalloc(C.byref(args), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        return out
    need = workspace_bytes(args)
    if callable(workspace):
        workspace = workspace(q.device, need)
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    args.workspace = workspace.data_ptr()
    args.workspace_bytes = workspace.numel() * workspace.element_size()
    if workspace.device != q.device:
        raise ValueError(f"workspace must live on {q.device} (got {workspace.device})")
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream()
        _lib.check(lib.pkh3_attn_fwd(C.byref(args), C.c_void_p(stream.cuda_stream)))
        # the workspace must outlive the kernels: tie it to the stream, not to this Python frame
        workspace.record_stream(stream)
    return out


def noalloc_init(device=None) -> None:
    """Set-up of the ``static_scratch=True`` calls on ``device`` (default: the current one): ``pkh3_noalloc_init``.
    Needed once per device before such a call is captured into a HIP graph; otherwise the first call does it."""
    lib = _lib.load()
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        _lib.check(lib.pkh3_noalloc_init())


@dataclass
class PreparedKV:
    """Keys and values of :func:`prepare_kv`, ready for any number of :func:`attention` calls."""

    workspace: torch.Tensor  # holds K', V, scales, row-norm maxima and the compacted key list
    B: int
    Sk: int
    H: int
    opts: dict               # the K-side options every later call must repeat


K_SIDE_OPTIONS = ("k_norm_weight", "norm_eps", "rope_k", "rope_mode", "key_mask", "fp8_qk")


def prepare_kv(k: torch.Tensor, v: torch.Tensor, *, q_rows: Optional[int] = None, block_sparse: bool = False,
               **opts) -> PreparedKV:
    """The K/V side of :func:`attention` on its own (``pkh3_kv_prepare``): for keys and values several calls
    share, e.g. the text keys of a block's cross-attention over the denoising steps.  ``opts``: ``k_norm_weight``,
    ``norm_eps``, ``rope_mode`` + ``rope_k``, ``key_mask``, ``fp8_qk``.  Dense calls need no more scratch than the
    K/V side itself; when calls with a ``block_mask`` will follow, say so (``block_sparse=True``) and give the largest
    query count among them (``q_rows``, default Sk), so that the workspace has room for their tile lists."""
    lib = _lib.load()
    unknown = set(opts) - set(K_SIDE_OPTIONS)
    if unknown:
        raise ValueError(f"prepare_kv takes the K-side options {K_SIDE_OPTIONS}, got {sorted(unknown)}")
    _check_bshd("k", k)
    B, Sk, H, D = k.shape
    full = dict(opts)
    if full.get("rope_mode", _lib.ROPE_NONE) != _lib.ROPE_NONE:
        full["rope_q"] = full.get("rope_k")  # the call validates four tables; the Q pair is not read here
    # a stand-in for q and o with the right shape and device (one row of storage): this entry point reads neither
    stand_in = torch.empty((1, 1, 1, D), dtype=k.dtype, device=k.device).expand(B, Sk, H, D)
    args, keep = fill_args(stand_in, k, v, stand_in, **full)
    args.Sq = int(q_rows or Sk)
    need = workspace_bytes(args)
    if block_sparse:
        # size with a block map present (only the pointers' presence matters to the sizing call)
        args.blk_row_ptr = args.blk_col_idx = k.data_ptr()
        need = max(need, workspace_bytes(args))   # dense calls carry scratch of their own kind: room for either
        args.blk_row_ptr = args.blk_col_idx = None
    ws = torch.empty(need, dtype=torch.uint8, device=k.device)
    args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
    args.q = args.o = None
    with torch.cuda.device(k.device):
        _lib.check(lib.pkh3_kv_prepare(C.byref(args), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    return PreparedKV(ws, int(B), int(Sk), int(H), dict(opts))


def attention_prepared(q: torch.Tensor, kv: PreparedKV, *, out: Optional[torch.Tensor] = None, **q_opts) -> torch.Tensor:
    """:func:`attention` of ``q`` against prepared keys and values.  ``q_opts``: the Q-side options
    (``q_norm_weight``, ``rope_q``, ``softmax_scale``, ``long_key_kernel``); the K-side ones come from ``kv``."""
    lib = _lib.load()
    clash = set(q_opts) & set(K_SIDE_OPTIONS)
    if clash:
        raise ValueError(f"K-side options belong to prepare_kv: {sorted(clash)}")
    if out is None:
        out = torch.empty_like(q)
    opts = dict(kv.opts)
    opts.update(q_opts)
    args, keep = fill_args(q, None, None, out, kv_prepared=True, prepared_keys=kv.Sk, **opts)
    if (args.B, args.H) != (kv.B, kv.H):
        raise ValueError(f"q has batch {args.B} and {args.H} heads, the prepared keys {kv.B} and {kv.H}")
    _on_device("prepared workspace", kv.workspace, q.device)
    need = workspace_bytes(args)
    if kv.workspace.numel() < need:
        raise ValueError(f"the prepared workspace holds {kv.workspace.numel()} bytes, this call needs {need} (give prepare_kv q_rows)")
    args.workspace, args.workspace_bytes = kv.workspace.data_ptr(), kv.workspace.numel()
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream()
        _lib.check(lib.pkh3_attn_fwd(C.byref(args), C.c_void_p(stream.cuda_stream)))
        kv.workspace.record_stream(stream)
    return out


def time_attention_kernel(q, k, v, *, iters: int = 10, **opts) -> float:
    """Mean milliseconds per launch of the attention kernel alone (prologue excluded), measured with
    HIP events on the current stream inside the measurement library (``libpkh3attn_bench.so``)."""
    lib = _lib.load_bench()
    out = torch.empty_like(q)
    args, keep = fill_args(q, k, v, out, **opts)
    ws = torch.empty(workspace_bytes(args), dtype=torch.uint8, device=q.device)
    args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
    ms = C.c_float(0.0)
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.pkh3_attn_time_kernel(C.byref(args), C.c_void_p(stream), int(iters), C.byref(ms)))
    return float(ms.value)


def rope_tables(position_ids: torch.Tensor, axis_dims=(32, 48, 48), theta: float = 10000.0):
    """cos/sin fp32 ``[S, 64]`` from the packed layout's ``position_ids`` ``[S, 3]`` float64 (device)."""
    lib = _lib.load()
    if position_ids.dim() != 2 or position_ids.shape[1] != 3:
        raise ValueError(f"position_ids must be [S, 3], got {tuple(position_ids.shape)}")
    if not position_ids.is_cuda:
        raise ValueError("position_ids must live in device memory")
    pos = position_ids.to(torch.float64).contiguous()
    S = pos.shape[0]
    cos = torch.empty((S, HEAD_DIM // 2), dtype=torch.float32, device=pos.device)
    sin = torch.empty_like(cos)
    dims = (C.c_int32 * 3)(*[int(x) for x in axis_dims])
    with torch.cuda.device(pos.device):
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.pkh3_rope_tables(pos.data_ptr(), S, dims, float(theta), cos.data_ptr(), sin.data_ptr(), C.c_void_p(stream)))
    return cos, sin
