"""Tensor-level front end of the projection entry points of the C ABI: the ``to_q / to_k / to_v /
to_out.0`` linear layers of the attention module with their LoRA adapters (target list
src/pika_h3/core/loader.py:9, injection src/pika_h3/core/loader.py:20-49) and the AdaLN modulation
that feeds them (patches/0001-h3-adaln-fp32.patch:34-40).  PyTorch supplies device memory and the
stream; all arithmetic happens in libpkh3attn.so.

Matrix operands live in "operand images" (uint8 tensors here): weights are packed once with
:func:`pack_weight` / :meth:`PackedLinear.from_weights`, activations by :func:`adaln_modulate` or
:func:`pack_rows`.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from .ops import HEAD_DIM, _on_device, fill_args, workspace_bytes

NORMS = {"none": _lib.NORM_NONE, "layer": _lib.NORM_LAYER, "rms": _lib.NORM_RMS}


def _stream(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _rows_bf16(name: str, t: torch.Tensor) -> torch.Tensor:
    if t.dim() != 2 or t.dtype != torch.bfloat16 or t.stride(1) != 1:
        raise ValueError(f"{name} must be a bfloat16 [rows, K] matrix with unit column stride, got {t.dtype} {tuple(t.shape)}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live in device memory (got {t.device}); the HIP library is the only compute path")
    return t


def packed_bytes(rows: int, K: int) -> int:
    n = _lib.load().pkh3_packed_bytes(int(rows), int(K))
    if n == 0:
        raise ValueError(f"cannot pack a [{rows}, {K}] matrix: K must be a multiple of 32 in [32, 4096]")
    return int(n)


def pack_weight(w: torch.Tensor, *, head_perm: bool = True) -> torch.Tensor:
    """``w`` bf16 ``[N, K]`` (``torch.nn.Linear.weight``) -> operand images.  ``head_perm=False`` for a V
    projection (and the LoRA B that goes with it)."""
    w = _rows_bf16("weight", w)
    N, K = w.shape
    out = torch.empty(packed_bytes(N, K), dtype=torch.uint8, device=w.device)
    with torch.cuda.device(w.device):
        _lib.check(_lib.load().pkh3_pack_weight(w.data_ptr(), w.stride(0), N, K, int(head_perm), out.data_ptr(), _stream(w.device)))
    return out


def pack_rows(x: torch.Tensor) -> torch.Tensor:
    """Activations bf16 ``[S, K]`` -> operand images."""
    x = _rows_bf16("x", x)
    S, K = x.shape
    out = torch.empty(packed_bytes(S, K), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().pkh3_pack_rows(x.data_ptr(), x.stride(0), S, K, out.data_ptr(), _stream(x.device)))
    return out


def adaln_modulate(x: torch.Tensor, *, shift: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None,
                   row_index: Optional[torch.Tensor] = None, norm: str = "layer", eps: float = 1e-6) -> torch.Tensor:
    """``norm(x) * (1 + scale[row_index]) + shift[row_index]`` for ``x`` bf16 ``[S, K]``, as operand images.
    ``shift`` / ``scale``: bf16 ``[table rows, K]``; ``row_index`` int32 ``[S]`` (None: table row 0)."""
    x = _rows_bf16("x", x)
    S, K = x.shape
    stride = 0
    for name, t in (("shift", shift), ("scale", scale)):
        if t is None:
            continue
        _rows_bf16(name, t)
        _on_device(name, t, x.device)
        if t.shape[1] != K:
            raise ValueError(f"{name} must have {K} columns, got {t.shape[1]}")
        if stride and t.stride(0) != stride:
            raise ValueError("shift and scale must share one row stride")
        stride = t.stride(0)
    if shift is not None and scale is not None and shift.shape[0] != scale.shape[0]:
        raise ValueError("shift and scale must have the same number of rows")
    if row_index is not None:
        if row_index.dtype != torch.int32 or tuple(row_index.shape) != (S,) or not row_index.is_contiguous():
            raise ValueError(f"row_index must be contiguous int32 [{S}]")
        _on_device("row_index", row_index, x.device)
    out = torch.empty(packed_bytes(S, K), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().pkh3_adaln_modulate(
            x.data_ptr(), x.stride(0), S, K, NORMS[norm], float(eps),
            None if shift is None else shift.data_ptr(), None if scale is None else scale.data_ptr(), stride,
            None if row_index is None else row_index.data_ptr(), out.data_ptr(), _stream(x.device)))
    return out


def modulation_tables(temb: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], hidden_size: int,
                      chunks: int = 6):
    """The per-timestep modulation tables of a block, as the reference's patched module forms them
    (patches/0001-h3-adaln-fp32.patch:126-133): ``linear(silu(temb.float()).to(weight.dtype))`` -- the activation
    in float32 whatever dtype ``temb`` arrives in, only its result cast to the projection's dtype --, viewed as
    ``[-1, chunks * hidden_size]`` and split into ``chunks`` tables ``[rows, hidden_size]`` (six for a block:
    shift, scale, gate of the attention half and of the MLP half; two for the output norm, patch lines 150-158).
    With several modalities behind one linear layer the rows come out timestep-major: row = timestep * modalities
    + modality (see :func:`modulation_row_index`).  A few rows by a few thousand columns: host-side torch, the tables
    are then inputs of :func:`adaln_modulate` (shift, scale) and :func:`out_proj` (gate)."""
    if temb.dim() != 2 or weight.dim() != 2 or weight.shape[1] != temb.shape[1]:
        raise ValueError(f"temb [rows, E] and weight [N, E] expected, got {tuple(temb.shape)} and {tuple(weight.shape)}")
    if weight.shape[0] % (chunks * hidden_size):
        raise ValueError(f"the layer has {weight.shape[0]} outputs, not a multiple of {chunks} x {hidden_size}")
    act = torch.nn.functional.silu(temb.float()).to(weight.dtype)
    out = torch.nn.functional.linear(act, weight, bias).view(-1, chunks * hidden_size)
    return tuple(t.contiguous() for t in out.chunk(chunks, dim=-1))


def modulation_row_index(timestep_indices: torch.Tensor, modality: Optional[torch.Tensor] = None, modalities: int = 1) -> torch.Tensor:
    """int32 table row per token for :func:`adaln_modulate` / :func:`out_proj`: ``timestep_indices`` (the per-row
    index of src/pika_h3/core/wrapper.py:182-190) alone, or ``timestep_indices * modalities + modality`` when the
    tables of :func:`modulation_tables` hold one row per (timestep, modality).  Which chunk of the un-vendored
    module belongs to which modality is not visible in the reference: ``modality`` is the caller's map from
    ``token_tags`` (0 video, 1 text, 2 audio, src/pika_h3/core/geometry.py:40-42) to chunk numbers."""
    idx = timestep_indices.to(torch.int64)
    if modality is not None:
        if modality.shape != timestep_indices.shape:
            raise ValueError("modality must have one entry per row")
        if int(modality.min()) < 0 or int(modality.max()) >= modalities:
            raise ValueError(f"modality numbers must lie in [0, {modalities})")
        idx = idx * int(modalities) + modality.to(idx.device, torch.int64)
    return idx.to(torch.int32).contiguous()


@dataclass
class PackedLinear:
    """One linear layer, packed: ``y = x W^T + bias + lora_scale * (x A^T) B^T``."""

    w_img: torch.Tensor
    N: int
    K: int
    bias: Optional[torch.Tensor] = None        # fp32 [N]
    lora_a_img: Optional[torch.Tensor] = None
    lora_b_img: Optional[torch.Tensor] = None
    lora_scale: float = 0.0

    @staticmethod
    def from_weights(weight: torch.Tensor, bias: Optional[torch.Tensor] = None, *, lora_a: Optional[torch.Tensor] = None,
                     lora_b: Optional[torch.Tensor] = None, lora_scale: float = 1.0, head_perm: bool = True,
                     merge_adapter: bool = False) -> "PackedLinear":
        """``weight [N, K]``, ``lora_a [rank, K]``, ``lora_b [N, rank]`` in bf16 on the device; rank must be 128.

        ``merge_adapter``: fold the adapter into the weight once, ``W' = bf16(W + lora_scale * B A)`` formed in float32
        (any rank), and run the layer as a plain linear: no down-projection launch and no second K segment at run
        time.  The reference keeps its adapters apart (PEFT ``add_adapter``, src/pika_h3/core/loader.py:36-37), and so
        does the default here; merged, the layer rounds ``W'`` to bf16 once instead of rounding ``x A^T``, so results
        differ from the unmerged layer by bf16 rounding of the weights (what PEFT's ``merge_and_unload`` does)."""
        N, K = weight.shape
        if merge_adapter and lora_a is not None and lora_b is not None:
            if lora_a.shape[1] != K or lora_b.shape[0] != N or lora_a.shape[0] != lora_b.shape[1]:
                raise ValueError(f"adapter shapes must be A [r, {K}] and B [{N}, r], got {tuple(lora_a.shape)} and {tuple(lora_b.shape)}")
            weight = (weight.float() + float(lora_scale) * (lora_b.float() @ lora_a.float())).to(torch.bfloat16)
            lora_a = lora_b = None
        pl = PackedLinear(pack_weight(weight, head_perm=head_perm), int(N), int(K))
        if bias is not None:
            if bias.numel() != N:
                raise ValueError(f"bias has {bias.numel()} elements, the layer has {N} outputs")
            pl.bias = bias.detach().to(device=weight.device, dtype=torch.float32).contiguous().view(N)
        if (lora_a is None) != (lora_b is None):
            raise ValueError("lora_a and lora_b go together")
        if lora_a is not None:
            if tuple(lora_a.shape) != (_lib.LORA_RANK, K) or tuple(lora_b.shape) != (N, _lib.LORA_RANK):
                raise ValueError(f"adapter shapes must be A [{_lib.LORA_RANK}, {K}] and B [{N}, {_lib.LORA_RANK}], got "
                                 f"{tuple(lora_a.shape)} and {tuple(lora_b.shape)}")
            pl.lora_a_img = pack_weight(lora_a.to(torch.bfloat16), head_perm=True)
            pl.lora_b_img = pack_weight(lora_b.to(torch.bfloat16), head_perm=head_perm)
            pl.lora_scale = float(lora_scale)
        return pl

    @staticmethod
    def from_module(mod, *, head_perm: bool = True, adapter: str = "default", merge_adapter: bool = False) -> "PackedLinear":
        """From a ``torch.nn.Linear`` or a PEFT-style LoRA wrapper around one (``base_layer``, ``lora_A[adapter]``,
        ``lora_B[adapter]``, ``scaling[adapter]``: what ``add_adapter`` leaves on the targets of
        src/pika_h3/core/loader.py:36-37)."""
        base = getattr(mod, "base_layer", mod)
        kw = {}
        if hasattr(mod, "lora_A") and adapter in mod.lora_A:
            kw = dict(lora_a=mod.lora_A[adapter].weight.detach(), lora_b=mod.lora_B[adapter].weight.detach(),
                      lora_scale=float(mod.scaling[adapter]))
        return PackedLinear.from_weights(base.weight.detach().to(torch.bfloat16), getattr(base, "bias", None),
                                         head_perm=head_perm, merge_adapter=merge_adapter, **kw)

    @staticmethod
    def share_adapter_buffer(q: "PackedLinear", k: "PackedLinear", v: "PackedLinear") -> bool:
        """Lay the down-projection images (A) of the three adapters of one attention module one behind the other in a
        single buffer and point the layers at it.  ``pkh3_qkv_proj`` then runs the three down-projections as one
        target of three heads (two workgroup tiles per 256 tokens instead of three half-empty ones).  Returns False,
        and changes nothing, unless all three layers carry an adapter over the same K with the same scale."""
        imgs = [q.lora_a_img, k.lora_a_img, v.lora_a_img]
        if any(t is None for t in imgs) or not (q.K == k.K == v.K) or not (q.lora_scale == k.lora_scale == v.lora_scale):
            return False
        head = 8 * (q.K // 32) * 1024                  # bytes of the 128 rows an adapter's A really has (8 blocks of 16)
        # four heads' worth: the last workgroup tile copies a fourth, unused head's weights too
        buf = torch.zeros(4 * head, dtype=torch.uint8, device=imgs[0].device)
        for i, t in enumerate(imgs):
            buf[i * head:(i + 1) * head].copy_(t[:head])
        q.lora_a_img, k.lora_a_img, v.lora_a_img = (buf[i * head:] for i in range(3))
        return True

    def check_device(self, name: str, device) -> None:
        """Every buffer of the layer is dereferenced by kernels running on ``device``."""
        for part, t in (("w_img", self.w_img), ("bias", self.bias), ("lora_a_img", self.lora_a_img), ("lora_b_img", self.lora_b_img)):
            if t is not None:
                _on_device(f"{name}.{part}", t, device)

    def c_struct(self) -> _lib.Linear:
        s = _lib.Linear()
        s.w_img = self.w_img.data_ptr()
        s.bias = None if self.bias is None else self.bias.data_ptr()
        s.lora_a_img = None if self.lora_a_img is None else self.lora_a_img.data_ptr()
        s.lora_b_img = None if self.lora_b_img is None else self.lora_b_img.data_ptr()
        s.lora_scale = self.lora_scale
        return s


def _scratch(workspace, device, nbytes: int) -> torch.Tensor:
    """``workspace``: None (allocate), a uint8 device tensor (used when large enough) or a callable
    ``(device, nbytes) -> tensor``, as in :func:`ops.attention`."""
    if callable(workspace):
        workspace = workspace(device, nbytes)
    if workspace is None or workspace.numel() * workspace.element_size() < nbytes:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
    _on_device("workspace", workspace, device)
    return workspace


def qkv_attention(x_img: torch.Tensor, S: int, q: PackedLinear, k: PackedLinear, v: PackedLinear, *, heads: int,
                  out: Optional[torch.Tensor] = None, return_q: bool = False, workspace=None, **opts) -> torch.Tensor:
    """One self-attention call from packed activations: ``to_q / to_k / to_v`` (+ adapters) with the K side's
    norm + rotation (+ fp8 quantisation) and the K/V layout in the GEMM epilogue, then the attention kernel on
    what the GEMM left in the workspace.  ``opts`` are those of :func:`ops.fill_args` (norm weights, rope
    tables, ``fp8_qk``, ``block_mask`` ...).  Returns O ``[1, S, H, D]`` bf16 (and Q when ``return_q``); with
    ``out_images=True`` O comes back as the packed operand images :func:`out_proj` takes (``o_img=``), written
    by the attention kernel itself.  ``workspace`` as in :func:`ops.attention` (the K/V images live there)."""
    lib = _lib.load()
    dev = x_img.device
    if not x_img.is_cuda:
        raise ValueError(f"x_img must live in device memory (got {dev}); the HIP library is the only compute path")
    K = q.K
    for name, pl in (("q", q), ("k", k), ("v", v)):
        if pl.N != heads * HEAD_DIM or pl.K != K:
            raise ValueError(f"{name} projection is [{pl.N}, {pl.K}], expected [{heads * HEAD_DIM}, {K}]")
        pl.check_device(name, dev)
    if x_img.dtype != torch.uint8 or not x_img.is_contiguous() or x_img.numel() < packed_bytes(S, K):
        raise ValueError("x_img is not a packed [S, K] activation buffer")
    qt = torch.empty((1, S, heads, HEAD_DIM), dtype=torch.bfloat16, device=dev)
    if out is None:
        out = (torch.empty(packed_bytes(S, heads * HEAD_DIM), dtype=torch.uint8, device=dev) if opts.get("out_images")
               else torch.empty_like(qt))
    args, keep = fill_args(qt, None, None, out, kv_prepared=True, **opts)
    ws = _scratch(workspace, dev, workspace_bytes(args))
    args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel() * ws.element_size()
    pa = _lib.QkvArgs()
    pa.x_img, pa.S, pa.K = x_img.data_ptr(), int(S), int(K)
    pa.q, pa.k, pa.v = q.c_struct(), k.c_struct(), v.c_struct()
    lws = None
    if any(pl.lora_a_img is not None for pl in (q, k, v)):
        lws = torch.empty(packed_bytes(S, 3 * _lib.LORA_RANK), dtype=torch.uint8, device=dev)
        pa.lora_workspace, pa.lora_workspace_bytes = lws.data_ptr(), lws.numel()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream()
        _lib.check(lib.pkh3_qkv_proj(C.byref(pa), C.byref(args), C.c_void_p(stream.cuda_stream)))
        _lib.check(lib.pkh3_attn_fwd(C.byref(args), C.c_void_p(stream.cuda_stream)))
        ws.record_stream(stream)
        if lws is not None:
            lws.record_stream(stream)
    return (out, qt) if return_q else out


def out_proj(o: Optional[torch.Tensor], proj: PackedLinear, *, gate: Optional[torch.Tensor] = None,
             row_index: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None,
             o_img: Optional[torch.Tensor] = None, rows: Optional[int] = None) -> torch.Tensor:
    """``residual + gate[row_index] * (o W^T + bias + adapter)`` for the attention output ``o`` bf16 ``[S, K]``
    (e.g. ``O.view(S, H*D)``).  ``gate`` bf16 ``[table rows, N]``, ``residual`` bf16 ``[S, N]``.  Instead of ``o``
    the packed images of ``rows`` output rows can be given (``o_img``, from ``qkv_attention(..., out_images=True)``)."""
    lib = _lib.load()
    if (o is None) == (o_img is None):
        raise ValueError("give either o or o_img")
    if o_img is not None:
        if rows is None or rows < 1:
            raise ValueError("o_img needs the number of rows")
        S, K = int(rows), proj.K
        if o_img.dtype != torch.uint8 or not o_img.is_contiguous() or o_img.numel() < packed_bytes(S, K):
            raise ValueError("o_img is not a packed [rows, K] activation buffer")
        if not o_img.is_cuda:
            raise ValueError(f"o_img must live in device memory (got {o_img.device}); the HIP library is the only compute path")
        dev = o_img.device
    else:
        o = _rows_bf16("o", o)
        S, K = o.shape
        if K != proj.K:
            raise ValueError(f"o has {K} columns, the projection expects {proj.K}")
        dev = o.device
        o_img = pack_rows(o)
    proj.check_device("proj", dev)
    y = torch.empty((S, proj.N), dtype=torch.bfloat16, device=dev)
    a = _lib.OutArgs()
    a.o_img, a.S, a.K, a.N = o_img.data_ptr(), S, K, proj.N
    a.proj = proj.c_struct()
    if gate is not None:
        _rows_bf16("gate", gate)
        _on_device("gate", gate, dev)
        if gate.shape[1] != proj.N:
            raise ValueError(f"gate must have {proj.N} columns")
        a.gate, a.gate_stride = gate.data_ptr(), gate.stride(0)
        if row_index is not None:
            if row_index.dtype != torch.int32 or tuple(row_index.shape) != (S,) or not row_index.is_contiguous():
                raise ValueError(f"row_index must be contiguous int32 [{S}]")
            _on_device("row_index", row_index, dev)
            a.row_index = row_index.data_ptr()
    if residual is not None:
        _rows_bf16("residual", residual)
        _on_device("residual", residual, dev)
        if tuple(residual.shape) != (S, proj.N):
            raise ValueError(f"residual must be [{S}, {proj.N}]")
        a.residual, a.residual_stride = residual.data_ptr(), residual.stride(0)
    a.y, a.y_stride = y.data_ptr(), y.stride(0)
    lws = None
    if proj.lora_a_img is not None:
        lws = torch.empty(packed_bytes(S, _lib.LORA_RANK), dtype=torch.uint8, device=dev)
        a.lora_workspace, a.lora_workspace_bytes = lws.data_ptr(), lws.numel()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream()
        _lib.check(lib.pkh3_out_proj(C.byref(a), C.c_void_p(stream.cuda_stream)))
        o_img.record_stream(stream)
        if lws is not None:
            lws.record_stream(stream)
    return y
