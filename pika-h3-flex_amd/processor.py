"""Attention processor for the H3 DiT blocks, in the shape diffusers' processor mechanism calls
(``processor(attn, hidden_states, ...)``).

The reference never builds attention itself: it loads ``diffusers.MiniMaxH3Transformer3DModel``
(src/pika_h3/core/loader.py:11-18) whose attention modules own ``to_q / to_k / to_v / to_out.0``
(the LoRA target list, src/pika_h3/core/loader.py:9) and calls the model with the packed-sequence
tensors of src/pika_h3/core/wrapper.py:192-204 (``position_ids [S,3]`` float64 among them).  This
processor is what gets attached to those modules: it runs the module's own projections (torch
GEMMs, LoRA included), hands ``[B, S, H, D]`` strided views to libpkh3attn.so for
QK-RMSNorm -> RoPE -> softmax(QK^T)V, and applies ``to_out``.

Everything the pinned diffusers source alone could settle is an explicit constructor argument:
RoPE pairing (``rope_mode``), axis split and theta, and where the norm weights are read from.
"""
from __future__ import annotations

from typing import Dict, Hashable, Optional, Tuple

import torch

from . import _lib
from .ops import BlockMask, PreparedKV, attention, attention_prepared, fp8_mode, prepare_kv, rope_tables
from .projections import PackedLinear, adaln_modulate, out_proj, pack_rows, qkv_attention


ADDITIVE_DROP_THRESHOLD = -1e3  # additive float masks: entries at or below this drop the key


def _norm_weight(mod, dim: int, device) -> Optional[torch.Tensor]:
    """fp32 weight of an RMSNorm-like module (``None`` module = no norm; no ``weight`` = ones)."""
    if mod is None:
        return None
    w = getattr(mod, "weight", None)
    if w is None:
        return torch.ones(dim, dtype=torch.float32, device=device)
    if w.numel() != dim:
        raise ValueError(f"QK-norm weight has {w.numel()} elements; only per-head norm over D={dim} is supported")
    return w.detach().to(device=device, dtype=torch.float32).contiguous()


def key_padding_mask(attention_mask: Optional[torch.Tensor], batch: int, keys: int) -> Optional[torch.Tensor]:
    """The forms diffusers modules hand a key-padding mask around in, as the bool ``[B, Sk]`` (True = attend) the
    library takes: bool or integer ``[B, Sk]``; additive float masks (0 = attend, -inf or a number <= -1000 = drop; other values are refused) of
    shape ``[B, Sk]``, ``[B, 1, Sk]`` or ``[B, 1, 1, Sk]``.  A mask that differs between the queries or the heads of
    a batch entry is not a key-padding mask and is refused."""
    if attention_mask is None:
        return None
    m = attention_mask
    if m.dim() > 2:
        if any(d != 1 for d in m.shape[1:-1]):
            raise ValueError(f"attention_mask {tuple(m.shape)} varies over queries or heads; only key-padding masks "
                             f"[B, Sk] (or broadcast forms of them) are supported")
        m = m.reshape(m.shape[0], m.shape[-1])
    if m.dim() != 2 or m.shape[-1] != keys or m.shape[0] not in (1, batch):
        raise ValueError(f"attention_mask must be [B, Sk] = [{batch}, {keys}] or a broadcast form, got {tuple(attention_mask.shape)}")
    if m.shape[0] != batch:
        m = m.expand(batch, keys)
    if m.is_floating_point():
        # additive form: 0 keeps a key, -inf / a large negative number drops it.  Anything else -- a {0, 1} keep-mask
        # cast to float, a soft bias -- is not a key-padding mask; turning it into keep/drop silently would attend
        # padding keys or drop a bias, so it is refused (one reduction and one host read per distinct mask tensor)
        keep = m == 0
        if not bool((keep | (m <= ADDITIVE_DROP_THRESHOLD)).all()):
            raise ValueError("floating-point attention_mask must be additive with entries 0 (attend) or <= "
                             f"{ADDITIVE_DROP_THRESHOLD:g} (drop); got other values (a 0/1 keep-mask must be bool or integer, "
                             "a soft additive bias is not supported)")
        m = keep
    elif m.dtype != torch.bool:
        m = m != 0
    return m


class PikaH3AttnProcessor:
    """Drop-in attention processor backed by the gfx950 HIP kernels.

    ``attn`` must expose ``to_q, to_k, to_v, to_out`` (``to_out[0]`` is the projection), ``heads``
    and optionally ``norm_q / norm_k`` (RMSNorm over the head dim, ``eps`` attribute honoured).
    """

    def __init__(
        self,
        *,
        rope_mode: int = _lib.ROPE_INTERLEAVED,
        rope_axes_dims: Tuple[int, int, int] = (32, 48, 48),
        rope_theta: float = 10000.0,
        norm_eps: float = 1e-6,
        fp8_qk=False,
        fused_projections: bool = False,
        lora_adapter: str = "default",
        merge_adapters: bool = False,
        cache_cross_kv: bool = False,
        cross_kv_cache_bytes: int = 1 << 30,
    ):
        self.rope_mode = int(rope_mode)
        self.rope_axes_dims = tuple(int(x) for x in rope_axes_dims)
        self.rope_theta = float(rope_theta)
        self.norm_eps = float(norm_eps)
        self.fp8_qk = fp8_mode(fp8_qk)  # False, True or "pow2"
        # self-attention of one document through the library's own projection GEMMs (LoRA as a second K segment,
        # K/V written by the GEMM epilogue in the attention kernel's layout) instead of the module's torch GEMMs
        self.fused_projections = bool(fused_projections)
        self.lora_adapter = str(lora_adapter)
        # fused projections only: fold each adapter into its weight when the weights are packed (one bf16 rounding of
        # W + scale * B A) instead of applying it at run time as the reference's PEFT layers do; off by default
        self.merge_adapters = bool(merge_adapters)
        # cross-attention: the text keys and values of a block are the same in every denoising step of a clip (the
        # model runs six times on one prompt, src/pika_h3/pipeline.py:13); with this switch a block projects and
        # prepares them once per (module, encoder_hidden_states tensor, mask tensor) and later steps reuse them
        self.cache_cross_kv = bool(cache_cross_kv)
        self.cross_kv_cache_bytes = int(cross_kv_cache_bytes)  # prepared workspaces kept at most (oldest dropped first)
        self._cross_kv: Dict[Hashable, Tuple[tuple, PreparedKV]] = {}
        self._packed: Dict[int, Tuple[object, Dict[str, PackedLinear]]] = {}
        # position grids are constant across layers and denoising steps: one table per grid
        self._rope_cache: Dict[Hashable, Tuple[Optional[torch.Tensor], Tuple[torch.Tensor, torch.Tensor]]] = {}
        # one scratch buffer per (device, stream), grown on demand and reused by every layer call on that stream
        self._workspaces: Dict[Tuple[str, int], torch.Tensor] = {}

    def _tables(self, position_ids: torch.Tensor, rope_key: Optional[Hashable] = None):
        """cos/sin tables of a position grid, cached.  With ``rope_key`` (e.g. the caller's geometry key) the cache
        is keyed by it and the grid's identity does not matter.  Without, the key is the grid tensor itself --
        address, length, device and in-place version counter -- and the entry keeps the tensor alive, so its
        address cannot be handed to another grid while the entry exists."""
        if rope_key is not None:
            key = ("key", rope_key, position_ids.shape[0], str(position_ids.device))
        else:
            key = ("tensor", position_ids.data_ptr(), position_ids.shape[0], str(position_ids.device),
                   position_ids._version)
        hit = self._rope_cache.get(key)
        if hit is None:
            if len(self._rope_cache) >= 8:
                self._rope_cache.pop(next(iter(self._rope_cache)))
            tabs = rope_tables(position_ids, self.rope_axes_dims, self.rope_theta)
            hit = (position_ids if rope_key is None else None, tabs)
            self._rope_cache[key] = hit
        return hit[1]

    def _workspace(self, device, nbytes: int) -> torch.Tensor:
        with torch.cuda.device(device):
            key = (str(device), int(torch.cuda.current_stream().cuda_stream))
        ws = self._workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._workspaces[key] = ws
        return ws

    def packed_weights(self, attn) -> Dict[str, PackedLinear]:
        """The module's four projections as operand images, packed on first use and kept with the module (weights
        are static at inference; call :meth:`forget` after changing them)."""
        hit = self._packed.get(id(attn))
        if hit is None or hit[0] is not attn:
            packed = {
                "q": PackedLinear.from_module(attn.to_q, adapter=self.lora_adapter, merge_adapter=self.merge_adapters),
                "k": PackedLinear.from_module(attn.to_k, adapter=self.lora_adapter, merge_adapter=self.merge_adapters),
                "v": PackedLinear.from_module(attn.to_v, head_perm=False, adapter=self.lora_adapter, merge_adapter=self.merge_adapters),
                "out": PackedLinear.from_module(attn.to_out[0], adapter=self.lora_adapter, merge_adapter=self.merge_adapters),
            }
            PackedLinear.share_adapter_buffer(packed["q"], packed["k"], packed["v"])
            hit = (attn, packed)
            self._packed[id(attn)] = hit
        return hit[1]

    def forget(self, attn=None) -> None:
        """Drop packed weights and prepared cross-attention keys (of one module, or all)."""
        if attn is None:
            self._packed.clear()
            self._cross_kv.clear()
        else:
            self._packed.pop(id(attn), None)
            for key in [k for k in self._cross_kv if k[0] == id(attn)]:
                del self._cross_kv[key]

    @staticmethod
    def _weights_state(attn) -> tuple:
        """Identity and in-place version of every parameter the prepared keys depend on: ``to_k`` / ``to_v`` (adapter
        weights of a LoRA wrapper included: they are sub-module parameters) and the K-side norm."""
        state = []
        for mod in (attn.to_k, attn.to_v, getattr(attn, "norm_k", None)):
            if mod is not None and hasattr(mod, "parameters"):
                state += [(id(p_), p_._version) for p_ in mod.parameters()]
        return tuple(state)

    def _prepared_cross_kv(self, attn, enc: torch.Tensor, mask: Optional[torch.Tensor], k_opts: dict, H: int,
                           cache_key: Optional[Hashable] = None) -> PreparedKV:
        """Prepared K/V of ``attn``'s cross-attention over ``enc``.  With ``cache_key`` (the caller's name for the
        prompt, e.g. a request id) the entry is found by (module, key) whatever tensors carry the text states in this
        step -- a model that re-projects or re-concatenates them per forward still hits.  Without it the entry is
        keyed by the identity and in-place version of the two tensors, which it keeps alive (so their addresses
        cannot be reused).  Either way the key also holds the identity and version of the module's K-side weights
        (adapters included), so training steps or a swapped adapter prepare the keys again.  The cache is bounded by
        the bytes of its workspaces (``cross_kv_cache_bytes``), oldest entries dropped first."""
        common = (float(k_opts["norm_eps"]), str(k_opts["fp8_qk"]), tuple(enc.shape), str(enc.device), self._weights_state(attn))
        if cache_key is not None:
            key = (id(attn), "key", cache_key) + common
        else:
            key = (id(attn), "tensor", enc.data_ptr(), enc._version,
                   None if mask is None else (mask.data_ptr(), mask._version)) + common
        hit = self._cross_kv.get(key)
        if hit is not None and hit[0][0] is attn and (cache_key is not None or (hit[0][1] is enc and hit[0][2] is mask)):
            return hit[1]
        B, Sk, _ = enc.shape
        k = attn.to_k(enc).view(B, Sk, H, -1)
        v = attn.to_v(enc).view(B, Sk, H, -1)
        if k.dtype != torch.bfloat16:
            k, v = k.to(torch.bfloat16), v.to(torch.bfloat16)
        kv = prepare_kv(k, v, **k_opts)
        self._cross_kv.pop(key, None)
        # entries found by key do not need the tensors; entries found by tensor identity keep them alive
        self._cross_kv[key] = ((attn, None, None) if cache_key is not None else (attn, enc, mask), kv)
        total = sum(e[1].workspace.numel() for e in self._cross_kv.values())
        while total > self.cross_kv_cache_bytes and len(self._cross_kv) > 1:
            oldest = next(iter(self._cross_kv))
            total -= self._cross_kv.pop(oldest)[1].workspace.numel()
        return kv

    def __call__(
        self,
        attn,
        hidden_states: torch.Tensor,
        encoder_hidden_states: Optional[torch.Tensor] = None,
        attention_mask: Optional[torch.Tensor] = None,
        *,
        position_ids: Optional[torch.Tensor] = None,
        rope_cos_sin: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
        block_mask: Optional[BlockMask] = None,
        fp8_qk=None,
        rope_key: Optional[Hashable] = None,
        adaln: Optional[dict] = None,
        gate: Optional[torch.Tensor] = None,
        gate_index: Optional[torch.Tensor] = None,
        residual: Optional[torch.Tensor] = None,
        cross_kv_key: Optional[Hashable] = None,
    ) -> torch.Tensor:
        """``hidden_states [B, S, H*D]`` -> ``[B, S, H*D]``.

        Self-attention when ``encoder_hidden_states`` is None, else cross-attention with K/V from
        ``encoder_hidden_states [B, Sk, C]`` and ``attention_mask`` a key-padding mask: bool
        ``[B, Sk]`` (True = attend) or one of the forms :func:`key_padding_mask` converts.  RoPE applies to self-attention only, from ``position_ids
        [S, 3]`` (or precomputed ``rope_cos_sin`` fp32 ``[S, D/2]`` tables); ``rope_key`` names the grid for the
        table cache (see :meth:`_tables`).  The softmax scale is ``attn.scale`` when the module has one, else
        ``1/sqrt(D)``.  fp8 QK^T is not defined together with a key mask: such a call runs in bf16.

        With ``fused_projections`` (self-attention, B = 1, no mask) the projections run in the library too, and the
        block's surroundings can ride along: ``adaln = dict(shift=, scale=, row_index=, norm=, eps=)`` applies
        ``norm(x) * (1 + scale[row_index]) + shift[row_index]`` to ``hidden_states`` before ``to_q/to_k/to_v``
        (patches/0001-h3-adaln-fp32.patch:34-40), and ``gate`` (bf16 ``[rows, C]``, gathered by ``gate_index``,
        int32 ``[S]``) and ``residual`` (``[B, S, C]``) make the result ``residual + gate * to_out(...)``.
        Without ``fused_projections`` those three arguments are rejected.

        ``cross_kv_key`` (with ``cache_cross_kv``): the caller's name for the prompt whose text states this call
        carries; prepared keys are then found by (module, key) instead of by tensor identity, see
        :meth:`_prepared_cross_kv`.
        """
        if hidden_states.dim() != 3:
            raise ValueError(f"hidden_states must be [B, S, C], got {tuple(hidden_states.shape)}")
        B, S, _ = hidden_states.shape
        H = int(attn.heads)
        mask_given = attention_mask  # the caller's tensor: what the cross-attention key cache recognises
        if attention_mask is not None:
            keys = S if encoder_hidden_states is None else encoder_hidden_states.shape[1]
            same = attention_mask.dtype == torch.bool and tuple(attention_mask.shape) == (B, keys)
            attention_mask = attention_mask if same else key_padding_mask(attention_mask, B, keys)
        fused = self.fused_projections and encoder_hidden_states is None and attention_mask is None and B == 1
        if not fused and (adaln is not None or gate is not None or residual is not None):
            raise ValueError("adaln / gate / residual need fused_projections, self-attention, B = 1 and no mask")
        if fused:
            return self._fused(attn, hidden_states, position_ids=position_ids, rope_cos_sin=rope_cos_sin, block_mask=block_mask,
                               fp8_qk=fp8_qk, rope_key=rope_key, adaln=adaln, gate=gate, gate_index=gate_index, residual=residual)
        qn, kn = getattr(attn, "norm_q", None), getattr(attn, "norm_k", None)
        eps = getattr(qn, "eps", None)
        eps = self.norm_eps if eps is None else float(eps)
        scale = getattr(attn, "scale", None)
        use_fp8 = (self.fp8_qk if fp8_qk is None else fp8_mode(fp8_qk)) if attention_mask is None else False
        q = attn.to_q(hidden_states)
        D = q.shape[-1] // H
        # [B, S, H*D] -> [B, S, H, D] views: no transpose copy, the kernels take the strides
        q = q.view(B, S, H, D)
        if q.dtype != torch.bfloat16:
            q = q.to(torch.bfloat16)
        if encoder_hidden_states is not None and self.cache_cross_kv and block_mask is None:
            k_opts = dict(k_norm_weight=_norm_weight(kn, D, q.device), norm_eps=eps, fp8_qk=use_fp8)
            if attention_mask is not None:
                k_opts.update(key_mask=attention_mask)
            kv = self._prepared_cross_kv(attn, encoder_hidden_states, mask_given, k_opts, H, cross_kv_key)
            out = attention_prepared(q, kv, q_norm_weight=_norm_weight(qn, D, q.device),
                                     softmax_scale=None if scale is None else float(scale))
            out = attn.to_out[0](out.view(B, S, H * D).to(hidden_states.dtype))
            return attn.to_out[1](out) if len(attn.to_out) > 1 else out
        kv_src = hidden_states if encoder_hidden_states is None else encoder_hidden_states
        k = attn.to_k(kv_src).view(B, kv_src.shape[1], H, D)
        v = attn.to_v(kv_src).view(B, kv_src.shape[1], H, D)
        if k.dtype != torch.bfloat16:
            k, v = k.to(torch.bfloat16), v.to(torch.bfloat16)
        opts = dict(
            q_norm_weight=_norm_weight(qn, D, q.device),
            k_norm_weight=_norm_weight(kn, D, q.device),
            norm_eps=eps,
            fp8_qk=use_fp8,
            block_mask=block_mask,
            softmax_scale=None if scale is None else float(scale),
        )
        if encoder_hidden_states is None:
            if rope_cos_sin is None and position_ids is not None:
                rope_cos_sin = self._tables(position_ids, rope_key)
            if rope_cos_sin is not None:
                opts.update(rope_mode=self.rope_mode, rope_q=rope_cos_sin, rope_k=rope_cos_sin)
            if attention_mask is not None:
                opts.update(key_mask=attention_mask)
        else:
            if attention_mask is not None:
                opts.update(key_mask=attention_mask)

        out = attention(q, k, v, workspace=self._workspace, **opts)
        out = out.view(B, S, H * D).to(hidden_states.dtype)
        out = attn.to_out[0](out)
        if len(attn.to_out) > 1:
            out = attn.to_out[1](out)
        return out

    def _fused(self, attn, hidden_states, *, position_ids, rope_cos_sin, block_mask, fp8_qk, rope_key, adaln, gate, gate_index,
               residual) -> torch.Tensor:
        _, S, C = hidden_states.shape
        H = int(attn.heads)
        if C != H * 128:
            raise ValueError(f"hidden size {C} is not heads x 128")
        x = hidden_states[0]
        if x.dtype != torch.bfloat16:
            x = x.to(torch.bfloat16)
        packed = self.packed_weights(attn)
        x_img = pack_rows(x) if adaln is None else adaln_modulate(x, **adaln)
        qn, kn = getattr(attn, "norm_q", None), getattr(attn, "norm_k", None)
        eps = getattr(qn, "eps", None)
        scale = getattr(attn, "scale", None)
        opts = dict(
            q_norm_weight=_norm_weight(qn, 128, x.device), k_norm_weight=_norm_weight(kn, 128, x.device),
            norm_eps=self.norm_eps if eps is None else float(eps),
            fp8_qk=self.fp8_qk if fp8_qk is None else fp8_mode(fp8_qk), block_mask=block_mask,
            softmax_scale=None if scale is None else float(scale),
        )
        if rope_cos_sin is None and position_ids is not None:
            rope_cos_sin = self._tables(position_ids, rope_key)
        if rope_cos_sin is not None:
            opts.update(rope_mode=self.rope_mode, rope_q=rope_cos_sin, rope_k=rope_cos_sin)
        # the attention kernel writes its output as the operand images of the out-projection: no packing pass
        o_img = qkv_attention(x_img, S, packed["q"], packed["k"], packed["v"], heads=H, out_images=True,
                              workspace=self._workspace, **opts)
        res = None
        if residual is not None:
            res = residual[0] if residual.dim() == 3 else residual
            if res.dtype != torch.bfloat16:
                res = res.to(torch.bfloat16)
        y = out_proj(None, packed["out"], gate=gate, row_index=gate_index, residual=res, o_img=o_img, rows=S)
        return y.view(1, S, C).to(hidden_states.dtype)
