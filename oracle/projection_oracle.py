"""CPU/any-device oracle for the projections around the attention path.  TEST INFRASTRUCTURE ONLY:
imported by ``tests/`` and by ``bench.py``'s checks, never by the product.

What it restates.  The linear layers ``to_q / to_k / to_v / to_out.0`` of the attention module carry LoRA
adapters of rank 128 (target list src/pika_h3/core/loader.py:9; ``LoraConfig(r, lora_alpha, ...)`` and
``add_adapter`` at src/pika_h3/core/loader.py:36-37; loaded at src/pika_h3/pipeline.py:105-107).  PEFT, the
library that applies them, is not installed here and not vendored by the reference; its published rule for a
LoRA linear layer is ``y = x W^T + b + (lora_alpha / r) * (x A^T) B^T`` and that is what
:func:`lora_linear` computes in float64.  The AdaLN modulation is the visible hunk of the reference's patch to
its diffusers pin (patches/0001-h3-adaln-fp32.patch:34-40): ``norm(x) * (1 + scale.index_select(0, idx)) +
shift.index_select(0, idx)`` with ``idx = timestep_indices``; which norm the un-vendored module applies is not
visible (a switch: LayerNorm without affine parameters, or RMSNorm without weight).

Pinning status (tests/test_projection_oracle.py):
  lora_linear     pinned: torch.nn.functional.linear for the base term, equality with the merged weight
                  W + s B A (the identity PEFT's merge relies on), zero adapter, rank-one closed form
  adaln_modulate  pinned: torch.nn.functional.layer_norm / rms_norm, index_select, zero-modulation identity,
                  per-row constant closed form
  modulation_tables  pinned: torch.nn.functional.silu in float32 + torch.nn.functional.linear; one rounding of
                  the activation against a two-rounding evaluation, row order of the view checked against an
                  explicit (timestep, modality) loop
  attention_block composition of the above with attention_oracle.reference_layer; pinned by its parts and
                  by an explicit per-row, per-head loop on a tiny case
"""
from __future__ import annotations

from typing import Optional

import torch

from . import attention_oracle as AO


def lora_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, *,
                lora_a: Optional[torch.Tensor] = None, lora_b: Optional[torch.Tensor] = None,
                lora_scale: float = 1.0) -> torch.Tensor:
    """``x [.., K]`` -> ``[.., N]`` in float64: base linear layer plus the scaled low-rank update."""
    x64 = x.to(torch.float64)
    y = x64 @ weight.to(device=x.device, dtype=torch.float64).t()
    if bias is not None:
        y = y + bias.to(device=x.device, dtype=torch.float64)
    if lora_a is not None:
        down = x64 @ lora_a.to(device=x.device, dtype=torch.float64).t()
        y = y + float(lora_scale) * (down @ lora_b.to(device=x.device, dtype=torch.float64).t())
    return y


def modulation_tables(temb: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], hidden_size: int,
                      chunks: int = 6):
    """patches/0001-h3-adaln-fp32.patch:126-133 restated: SiLU in float32 (``x * sigmoid(x)``, written out), the
    result rounded to the projection's dtype, the linear layer in float64 on those rounded values, rows viewed as
    ``[-1, chunks * hidden_size]`` and split.  Returns ``chunks`` float64 tables."""
    t32 = temb.to(torch.float32)
    act = (t32 * (1.0 / (1.0 + torch.exp(-t32)))).to(weight.dtype)
    out = act.to(torch.float64) @ weight.to(torch.float64).t()
    if bias is not None:
        out = out + bias.to(torch.float64)
    return tuple(out.view(-1, chunks * hidden_size).chunk(chunks, dim=-1))


def adaln_modulate(x: torch.Tensor, *, shift: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None,
                   row_index: Optional[torch.Tensor] = None, norm: str = "layer", eps: float = 1e-6) -> torch.Tensor:
    """``norm(x) * (1 + scale[row_index]) + shift[row_index]`` over rows ``x [S, K]``, float64."""
    x64 = x.to(torch.float64)
    if norm == "layer":
        mu = x64.mean(dim=-1, keepdim=True)
        var = ((x64 - mu) ** 2).mean(dim=-1, keepdim=True)
        y = (x64 - mu) * torch.rsqrt(var + eps)
    elif norm == "rms":
        y = x64 * torch.rsqrt((x64 * x64).mean(dim=-1, keepdim=True) + eps)
    elif norm == "none":
        y = x64
    else:
        raise ValueError(f"unknown norm {norm!r}")
    idx = torch.zeros(x.shape[0], dtype=torch.long, device=x.device) if row_index is None else row_index.to(device=x.device, dtype=torch.long)
    if scale is not None:
        y = y * (1.0 + scale.to(device=x.device, dtype=torch.float64).index_select(0, idx))
    if shift is not None:
        y = y + shift.to(device=x.device, dtype=torch.float64).index_select(0, idx)
    return y


def attention_block(x: torch.Tensor, lin: dict, *, heads: int, shift=None, scale=None, gate=None, row_index=None,
                    norm: str = "layer", eps: float = 1e-6, residual: bool = True, round_bf16: bool = True,
                    **attn_opts) -> dict:
    """The attention half of one DiT block on rows ``x [S, C]``: modulate -> to_q/to_k/to_v (+LoRA) ->
    attention (``attn_opts`` as for ``attention_oracle.reference_layer``) -> to_out.0 (+LoRA) -> gated
    residual.  ``lin`` maps ``"q" | "k" | "v" | "out"`` to keyword dicts for :func:`lora_linear`.
    ``round_bf16`` rounds the tensors the product stores in bf16 between its kernels (modulated rows,
    Q/K/V, attention output), so that the comparison isolates arithmetic from storage precision.
    Returns every intermediate."""
    def rb(t):
        return t.to(torch.bfloat16).to(torch.float64) if round_bf16 else t

    S, C = x.shape
    xm = rb(adaln_modulate(x, shift=shift, scale=scale, row_index=row_index, norm=norm, eps=eps))
    q, k, v = (rb(lora_linear(xm, **lin[n])).view(1, S, heads, -1) for n in ("q", "k", "v"))
    o = rb(AO.reference_layer(q, k, v, **attn_opts)).view(S, -1)
    y = lora_linear(o, **lin["out"])
    if gate is not None:
        idx = torch.zeros(S, dtype=torch.long, device=x.device) if row_index is None else row_index.to(device=x.device, dtype=torch.long)
        y = y * gate.to(device=x.device, dtype=torch.float64).index_select(0, idx)
    if residual:
        y = y + x.to(torch.float64)
    return dict(xm=xm, q=q, k=k, v=v, o=o, y=y)
