"""Seeded synthetic inputs for the benchmark configurations (no dataset, no checkpoint):
hidden states ~ N(0,1) projected by random-init Wq/Wk/Wv (std 0.02), positions from the video /
audio grids.  Random numbers are drawn on the CPU from ``torch.Generator().manual_seed(seed)`` and
then moved, so the same seed gives the same inputs on every machine; the projections run on the
target device in bf16.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .layout import audio_position_ids, video_position_ids

HEAD_DIM = 128


@dataclass
class AttnInputs:
    q: torch.Tensor                    # [1, Sq, H, D] bf16 (views into a [1, S, H*D] projection)
    k: torch.Tensor                    # [1, Sk, H, D]
    v: torch.Tensor
    position_ids: Optional[torch.Tensor]  # [Sq, 3] float64 or None (cross-attention)
    key_mask: Optional[torch.Tensor]   # [1, Sk] bool or None
    name: str
    tokens_per_frame: int = 0

    @property
    def flops(self) -> float:
        """4*Sq*Sk*D*H with Sk counted over the keys that are attended."""
        sk = self.k.shape[1] if self.key_mask is None else int(self.key_mask.sum())
        return 4.0 * self.q.shape[1] * sk * HEAD_DIM * self.q.shape[2]


def _project(x: torch.Tensor, w: torch.Tensor, heads: int) -> torch.Tensor:
    y = torch.matmul(x, w.t())
    return y.view(1, x.shape[0], heads, HEAD_DIM)


def _randn(shape, gen, device, std=1.0, chunk_rows=16384):
    """CPU-seeded normal tensor delivered as bf16 on ``device`` without holding all of it in fp32."""
    rows = shape[0]
    out = torch.empty(shape, dtype=torch.bfloat16, device=device)
    for r0 in range(0, rows, chunk_rows):
        r1 = min(rows, r0 + chunk_rows)
        blk = torch.randn((r1 - r0,) + tuple(shape[1:]), generator=gen, dtype=torch.float32)
        if std != 1.0:
            blk *= std
        out[r0:r1] = blk.to(torch.bfloat16).to(device)
    return out


def self_attention_inputs(
    *, frames: int, rows_h: int, rows_w: int, heads: int = 24, audio_latents: int = 0, seed: int = 0,
    device="cuda", name: str = "self",
) -> AttnInputs:
    """Joint video(+audio) self-attention layer inputs.  Video rows first, audio rows after them."""
    gen = torch.Generator().manual_seed(int(seed))
    hidden = heads * HEAD_DIM
    pos = video_position_ids(frames, rows_h, rows_w)
    if audio_latents:
        pos = torch.cat([pos, audio_position_ids(audio_latents)], dim=0)
    S = pos.shape[0]
    x = _randn((S, hidden), gen, device)
    ws = [_randn((hidden, hidden), gen, device, std=0.02) for _ in range(3)]
    q, k, v = (_project(x, w, heads) for w in ws)
    return AttnInputs(q, k, v, pos.to(device), None, name, tokens_per_frame=rows_h * rows_w)


def cross_attention_inputs(
    *, q_tokens: int, text_tokens: int = 512, valid_range=(60, 480), heads: int = 24, seed: int = 0,
    device="cuda", name: str = "cross",
) -> AttnInputs:
    """Text cross-attention: Q from ``q_tokens`` rows, K/V from ``text_tokens`` rows of which a seeded
    number in ``valid_range`` (inclusive) is valid and the rest is padding."""
    gen = torch.Generator().manual_seed(int(seed))
    hidden = heads * HEAD_DIM
    x = _randn((q_tokens, hidden), gen, device)
    t = _randn((text_tokens, hidden), gen, device)
    ws = [_randn((hidden, hidden), gen, device, std=0.02) for _ in range(3)]
    lo, hi = valid_range
    n_valid = int(torch.randint(int(lo), int(hi) + 1, (1,), generator=gen))
    n_valid = max(1, min(n_valid, text_tokens))
    mask = (torch.arange(text_tokens) < n_valid)[None, :].to(device)
    q = _project(x, ws[0], heads)
    k = _project(t, ws[1], heads)
    v = _project(t, ws[2], heads)
    return AttnInputs(q, k, v, None, mask, name)


def plumbing_inputs(*, heads: int = 4, seq: int = 1024, seed: int = 0, device="cuda") -> AttnInputs:
    """B=1, H=4, S=1024, D=128 with Q, K, V ~ N(0,1) straight from the seed (no projection)."""
    gen = torch.Generator().manual_seed(int(seed))
    q, k, v = (_randn((seq, heads * HEAD_DIM), gen, device).view(1, seq, heads, HEAD_DIM) for _ in range(3))
    return AttnInputs(q, k, v, None, None, "plumbing")


@dataclass
class BlockInputs:
    """The attention half of one DiT block at a self-attention configuration: hidden states, the four projections
    with their LoRA adapters (rank 128 on ``to_q, to_k, to_v, to_out.0``, src/pika_h3/core/loader.py:9), AdaLN
    tables gathered per row by ``row_index`` (three timestep groups), and the position grid."""

    x: torch.Tensor                    # [S, C] bf16
    linears: dict                      # "q" | "k" | "v" | "out" -> dict(weight, bias, lora_a, lora_b, lora_scale)
    shift: torch.Tensor                # [T, C] bf16
    scale: torch.Tensor
    gate: torch.Tensor
    row_index: torch.Tensor            # [S] int32
    position_ids: torch.Tensor         # [S, 3] float64
    heads: int
    name: str

    @property
    def attention_flops(self) -> float:
        S = self.x.shape[0]
        return 4.0 * S * S * HEAD_DIM * self.heads

    @property
    def projection_flops(self) -> float:
        """2*S*C*N over the four projections plus the adapters' two rank-128 products each."""
        S, C = self.x.shape
        r = next(iter(self.linears.values()))["lora_a"].shape[0]
        return 4 * (2.0 * S * C * C) + 4 * (2.0 * S * C * r + 2.0 * S * r * C)


def block_inputs(*, frames: int, rows_h: int, rows_w: int, heads: int = 24, lora_rank: int = 128, lora_alpha: int = 64,
                 groups: int = 3, seed: int = 0, device="cuda", name: str = "block") -> BlockInputs:
    gen = torch.Generator().manual_seed(int(seed))
    C = heads * HEAD_DIM
    pos = video_position_ids(frames, rows_h, rows_w)
    S = pos.shape[0]
    x = _randn((S, C), gen, device)
    lin = {}
    for n in ("q", "k", "v", "out"):
        lin[n] = dict(
            weight=_randn((C, C), gen, device, std=0.02),
            bias=(torch.randn((C,), generator=gen) * 0.02).to(device),
            lora_a=_randn((lora_rank, C), gen, device, std=0.02),
            lora_b=_randn((C, lora_rank), gen, device, std=0.02),
            lora_scale=float(lora_alpha) / float(lora_rank),
        )
    shift, scale, gate = (_randn((groups, C), gen, device, std=0.2) for _ in range(3))
    row_index = (torch.arange(S) * groups // S).to(torch.int32).to(device)
    return BlockInputs(x, lin, shift, scale, gate, row_index, pos.to(device), heads, name)


# The benchmark configurations by name.
CONFIGS = {
    "plumbing": dict(kind="plumbing", heads=4, seq=1024),
    "480p": dict(kind="self", frames=31, rows_h=30, rows_w=52),
    "768p": dict(kind="self", frames=31, rows_h=48, rows_w=84),
    "joint": dict(kind="self", frames=31, rows_h=30, rows_w=52, audio_latents=640),
    "cross": dict(kind="cross", q_tokens=49640, text_tokens=512),
}


def make(name: str, *, seed: int = 0, device="cuda") -> AttnInputs:
    cfg = dict(CONFIGS[name])
    kind = cfg.pop("kind")
    if kind == "plumbing":
        return plumbing_inputs(seed=seed, device=device, **cfg)
    if kind == "self":
        return self_attention_inputs(seed=seed, device=device, name=name, **cfg)
    return cross_attention_inputs(seed=seed, device=device, name=name, **cfg)
