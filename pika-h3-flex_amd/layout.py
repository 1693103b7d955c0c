"""Host-side geometry of the packed token sequence: which (t, h, w) position each row carries and
which 64x64 tiles a local spatio-temporal window keeps.  Pure index arithmetic on the CPU; the
results are small tensors that are built once per request geometry and reused by every layer and
denoising step (the reference caches its layout the same way, src/pika_h3/core/wrapper.py:71-78).
"""
from __future__ import annotations

import torch

TILE = 64


def video_position_ids(num_latent_frames: int, rows_h: int, rows_w: int) -> torch.Tensor:
    """``[F*rows_h*rows_w, 3]`` float64 positions of video rows.

    Video rows are frame-major, then row-major over the (h, w) patch grid
    (src/pika_h3/core/packing.py:49-54, :65-69), so row n sits at
    ``t = n // (rows_h*rows_w)``, ``h = (n % (rows_h*rows_w)) // rows_w``, ``w = n % rows_w``.
    The dtype follows the reference's position grid (src/pika_h3/core/packing.py:128).
    """
    if min(num_latent_frames, rows_h, rows_w) < 1:
        raise ValueError("num_latent_frames, rows_h, rows_w must be >= 1")
    n = torch.arange(num_latent_frames * rows_h * rows_w, dtype=torch.int64)
    per = rows_h * rows_w
    pos = torch.stack([n // per, (n % per) // rows_w, n % rows_w], dim=1)
    return pos.to(torch.float64)


def audio_position_ids(num_audio_latents: int, channels: int = 2) -> torch.Tensor:
    """``[channels*T, 3]`` float64 positions of audio rows: a 1-D grid, only the t axis varies.

    Audio rows are channel-major -- all rows of the left channel, then all of the right
    (src/pika_h3/core/packing.py:82-89) -- so row n carries latent index ``n % T`` on the t axis.
    """
    if num_audio_latents < 0 or channels < 1:
        raise ValueError("num_audio_latents must be >= 0 and channels >= 1")
    t = torch.arange(num_audio_latents, dtype=torch.float64).repeat(channels)
    pos = torch.zeros((t.numel(), 3), dtype=torch.float64)
    pos[:, 0] = t
    return pos


def local_window_tile_map(
    seq_len: int, tokens_per_frame: int, *, window_frames: int = 2, global_fraction: float = 0.10, seed: int = 0
) -> torch.Tensor:
    """bool ``[ceil(S/64), ceil(S/64)]`` map of the 64x64 tiles a local spatio-temporal window keeps.

    Tile (i, j) is kept when the latent-frame ranges covered by query tile i and key tile j are at
    most ``window_frames`` apart, or when a seeded draw selects it as one of the ``global_fraction``
    random global tiles.  The diagonal is always kept, so no query row is left without keys.
    """
    if seq_len < 1 or tokens_per_frame < 1:
        raise ValueError("seq_len and tokens_per_frame must be >= 1")
    if not 0.0 <= global_fraction <= 1.0:
        raise ValueError("global_fraction must be in [0, 1]")
    nt = (seq_len + TILE - 1) // TILE
    first = torch.arange(nt, dtype=torch.int64) * TILE
    last = torch.clamp(first + TILE - 1, max=seq_len - 1)
    lo, hi = first // tokens_per_frame, last // tokens_per_frame
    gap = torch.maximum(lo[None, :] - hi[:, None], lo[:, None] - hi[None, :])  # frames between the two ranges
    keep = gap <= window_frames
    if global_fraction > 0.0:
        g = torch.Generator().manual_seed(int(seed))
        keep |= torch.rand((nt, nt), generator=g) < global_fraction
    keep |= torch.eye(nt, dtype=torch.bool)
    return keep
