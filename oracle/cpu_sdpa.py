"""CPU baseline for the benchmark: the path a PyTorch user gets on the host without this library --
RMSNorm + rotary embedding in torch ops, then the library routine
``torch.nn.functional.scaled_dot_product_attention`` (non-causal).  TEST/BENCH INFRASTRUCTURE ONLY:
imported by ``bench.py``'s ``cpu_baseline`` leg and by tests, never by the product.

This is the route the reference's model takes on a machine without a GPU kernel: its attention runs
inside ``diffusers.MiniMaxH3Transformer3DModel`` (src/pika_h3/core/loader.py:11-18, called at
src/pika_h3/core/wrapper.py:248) on whatever kernel torch dispatches (README.md:183).
"""
from __future__ import annotations

import time
from typing import Optional

import torch
import torch.nn.functional as F


def _rope_interleaved(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    c, s = cos[None, :, None, :], sin[None, :, None, :]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    return torch.stack([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1).flatten(-2)


def sdpa_layer(q, k, v, *, q_norm_weight=None, k_norm_weight=None, eps=1e-6, rope_q=None, rope_k=None,
               key_mask=None, dtype=torch.float32):
    """``[B, S, H, D]`` inputs -> ``[B, Sq, H, D]``; norm/rope in fp32, SDPA in ``dtype``."""
    qf, kf = q.float(), k.float()
    if q_norm_weight is not None:
        qf = F.rms_norm(qf, (qf.shape[-1],), q_norm_weight.float(), eps)
    if k_norm_weight is not None:
        kf = F.rms_norm(kf, (kf.shape[-1],), k_norm_weight.float(), eps)
    if rope_q is not None:
        rk = rope_q if rope_k is None else rope_k
        qf = _rope_interleaved(qf, rope_q[0].float(), rope_q[1].float())
        kf = _rope_interleaved(kf, rk[0].float(), rk[1].float())
    mask = None if key_mask is None else key_mask.to(torch.bool)[:, None, None, :]
    o = F.scaled_dot_product_attention(
        qf.to(dtype).transpose(1, 2), kf.to(dtype).transpose(1, 2), v.to(dtype).transpose(1, 2), attn_mask=mask
    )
    return o.transpose(1, 2)


def time_cpu_baseline(q, k, v, *, sample_rows: int, threads: Optional[int] = None, repeats: int = 1, **opts):
    """Time :func:`sdpa_layer` on the first ``sample_rows`` query rows against the full K/V on the host.
    Returns (seconds per call, threads used)."""
    if threads:
        torch.set_num_threads(int(threads))
    qs = q[:, :sample_rows].cpu()
    kc, vc = k.cpu(), v.cpu()
    if opts.get("rope_q") is not None:
        rq = tuple(t.cpu() for t in opts["rope_q"])
        opts = dict(opts, rope_q=(rq[0][:sample_rows], rq[1][:sample_rows]), rope_k=rq)
    for key in ("q_norm_weight", "k_norm_weight"):
        if opts.get(key) is not None:
            opts[key] = opts[key].cpu()
    sdpa_layer(qs[:, :64], kc, vc, **{**opts, **({"rope_q": (opts["rope_q"][0][:64], opts["rope_q"][1][:64])} if opts.get("rope_q") else {})})
    t0 = time.perf_counter()
    for _ in range(repeats):
        sdpa_layer(qs, kc, vc, **opts)
    return (time.perf_counter() - t0) / repeats, torch.get_num_threads()
