"""Writes tests/golden/cases.npz: small seeded input/output vectors of the attention path, the
outputs computed by the float64 oracle (oracle/attention_oracle.py) in this container.

The reference ships no golden vectors for attention and its attention module cannot be imported
(un-vendored diffusers pin), so these vectors come from the oracle, whose functions are pinned by
tests/test_oracle.py.  They freeze the oracle's results (CPU test) and give the GPU path a fixed
target that does not depend on regenerating inputs (GPU test).

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attention_oracle as O  # noqa: E402

CASES = {
    # name: (Sq, Sk, H, options)
    "self_norm_rope_interleaved": dict(Sq=101, Sk=101, H=2, norm=True, rope=O.ROPE_INTERLEAVED),
    "self_norm_rope_half": dict(Sq=70, Sk=70, H=1, norm=True, rope=O.ROPE_HALF),
    "cross_key_mask": dict(Sq=90, Sk=130, H=2, norm=True, mask_valid=47),
    "block_sparse": dict(Sq=200, Sk=200, H=1, norm=True, tile_map=[[1, 0, 1, 0], [1, 1, 0, 0], [0, 0, 1, 1], [1, 0, 0, 1]]),
    "fp8_qk": dict(Sq=130, Sk=130, H=1, norm=True, rope=O.ROPE_INTERLEAVED, fp8=True),
    "plain_no_norm": dict(Sq=33, Sk=77, H=2, norm=False, std=0.4),
}


def build_case(name, cfg, seed):
    g = torch.Generator().manual_seed(seed)
    D = 128
    std = cfg.get("std", 1.0)
    q = (torch.randn((1, cfg["Sq"], cfg["H"], D), generator=g) * std).to(torch.bfloat16)
    k = (torch.randn((1, cfg["Sk"], cfg["H"], D), generator=g) * std).to(torch.bfloat16)
    v = torch.randn((1, cfg["Sk"], cfg["H"], D), generator=g).to(torch.bfloat16)
    arrays = {"q": q.view(torch.int16).numpy(), "k": k.view(torch.int16).numpy(), "v": v.view(torch.int16).numpy()}
    kw = {}
    if cfg.get("norm"):
        qw = (1.0 + 0.1 * torch.randn(D, generator=g)).float()
        kw_ = (1.0 + 0.1 * torch.randn(D, generator=g)).float()
        arrays["q_norm_w"], arrays["k_norm_w"] = qw.numpy(), kw_.numpy()
        kw.update(q_norm_weight=qw, k_norm_weight=kw_)
    if cfg.get("rope"):
        pos = torch.rand((cfg["Sq"], 3), generator=g, dtype=torch.float64) * torch.tensor([30.0, 29.0, 51.0], dtype=torch.float64)
        arrays["position_ids"] = pos.numpy()
        arrays["rope_mode"] = np.int32(cfg["rope"])
        kw.update(rope_q=O.rope_tables(pos), rope_mode=cfg["rope"])
    if "mask_valid" in cfg:
        mask = torch.arange(cfg["Sk"])[None, :] < cfg["mask_valid"]
        arrays["key_mask"] = mask.numpy()
        kw.update(key_mask=mask)
    if "tile_map" in cfg:
        tm = torch.tensor(cfg["tile_map"], dtype=torch.bool)
        arrays["tile_map"] = tm.numpy()
        kw.update(tile_map=tm)
    if cfg.get("fp8"):
        arrays["fp8"] = np.int32(1)
        kw.update(fp8_qk=True)
    out = O.reference_layer(q, k, v, **kw)
    arrays["out"] = out.to(torch.float32).numpy()
    return {f"{name}/{key}": val for key, val in arrays.items()}


def main():
    blob = {}
    for i, (name, cfg) in enumerate(CASES.items()):
        blob.update(build_case(name, cfg, seed=1000 + i))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cases.npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {path}: {len(CASES)} cases, {os.path.getsize(path) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
