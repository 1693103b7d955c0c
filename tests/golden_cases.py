"""Loader for tests/golden/cases.npz (see tests/golden/make_golden.py)."""
import os

import numpy as np
import torch

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cases.npz")


def load():
    """{case name: {array name: tensor}}; bf16 tensors are restored from their int16 bit patterns."""
    data = np.load(PATH, allow_pickle=False)
    cases = {}
    for key in data.files:
        name, arr = key.split("/")
        val = data[key]
        if arr in ("q", "k", "v"):
            t = torch.from_numpy(val).view(torch.bfloat16)
        elif val.shape == ():
            t = int(val)
        else:
            t = torch.from_numpy(val)
        cases.setdefault(name, {})[arr] = t
    return cases


def oracle_kwargs(case, O):
    kw = {}
    if "q_norm_w" in case:
        kw.update(q_norm_weight=case["q_norm_w"], k_norm_weight=case["k_norm_w"])
    if "position_ids" in case:
        kw.update(rope_q=O.rope_tables(case["position_ids"]), rope_mode=case["rope_mode"])
    if "key_mask" in case:
        kw.update(key_mask=case["key_mask"])
    if "tile_map" in case:
        kw.update(tile_map=case["tile_map"])
    if case.get("fp8"):
        kw.update(fp8_qk=True)
    return kw
