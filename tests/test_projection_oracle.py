"""Pins the projection / AdaLN oracle (oracle/projection_oracle.py) against library routines, closed forms and
identities chosen so that a dropped term, a transposed operand or a wrong index fails one of them."""
import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as AO
from oracle import projection_oracle as PO


def _r(*shape, seed=0, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


def test_lora_linear_base_term_is_the_library_linear():
    x, w, b = _r(7, 12, seed=1), _r(5, 12, seed=2), _r(5, seed=3)
    assert torch.allclose(PO.lora_linear(x, w, b), F.linear(x, w, b), atol=1e-13)
    assert torch.allclose(PO.lora_linear(x, w), F.linear(x, w), atol=1e-13)
    # a non-square weight in the wrong orientation cannot even multiply
    with pytest.raises(RuntimeError):
        PO.lora_linear(x, w.t().contiguous())


def test_lora_linear_equals_merged_weight_and_scales_linearly():
    x, w, b = _r(9, 16, seed=4), _r(6, 16, seed=5), _r(6, seed=6)
    a, bb = _r(3, 16, seed=7), _r(6, 3, seed=8)
    s = 0.37
    y = PO.lora_linear(x, w, b, lora_a=a, lora_b=bb, lora_scale=s)
    merged = w + s * (bb @ a)          # the identity PEFT's merge of an adapter into its base layer relies on
    assert torch.allclose(y, F.linear(x, merged, b), atol=1e-12)
    # zero B (PEFT's initialisation): the adapter is a no-op; scale 0 likewise
    assert torch.equal(PO.lora_linear(x, w, b, lora_a=a, lora_b=torch.zeros_like(bb), lora_scale=s), PO.lora_linear(x, w, b))
    assert torch.equal(PO.lora_linear(x, w, b, lora_a=a, lora_b=bb, lora_scale=0.0), PO.lora_linear(x, w, b))
    # the update is linear in the scale
    d1 = PO.lora_linear(x, w, b, lora_a=a, lora_b=bb, lora_scale=1.0) - PO.lora_linear(x, w, b)
    d2 = PO.lora_linear(x, w, b, lora_a=a, lora_b=bb, lora_scale=2.0) - PO.lora_linear(x, w, b)
    assert torch.allclose(d2, 2 * d1, atol=1e-12)


def test_lora_linear_rank_one_closed_form():
    x = _r(4, 8, seed=9)
    a = torch.zeros(1, 8, dtype=torch.float64); a[0, 2] = 1.0      # picks feature 2 of x
    b = torch.zeros(5, 1, dtype=torch.float64); b[3, 0] = 2.0      # writes twice that into output 3
    y = PO.lora_linear(x, torch.zeros(5, 8, dtype=torch.float64), lora_a=a, lora_b=b, lora_scale=0.5)
    expect = torch.zeros(4, 5, dtype=torch.float64); expect[:, 3] = x[:, 2]
    assert torch.allclose(y, expect, atol=1e-15)


@pytest.mark.parametrize("norm", ["layer", "rms"])
def test_adaln_matches_library_norms_and_index_select(norm):
    S, K, T = 11, 24, 3
    x = _r(S, K, seed=10) * 3 + 0.7
    shift, scale = _r(T, K, seed=11), _r(T, K, seed=12) * 0.2
    idx = torch.tensor([0, 2, 1, 1, 0, 2, 2, 0, 1, 0, 2])
    y = PO.adaln_modulate(x, shift=shift, scale=scale, row_index=idx, norm=norm, eps=1e-6)
    base = F.layer_norm(x, (K,), eps=1e-6) if norm == "layer" else F.rms_norm(x, (K,), eps=1e-6)
    expect = base * (1.0 + scale.index_select(0, idx)) + shift.index_select(0, idx)   # the patch's line
    assert torch.allclose(y, expect, atol=1e-12)
    # explicit row loop: row s uses table row idx[s], not s and not a transposed table
    for s_ in range(S):
        assert torch.allclose(y[s_], base[s_] * (1 + scale[idx[s_]]) + shift[idx[s_]], atol=1e-12)
    # zero modulation is the bare norm; no index means table row 0
    assert torch.allclose(PO.adaln_modulate(x, norm=norm), base, atol=1e-12)
    y0 = PO.adaln_modulate(x, shift=shift, scale=scale, norm=norm)
    assert torch.allclose(y0, base * (1 + scale[0]) + shift[0], atol=1e-12)


def test_adaln_closed_forms():
    # LayerNorm of a two-valued row: values +-1 exactly (up to eps); RMSNorm of a constant row c: sign(c)
    x = torch.tensor([[3.0, 5.0, 3.0, 5.0], [-2.0, -2.0, -2.0, -2.0]], dtype=torch.float64)
    ln = PO.adaln_modulate(x, norm="layer", eps=0.0)
    assert torch.allclose(ln[0], torch.tensor([-1.0, 1.0, -1.0, 1.0], dtype=torch.float64), atol=1e-12)
    rms = PO.adaln_modulate(x, norm="rms", eps=0.0)
    assert torch.allclose(rms[1], -torch.ones(4, dtype=torch.float64), atol=1e-12)
    # eps matters: a constant row under LayerNorm is 0 / sqrt(eps) = 0
    assert torch.allclose(PO.adaln_modulate(x, norm="layer", eps=1e-6)[1], torch.zeros(4, dtype=torch.float64), atol=1e-9)
    # shift-only / scale-only
    sh = torch.full((1, 4), 0.5, dtype=torch.float64)
    assert torch.allclose(PO.adaln_modulate(x, shift=sh, norm="layer", eps=0.0)[0], ln[0] + 0.5, atol=1e-12)
    assert torch.allclose(PO.adaln_modulate(x, scale=sh, norm="layer", eps=0.0)[0], ln[0] * 1.5, atol=1e-12)


def test_attention_block_is_the_composition_of_its_parts():
    S, C, H = 70, 256, 2
    x = (_r(S, C, seed=20) * 0.5).to(torch.bfloat16)
    T = 2
    shift, scale, gate = (_r(T, C, seed=s) * 0.1 for s in (21, 22, 23))
    idx = (torch.arange(S) % T).to(torch.int32)
    mk = lambda n, seed: dict(weight=_r(n, C, seed=seed) * 0.05, bias=_r(n, seed=seed + 1) * 0.01,
                              lora_a=_r(4, C, seed=seed + 2) * 0.05, lora_b=_r(n, 4, seed=seed + 3) * 0.05, lora_scale=0.5)
    lin = {"q": mk(C, 30), "k": mk(C, 40), "v": mk(C, 50), "out": mk(C, 60)}
    w = torch.ones(128)
    got = PO.attention_block(x, lin, heads=H, shift=shift, scale=scale, gate=gate, row_index=idx, round_bf16=False,
                             q_norm_weight=w, k_norm_weight=w)
    # by hand, step by step, with library routines
    xm = F.layer_norm(x.double(), (C,), eps=1e-6) * (1 + scale[idx.long()]) + shift[idx.long()]
    merged = {n: (d["weight"] + d["lora_scale"] * d["lora_b"] @ d["lora_a"], d["bias"]) for n, d in lin.items()}
    q, k, v = (F.linear(xm, *merged[n]).view(1, S, H, 128) for n in ("q", "k", "v"))
    qn, kn = (F.rms_norm(t, (128,), eps=1e-6) for t in (q, k))
    o = F.scaled_dot_product_attention(qn.transpose(1, 2), kn.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2).reshape(S, C)
    y = x.double() + gate[idx.long()] * F.linear(o, *merged["out"])
    assert torch.allclose(got["xm"], xm, atol=1e-10) and torch.allclose(got["o"], o, atol=1e-9)
    assert torch.allclose(got["y"], y, atol=1e-9)
    # the bf16 storage points only move the result within bf16 precision
    rounded = PO.attention_block(x, lin, heads=H, shift=shift, scale=scale, gate=gate, row_index=idx,
                                 q_norm_weight=w, k_norm_weight=w)
    err, cos = AO.max_abs_and_cosine(rounded["y"], y)
    assert err < 2e-2 and cos > 0.9999


def test_modulation_tables_activate_in_float32():
    """patches/0001-h3-adaln-fp32.patch:126-133: SiLU in float32 whatever dtype temb arrives in, then the cast, then
    the linear layer; rows of the view are (timestep, modality) pairs, timestep-major."""
    from pika_h3_flex_amd import projections as P

    g = torch.Generator().manual_seed(3)
    T, E, hidden, M = 3, 64, 32, 2
    temb = (torch.randn((T, E), generator=g) * 3).to(torch.bfloat16)
    weight = (torch.randn((6 * hidden * M, E), generator=g) * 0.1).to(torch.bfloat16)
    bias = (torch.randn(6 * hidden * M, generator=g) * 0.1).to(torch.bfloat16)
    ref = PO.modulation_tables(temb, weight, bias, hidden)
    # the library routine for the activation, in float32, agrees with the written-out form
    lib = torch.nn.functional.linear(torch.nn.functional.silu(temb.float()).to(torch.bfloat16).double(), weight.double(), bias.double())
    assert torch.allclose(torch.cat(ref, -1).reshape(T, -1), lib, atol=1e-12)
    # the activation is monotone in precision: taken on float32 input it is at least as close to the float64 value
    # as any bfloat16 evaluation can be (this torch build's bfloat16 SiLU already computes in float32 and rounds
    # once, so on it the patch changes no bit; an evaluation that rounds the sigmoid first does differ)
    exact = temb.double() * torch.sigmoid(temb.double())
    one_rounding = torch.nn.functional.silu(temb.float()).to(torch.bfloat16).double()
    two_roundings = (temb * torch.sigmoid(temb.float()).to(torch.bfloat16)).double()
    assert float((one_rounding - exact).abs().max()) <= float((two_roundings - exact).abs().max())
    assert float((one_rounding - two_roundings).abs().max()) > 0.0
    got = P.modulation_tables(temb, weight, bias, hidden)
    assert len(got) == 6 and all(t.shape == (T * M, hidden) and t.dtype == torch.bfloat16 for t in got)
    for a, b in zip(got, ref):
        assert float((a.double() - b).abs().max()) <= 2.0 ** -7 * max(1.0, float(b.abs().max()))  # one bf16 rounding of the output
    # row order: row t*M + m of chunk c is the slice [(m*6 + c)*hidden, +hidden) of timestep t's output
    for t in range(T):
        for m in range(M):
            for c in range(6):
                want = lib[t, (m * 6 + c) * hidden:(m * 6 + c + 1) * hidden]
                assert torch.equal(ref[c][t * M + m], want)
    # two chunks: the output norm's table (patch lines 150-158)
    assert len(P.modulation_tables(temb, weight[: 2 * hidden], bias[: 2 * hidden], hidden, chunks=2)) == 2
    with pytest.raises(ValueError):
        P.modulation_tables(temb, weight[:100], None, hidden)


def test_modulation_row_index():
    from pika_h3_flex_amd import projections as P

    ti = torch.tensor([0, 0, 2, 1, 2])
    assert P.modulation_row_index(ti).tolist() == [0, 0, 2, 1, 2] and P.modulation_row_index(ti).dtype == torch.int32
    mod = torch.tensor([1, 0, 0, 2, 1])
    assert P.modulation_row_index(ti, mod, 3).tolist() == [1, 0, 6, 5, 7]
    with pytest.raises(ValueError):
        P.modulation_row_index(ti, torch.tensor([0, 0, 3, 0, 0]), 3)
    with pytest.raises(ValueError):
        P.modulation_row_index(ti, mod[:3], 3)
