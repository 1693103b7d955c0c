"""Pins the CPU oracle: every function is checked against a library routine, a closed form, an
invariant or a brute-force loop that a plausible mistake (dropped term, wrong sign or index,
transposed operand) would break.  The reference has no golden vectors for attention, so these
checks -- not retyped formulas -- are what the oracle's authority rests on."""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as O

torch.manual_seed(0)


def _r(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=dtype)


# ------------------------------------------------------------------------------------- RMSNorm
def test_rms_norm_matches_torch_library():
    x, w = _r(2, 9, 3, 128, seed=1), _r(128, seed=2)
    ref = F.rms_norm(x, (128,), w, 1e-6)
    assert torch.allclose(O.rms_norm(x, w, 1e-6), ref, atol=1e-12)


def test_rms_norm_unit_weight_gives_unit_rms_rows():
    y = O.rms_norm(_r(4, 7, 2, 128, seed=3) * 13.0, torch.ones(128), 1e-6)
    assert torch.allclose((y * y).mean(-1).sqrt(), torch.ones(4, 7, 2, dtype=torch.float64), atol=1e-6)


def test_rms_norm_scalar_closed_form_and_eps():
    x = torch.full((1, 1, 1, 128), 3.0, dtype=torch.float64)
    assert torch.allclose(O.rms_norm(x, None, 0.0), torch.ones_like(x))
    # eps enters under the square root: x / sqrt(x^2 + eps)
    assert torch.allclose(O.rms_norm(x, None, 7.0), x / math.sqrt(16.0))


# ------------------------------------------------------------------------------------- RoPE
def _pos(S, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.rand((S, 3), generator=g, dtype=torch.float64) * torch.tensor([30.0, 29.0, 51.0], dtype=torch.float64)


def test_rope_tables_layout_and_frequencies():
    pos = torch.tensor([[2.0, 3.0, 5.0]], dtype=torch.float64)
    cos, sin = O.rope_tables(pos, (32, 48, 48), 10000.0)
    assert cos.shape == (1, 64)
    # pair 0 of each axis turns by the raw position; the last pair of the t axis by pos * theta^(-30/32)
    for col, p in ((0, 2.0), (16, 3.0), (40, 5.0)):
        assert abs(cos[0, col] - math.cos(p)) < 1e-12 and abs(sin[0, col] - math.sin(p)) < 1e-12
    ang = 2.0 * 10000.0 ** (-30.0 / 32.0)
    assert abs(cos[0, 15] - math.cos(ang)) < 1e-12
    ang = 5.0 * 10000.0 ** (-46.0 / 48.0)
    assert abs(sin[0, 63] - math.sin(ang)) < 1e-12


@pytest.mark.parametrize("mode", [O.ROPE_INTERLEAVED, O.ROPE_HALF])
def test_rope_equals_complex_multiplication(mode):
    S = 11
    x = _r(1, S, 2, 128, seed=5)
    cos, sin = O.rope_tables(_pos(S, 1))
    y = O.apply_rope(x, cos, sin, mode)
    rot = torch.complex(cos, sin)[None, :, None, :]
    if mode == O.ROPE_INTERLEAVED:
        z = torch.view_as_complex(x.reshape(1, S, 2, 64, 2).contiguous()) * rot
        ref = torch.view_as_real(z).reshape(1, S, 2, 128)
    else:
        z = torch.complex(x[..., :64], x[..., 64:]) * rot
        ref = torch.cat([z.real, z.imag], -1)
    assert torch.allclose(y, ref, atol=1e-12)


@pytest.mark.parametrize("mode", [O.ROPE_INTERLEAVED, O.ROPE_HALF])
def test_rope_invariants(mode):
    S = 6
    x = _r(1, S, 1, 128, seed=6)
    cos, sin = O.rope_tables(_pos(S, 2))
    y = O.apply_rope(x, cos, sin, mode)
    # rotation: norms preserved (pairwise, hence per row)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-10)
    # position 0 is the identity
    c0, s0 = O.rope_tables(torch.zeros((S, 3), dtype=torch.float64))
    assert torch.allclose(O.apply_rope(x, c0, s0, mode), x, atol=1e-14)


@pytest.mark.parametrize("mode", [O.ROPE_INTERLEAVED, O.ROPE_HALF])
def test_rope_scores_depend_on_relative_position_only(mode):
    q, k = _r(1, 1, 1, 128, seed=7), _r(1, 1, 1, 128, seed=8)
    pq, pk = torch.tensor([[3.0, 4.0, 5.0]], dtype=torch.float64), torch.tensor([[1.0, 9.0, 2.0]], dtype=torch.float64)
    shift = torch.tensor([[7.5, -2.0, 11.0]], dtype=torch.float64)

    def score(a, b):
        qa = O.apply_rope(q, *O.rope_tables(a), mode)
        kb = O.apply_rope(k, *O.rope_tables(b), mode)
        return float((qa * kb).sum())

    assert abs(score(pq, pk) - score(pq + shift, pk + shift)) < 1e-9
    assert abs(score(pq, pk) - score(pq + shift, pk)) > 1e-3  # and it does depend on the offset


def test_rope_axis_independence_interleaved():
    """Changing only the h coordinate touches only the h slice, dims 32..79 of the 32/48/48 split."""
    x = _r(1, 1, 1, 128, seed=9)
    a = torch.tensor([[3.0, 4.0, 5.0]], dtype=torch.float64)
    b = torch.tensor([[3.0, 8.0, 5.0]], dtype=torch.float64)
    ya = O.apply_rope(x, *O.rope_tables(a), O.ROPE_INTERLEAVED)
    yb = O.apply_rope(x, *O.rope_tables(b), O.ROPE_INTERLEAVED)
    changed = (ya - yb).abs()[0, 0, 0] > 1e-12
    assert not changed[:32].any() and not changed[80:].any() and changed[32:80].any()


# ------------------------------------------------------------------------------------- attention
def test_attention_matches_torch_sdpa_library():
    q, k, v = _r(2, 50, 3, 128, seed=10), _r(2, 70, 3, 128, seed=11), _r(2, 70, 3, 128, seed=12)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2)
    assert torch.allclose(O.attention(q, k, v), ref, atol=1e-10)


def test_attention_brute_force_python_loops():
    B, Sq, Sk, H, Dh = 1, 3, 5, 2, 4
    q, k, v = _r(B, Sq, H, Dh, seed=13), _r(B, Sk, H, Dh, seed=14), _r(B, Sk, H, Dh, seed=15)
    out = O.attention(q, k, v)
    for h, i in itertools.product(range(H), range(Sq)):
        logits = [sum(float(q[0, i, h, d]) * float(k[0, j, h, d]) for d in range(Dh)) / math.sqrt(Dh) for j in range(Sk)]
        mx = max(logits)
        wts = [math.exp(x - mx) for x in logits]
        den = sum(wts)
        for d in range(Dh):
            val = sum(wts[j] * float(v[0, j, h, d]) for j in range(Sk)) / den
            assert abs(val - float(out[0, i, h, d])) < 1e-12


def test_attention_closed_forms():
    q, k, v = _r(1, 8, 2, 128, seed=16), _r(1, 12, 2, 128, seed=17), _r(1, 12, 2, 128, seed=18)
    # constant V: every output row is that V row
    vc = v[:, :1].expand(-1, 12, -1, -1)
    assert torch.allclose(O.attention(q, k, vc), vc[:, :1].expand(-1, 8, -1, -1), atol=1e-12)
    # zero K: uniform weights, output = mean of V over keys
    assert torch.allclose(O.attention(q, torch.zeros_like(k), v), v.mean(1, keepdim=True).expand(-1, 8, -1, -1), atol=1e-12)
    # one dominant logit: output -> that key's V row
    kd = torch.zeros_like(k)
    kd[:, 5] = q[:, 0] * 100.0
    out = O.attention(q[:, :1], kd, v)
    assert torch.allclose(out[:, 0], v[:, 5], atol=1e-9)


def test_attention_invariances():
    q, k, v = _r(1, 9, 2, 128, seed=19), _r(1, 14, 2, 128, seed=20), _r(1, 14, 2, 128, seed=21)
    base = O.attention(q, k, v)
    perm = torch.randperm(14, generator=torch.Generator().manual_seed(1))
    assert torch.allclose(O.attention(q, k[:, perm], v[:, perm]), base, atol=1e-12)  # joint key permutation
    qperm = torch.randperm(9, generator=torch.Generator().manual_seed(2))
    assert torch.allclose(O.attention(q[:, qperm], k, v), base[:, qperm], atol=1e-12)  # query permutation
    # the scale argument is 1/sqrt(D) by default and is applied to the logits
    assert torch.allclose(O.attention(q, k, v, scale=1.0 / math.sqrt(128.0)), base, atol=1e-14)
    assert torch.allclose(O.attention(q * 2.0, k, v, scale=0.5 / math.sqrt(128.0)), base, atol=1e-12)
    # restricting to rows gives those rows
    rows = torch.tensor([7, 0, 3])
    assert torch.allclose(O.attention(q, k, v, q_rows=rows), base[:, rows], atol=1e-14)


def test_key_mask_equals_slicing():
    q, k, v = _r(2, 6, 2, 128, seed=22), _r(2, 20, 2, 128, seed=23), _r(2, 20, 2, 128, seed=24)
    mask = torch.zeros((2, 20), dtype=torch.bool)
    mask[0, :7] = True
    mask[1, [1, 4, 5, 11, 19]] = True
    out = O.attention(q, k, v, key_mask=mask)
    for b in range(2):
        idx = mask[b].nonzero()[:, 0]
        assert torch.allclose(out[b : b + 1], O.attention(q[b : b + 1], k[b : b + 1, idx], v[b : b + 1, idx]), atol=1e-12)
    assert torch.allclose(O.attention(q, k, v, key_mask=torch.ones((2, 20), dtype=torch.bool)), O.attention(q, k, v), atol=1e-14)
    assert torch.count_nonzero(O.attention(q, k, v, key_mask=torch.zeros((2, 20), dtype=torch.bool))) == 0


def test_tile_map_equals_dense_with_dropped_tiles():
    Sq, Sk = 150, 200
    q, k, v = _r(1, Sq, 2, 128, seed=25), _r(1, Sk, 2, 128, seed=26), _r(1, Sk, 2, 128, seed=27)
    tm = torch.tensor([[1, 0, 1, 0], [0, 1, 1, 0], [1, 1, 0, 1]], dtype=torch.bool)
    out = O.attention(q, k, v, tile_map=tm)
    em = O.expand_tile_map(tm, Sq, Sk)
    assert em.shape == (Sq, Sk) and bool(em[63, 128]) and not bool(em[64, 0]) and bool(em[149, 199])
    bias = torch.zeros((Sq, Sk), dtype=torch.float64).masked_fill(~em, float("-inf"))
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask=bias).transpose(1, 2)
    assert torch.allclose(out, ref, atol=1e-10)
    assert torch.allclose(O.attention(q, k, v, tile_map=torch.ones((3, 4), dtype=torch.bool)), O.attention(q, k, v), atol=1e-14)


# ------------------------------------------------------------------------------------- fp8 e4m3
def _decode_e4m3fn(code: int) -> float:
    s, e, m = code >> 7, (code >> 3) & 0xF, code & 7
    if e == 0xF and m == 7:
        return float("nan")
    val = (m / 8.0) * 2.0 ** -6 if e == 0 else (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return -val if s else val


def test_fp8_round_is_nearest_representable_ties_even():
    grid = sorted({_decode_e4m3fn(c) for c in range(256) if not math.isnan(_decode_e4m3fn(c))})
    assert max(grid) == 448.0 and min(x for x in grid if x > 0) == 2.0 ** -9
    g = np.array(grid)
    # representable values are fixed points
    assert np.array_equal(O.fp8_e4m3_round(g), g)
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.uniform(-460, 460, 4000), rng.normal(0, 1, 4000), rng.uniform(-0.02, 0.02, 2000)])
    r = O.fp8_e4m3_round(x)
    xc = np.clip(x, -448, 448)
    # brute force: nearest grid point
    nearest = g[np.abs(g[None, :] - xc[:, None]).argmin(1)]
    dist_r, dist_n = np.abs(r - xc), np.abs(nearest - xc)
    assert np.all(np.isin(r, g)) and np.allclose(dist_r, dist_n, atol=0, rtol=0)
    # exact midpoints go to the even mantissa: between 1.0 (m=0) and 1.125 (m=1) -> 1.0; 1.125..1.25 -> 1.25
    assert O.fp8_e4m3_round(np.array([1.0625]))[0] == 1.0 and O.fp8_e4m3_round(np.array([1.1875]))[0] == 1.25


def test_fp8_round_agrees_with_torch_cast():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.uniform(-448, 448, 5000), rng.normal(0, 2, 5000)]).astype(np.float32)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).to(torch.float64).numpy()
    assert np.array_equal(O.fp8_e4m3_round(x.astype(np.float64)), ref)
    # the device-side variant of the rounding (used when the oracle runs on the GPU box's card) is that cast
    assert np.array_equal(O.fp8_e4m3_round_torch(torch.from_numpy(x)).numpy(), ref)
    # ... including every representable value, the extremes and values just below/above the midpoints
    grid = np.array(sorted({_decode_e4m3fn(c) for c in range(256) if not math.isnan(_decode_e4m3fn(c))}), dtype=np.float32)
    mids = ((grid[1:] + grid[:-1]) / 2).astype(np.float32)
    probe = np.concatenate([grid, mids, np.nextafter(mids, np.float32(1e9)), np.nextafter(mids, np.float32(-1e9))])
    assert np.array_equal(O.fp8_e4m3_round_torch(torch.from_numpy(probe)).numpy(), O.fp8_e4m3_round(probe.astype(np.float64)))


def test_fake_quant_blocks_scales_and_error_bound():
    x = _r(1, 130, 2, 128, seed=28) * 3.0
    deq, scales = O.fake_quant_fp8_blocks(x)
    assert scales.shape == (1, 2, 3)
    for blk, h in itertools.product(range(3), range(2)):
        rows = x[0, blk * 64 : (blk + 1) * 64, h]
        amax = float(rows.abs().max())
        assert abs(float(scales[0, h, blk]) - amax / 448.0) <= 1e-6 * amax
        err = (deq[0, blk * 64 : (blk + 1) * 64, h] - rows).abs()
        # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normals, absolute <= scale * 2^-10 for subnormals
        bound = torch.maximum(rows.abs() * 2.0 ** -4, torch.tensor(float(scales[0, h, blk]) * 2.0 ** -10)) * (1 + 1e-6)
        assert bool((err <= bound).all())
    # the block absmax itself is represented exactly (it maps to 448)
    i = x[0, :64, 0].abs().argmax()
    assert abs(float(deq[0, :64, 0].flatten()[i]) - float(x[0, :64, 0].flatten()[i])) < 1e-5 * float(x[0, :64, 0].abs().max())


def test_pow2_ceil_over_every_float32_exponent():
    """The bit rule against math.frexp (an independent path: frexp returns m in [0.5, 1) and e with x = m * 2^e, so
    the smallest power of two >= x is 2^(e-1) when m == 0.5 and 2^e otherwise), on every normal exponent: the power
    itself, one ulp above, one ulp below, and a mid-binade value."""
    vals = []
    for e in range(-126, 128):
        p = np.float32(2.0) ** np.float32(e)
        vals += [p, np.nextafter(p, np.float32(np.inf)), np.float32(p * np.float32(1.5))]
        if e > -126:
            vals.append(np.nextafter(p, np.float32(0)))
    vals = np.array([v for v in vals if np.isfinite(v)], dtype=np.float32)
    got = O.pow2_ceil_f32(torch.from_numpy(vals)).numpy().astype(np.float64)
    for v, g in zip(vals.astype(np.float64), got):
        m, e = math.frexp(float(v))
        want = math.ldexp(1.0, e - 1 if m == 0.5 else e)
        want = min(want, 2.0 ** 127)     # the largest scale an 8-bit exponent names
        assert g == want, (v, g, want)
        assert g >= min(v, 2.0 ** 127) and (g / 2 < v or g == 2.0 ** -126)


def test_fake_quant_pow2_scales():
    x = _r(1, 130, 2, 128, seed=29) * 3.0
    x[0, 64:128, 1] = 0.0                      # a block of zeros: scale 1, values 0
    x[0, 0, 0, 0] = 448.0 * 2.0 ** -5          # absmax / 448 an exact power of two: the scale is that power
    x[0, :64, 0] = x[0, :64, 0].clamp(-14.0, 14.0)
    deq, scales = O.fake_quant_fp8_blocks(x, pow2_scales=True)
    ref_deq, ref_scales = O.fake_quant_fp8_blocks(x)
    assert float(scales[0, 0, 0]) == 2.0 ** -5 and float(scales[0, 1, 1]) == 1.0
    assert torch.count_nonzero(deq[0, 64:128, 1]) == 0
    for blk, h in itertools.product(range(3), range(2)):
        s = float(scales[0, h, blk])
        rows = x[0, blk * 64 : (blk + 1) * 64, h].double()
        if float(rows.abs().max()) == 0:
            continue
        m, e = math.frexp(s)
        assert m == 0.5                                             # a power of two
        assert float(ref_scales[0, h, blk]) <= s < 2 * float(ref_scales[0, h, blk])
        # brute force: the nearest e4m3 value of rows / s, scaled back (division by a power of two is exact)
        want = torch.from_numpy(O.fp8_e4m3_round((rows / s).numpy())) * s
        assert torch.equal(deq[0, blk * 64 : (blk + 1) * 64, h], want)
        assert float((rows / s).abs().max()) <= 448.0               # nothing saturates
        err = (want - rows).abs()
        assert bool((err <= torch.maximum(rows.abs() * 2.0 ** -4, torch.tensor(s * 2.0 ** -10)) * (1 + 1e-9)).all())


def test_reference_layer_pow2_folds_the_softmax_scale_into_q():
    """fp8_qk="pow2": K as fake_quant(pow2), Q as fake_quant(pow2) of q * scale * log2(e), divided back."""
    q, k, v = _r(1, 96, 2, 128, seed=30), _r(1, 80, 2, 128, seed=31), _r(1, 80, 2, 128, seed=32)
    w = torch.ones(128)
    got = O.reference_layer(q, k, v, q_norm_weight=w, k_norm_weight=w, fp8_qk="pow2", scale=0.11)
    cq = float(np.float32(0.11) * np.float32(1.4426950408889634))
    qn, kn = O.rms_norm(q, w, 1e-6), O.rms_norm(k, w, 1e-6)
    qd = O.fake_quant_fp8_blocks(qn.float() * cq, pow2_scales=True)[0] / cq
    kd = O.fake_quant_fp8_blocks(kn, pow2_scales=True)[0]
    want = O.attention(qd, kd, v, scale=0.11)
    assert torch.equal(got, want)
    # and it stays an fp8-grade approximation of the unquantised layer, like the absmax form
    plain = O.reference_layer(q, k, v, q_norm_weight=w, k_norm_weight=w, scale=0.11)
    absmax = O.reference_layer(q, k, v, q_norm_weight=w, k_norm_weight=w, fp8_qk=True, scale=0.11)
    assert O.max_abs_and_cosine(got, plain)[1] >= 0.999 and O.max_abs_and_cosine(absmax, plain)[1] >= 0.999


def test_reference_layer_composes_the_parts():
    S = 40
    q, k, v = (_r(1, S, 2, 128, seed=s).to(torch.bfloat16) for s in (30, 31, 32))
    w = 1.0 + 0.1 * _r(128, seed=33)
    tabs = O.rope_tables(_pos(S, 3))
    out = O.reference_layer(q, k, v, q_norm_weight=w, k_norm_weight=w, rope_q=tabs, rope_mode=O.ROPE_INTERLEAVED)
    qn = O.apply_rope(O.rms_norm(q, w, 1e-6), *tabs, O.ROPE_INTERLEAVED)
    kn = O.apply_rope(O.rms_norm(k, w, 1e-6), *tabs, O.ROPE_INTERLEAVED)
    ref = F.scaled_dot_product_attention(qn.transpose(1, 2), kn.transpose(1, 2), v.double().transpose(1, 2)).transpose(1, 2)
    assert torch.allclose(out, ref, atol=1e-10)


def test_cpu_sdpa_baseline_agrees_with_oracle():
    """The timed CPU baseline computes the same function as the oracle (fp32 tolerance)."""
    from oracle import cpu_sdpa

    S = 70
    q, k, v = (_r(1, S, 2, 128, seed=s, dtype=torch.float32).to(torch.bfloat16) for s in (34, 35, 36))
    w = torch.ones(128)
    tabs = O.rope_tables(_pos(S, 4))
    ref = O.reference_layer(q, k, v, q_norm_weight=w, k_norm_weight=w, rope_q=tabs, rope_mode=O.ROPE_INTERLEAVED)
    out = cpu_sdpa.sdpa_layer(q, k, v, q_norm_weight=w, k_norm_weight=w, rope_q=tabs)
    assert (out.double() - ref).abs().max() < 1e-4


def test_bf16_operands_option_rounds_q_and_k_only():
    S = 20
    q, k, v = (_r(1, S, 1, 128, seed=s) for s in (40, 41, 42))
    a = O.reference_layer(q, k, v, bf16_operands=True)
    cq = 128 ** -0.5 * math.log2(math.e)  # Q is rounded carrying the log2-domain softmax factor
    b = O.attention((q.double() * cq).to(torch.bfloat16).double() / cq, k.to(torch.bfloat16).double(), v)
    assert torch.equal(a, b)
    # and stays within bf16 rounding of the exact result
    assert (a - O.reference_layer(q, k, v)).abs().max() < 2e-2
    assert not torch.equal(a, O.reference_layer(q, k, v))
