"""GPU parity over seeded random combinations of shapes and options: batch, heads, ragged and rectangular
lengths around the tile edges, both RoPE pairings, norm on/off, large norm weights (running-max softmax path),
key masks (some rows fully masked), block-sparse maps, fp8 QK^T, and both forms of the dense kernel.
Every case is checked against the float64 oracle to the bar of its path."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

D = 128
LENGTHS_Q = [1, 7, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 383, 384, 385, 513, 700, 1025, 1100]
LENGTHS_K = [1, 5, 32, 33, 64, 65, 96, 100, 257, 640, 1023, 1024, 1025, 1500]


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_combinations(seed):
    import pika_h3_flex_amd as pk
    from oracle import attention_oracle as O

    rng = random.Random(seed)
    for case in range(40):
        B, H = rng.choice([1, 1, 2]), rng.choice([1, 2, 3])
        Sq = rng.choice(LENGTHS_Q)
        Sk = Sq if rng.random() < 0.5 else rng.choice(LENGTHS_K)
        mode = rng.choice(["plain", "plain", "mask", "sparse", "fp8", "sparse_fp8"])
        rope = rng.choice([0, 1, 2]) if Sq == Sk else 0
        norm = rng.random() < 0.8
        wscale = rng.choice([1.0, 1.0, 1.0, 3.5])
        long_form = rng.random() < 0.4
        g = torch.Generator().manual_seed(1000 * seed + case)
        q = torch.randn((B, Sq, H, D), generator=g).to(torch.bfloat16)
        k = torch.randn((B, Sk, H, D), generator=g).to(torch.bfloat16)
        v = torch.randn((B, Sk, H, D), generator=g).to(torch.bfloat16)
        opts, ref = {}, {}
        if norm:
            qw = (1.0 + 0.1 * torch.randn(D, generator=g)) * wscale
            kw = 1.0 + 0.1 * torch.randn(D, generator=g)
            opts.update(q_norm_weight=qw.cuda(), k_norm_weight=kw.cuda())
            ref.update(q_norm_weight=qw, k_norm_weight=kw)
        if rope:
            tabs = O.rope_tables(torch.rand((Sq, 3), generator=g, dtype=torch.float64) * 30)
            opts.update(rope_mode=rope, rope_q=tuple(t.float().contiguous().cuda() for t in tabs))
            ref.update(rope_mode=rope, rope_q=tabs)
        if mode == "mask":
            m = torch.rand((B, Sk), generator=g) < 0.6
            if rng.random() < 0.3:
                m[0] = False  # a batch with no valid key at all: its rows must come back as zeros
            opts.update(key_mask=m.cuda())
            ref.update(key_mask=m)
        if mode in ("sparse", "sparse_fp8"):
            tm = torch.rand(((Sq + 63) // 64, (Sk + 63) // 64), generator=g) < 0.4
            opts.update(block_mask=pk.BlockMask.from_dense(tm, device="cuda"))
            ref.update(tile_map=tm)
        fp8 = mode in ("fp8", "sparse_fp8")
        if fp8:
            opts.update(fp8_qk=True)
            ref.update(fp8_qk=True)
        elif wscale > 1 or not norm:
            ref.update(bf16_operands=True)  # large logits: the oracle rounds its operands like the matrix unit
        out = pk.attention(q.cuda(), k.cuda(), v.cuda(), long_key_kernel=long_form, **opts)
        torch.cuda.synchronize()
        expect = torch.nan_to_num(O.reference_layer(q, k, v, **ref), nan=0.0)  # rows without keys: zeros
        err, cos = O.max_abs_and_cosine(out.cpu(), expect)
        label = (f"seed {seed} case {case}: B={B} H={H} Sq={Sq} Sk={Sk} {mode} rope={rope} norm={norm} w={wscale} "
                 f"long_form={long_form}: max_abs={err:.3e} cos={cos:.6f}")
        print(label, flush=True)
        assert torch.isfinite(out.float()).all(), label
        all_zero = float(expect.abs().max()) == 0.0
        if fp8:
            assert cos >= 0.995 or (all_zero and err == 0.0), label
        else:
            assert err <= 2e-2 and (cos >= 0.9999 or all_zero), label


@pytest.mark.parametrize("seed", [0, 1])
def test_random_long_dense_calls_with_a_shared_last_round(seed):
    """Seeded long dense calls whose query tiles overflow whole rounds of workgroups by a random amount, so that the last
    tiles are shared out among 2 to 8 workgroups each (one or two sections, whatever the planner picks for the remainder):
    batches, key masks (compacted key counts differ per batch), rotation, fp8 with both scale rules, large logits
    (running-max merge).  Checked against the plain long form on the same inputs (one workgroup per query tile), for
    identical bits on a repeated call, and against the oracle on sampled rows of the last tiles."""
    import pika_h3_flex_amd as pk
    from oracle import attention_oracle as O

    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rng = random.Random(100 + seed)
    for case in range(10):
        B, H = rng.choice([(1, 24), (1, 16), (2, 12), (3, 8), (1, 40)])
        tiles = (cus + rng.randint(1, cus - 1) + B * H - 1) // (B * H)          # query tiles per (batch, head)
        Sq = tiles * 384 - rng.randint(0, 383)
        Sk = rng.choice([1100, 1536, 2500, 3100, 4700, 6000])
        mode = rng.choice(["plain", "plain", "mask", "fp8", "pow2", "large"])
        rope = rng.choice([0, 1, 2])
        g = torch.Generator().manual_seed(5000 * seed + case)
        q = torch.randn((B, Sq, H, D), generator=g).to(torch.bfloat16)
        k = torch.randn((B, Sk, H, D), generator=g).to(torch.bfloat16)
        v = torch.randn((B, Sk, H, D), generator=g).to(torch.bfloat16)
        qw = (1.0 + 0.1 * torch.randn(D, generator=g)) * (3.5 if mode == "large" else 1.0)
        kw = 1.0 + 0.1 * torch.randn(D, generator=g)
        opts = dict(q_norm_weight=qw.cuda(), k_norm_weight=kw.cuda())
        ref = dict(q_norm_weight=qw, k_norm_weight=kw)
        if rope:
            tq = O.rope_tables(torch.rand((Sq, 3), generator=g, dtype=torch.float64) * 30)
            tk = O.rope_tables(torch.rand((Sk, 3), generator=g, dtype=torch.float64) * 30)
            dev = lambda t: tuple(x.float().contiguous().cuda() for x in t)
            opts.update(rope_mode=rope, rope_q=dev(tq), rope_k=dev(tk))
            ref.update(rope_mode=rope, rope_q=tq, rope_k=tk)
        if mode == "mask":
            m = torch.rand((B, Sk), generator=g) < 0.7
            m[B - 1, : Sk // 2] = False            # the batches keep different numbers of keys
            opts.update(key_mask=m.cuda())
            ref.update(key_mask=m)
        if mode in ("fp8", "pow2"):
            opts.update(fp8_qk=True if mode == "fp8" else "pow2")
            ref.update(fp8_qk=True if mode == "fp8" else "pow2")
        if mode == "large":
            ref.update(bf16_operands=True)
        qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
        out = pk.attention(qc, kc, vc, **opts)
        again = pk.attention(qc, kc, vc, **opts)
        plain = pk.attention(qc, kc, vc, long_key_kernel=True, **opts)
        torch.cuda.synchronize()
        label = f"seed {seed} case {case}: B={B} H={H} Sq={Sq} ({B * H * tiles} query tiles on {cus} CUs) Sk={Sk} {mode} rope={rope}"
        assert torch.isfinite(out.float()).all(), label
        assert torch.equal(out, again), label
        err, cos = O.max_abs_and_cosine(out.cpu(), plain.cpu())
        # the two forms add the same products in a different order: a bf16 step of the output at most
        assert err <= 2.0 ** -6 * max(1.0, float(plain.float().abs().max())) and cos >= 0.99999, (label, err, cos)
        # oracle on rows of the last query tile of the last (batch, head): tiles the shared round holds
        rows = torch.tensor(sorted({Sq - 1, Sq - 2, Sq - 33, max(0, Sq - 200), max(0, Sq - 384), (tiles - 1) * 384}))
        expect = O.reference_layer(q[B - 1:, :, H - 1:], k[B - 1:, :, H - 1:], v[B - 1:, :, H - 1:], q_rows=rows,
                                   **{n: (t[B - 1:] if n == "key_mask" else t) for n, t in ref.items()})
        got = out[B - 1:, rows.cuda()][:, :, H - 1:].cpu()
        err, cos = O.max_abs_and_cosine(got, expect)
        print(f"{label}: vs oracle max_abs={err:.3e} cos={cos:.6f}", flush=True)
        if mode in ("fp8", "pow2"):
            assert cos >= 0.995, label
        else:
            assert err <= 2e-2 and cos >= 0.9999, label


@pytest.mark.parametrize("seed", [0, 1])
def test_random_block_sparse_calls_that_fill_the_part(seed):
    """Seeded block-sparse calls with more workgroups than the part has CUs, the size from which their units are handed
    out through the per-XCD work queues: random tile maps (density 0.03 to 0.5) with some row-blocks that keep nothing
    and some that keep everything, so that the workgroups' tile lists differ widely in length; rectangular lengths,
    rotation, fp8 with both scale rules.  Checked for identical bits on a repeated call and against the oracle on
    sampled rows of the first, last, an empty and a full row-block."""
    import pika_h3_flex_amd as pk
    from oracle import attention_oracle as O

    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rng = random.Random(300 + seed)
    for case in range(8):
        B, H = rng.choice([(1, 24), (1, 16), (2, 12), (3, 8)])
        groups = (cus + rng.randint(1, 2 * cus) + B * H - 1) // (B * H)        # workgroups (4 row-blocks) per (batch, head)
        Sq = groups * 256 - rng.randint(0, 255)
        Sk = Sq if rng.random() < 0.5 else rng.choice([700, 1536, 2500, 4100])
        mode = rng.choice(["bf16", "bf16", "fp8", "pow2"])
        rope = rng.choice([0, 1, 2]) if Sq == Sk else 0
        g = torch.Generator().manual_seed(9000 * seed + case)
        q = torch.randn((B, Sq, H, D), generator=g).to(torch.bfloat16)
        k = torch.randn((B, Sk, H, D), generator=g).to(torch.bfloat16)
        v = torch.randn((B, Sk, H, D), generator=g).to(torch.bfloat16)
        qw = 1.0 + 0.1 * torch.randn(D, generator=g)
        kw = 1.0 + 0.1 * torch.randn(D, generator=g)
        opts = dict(q_norm_weight=qw.cuda(), k_norm_weight=kw.cuda())
        ref = dict(q_norm_weight=qw, k_norm_weight=kw)
        if rope:
            tabs = O.rope_tables(torch.rand((Sq, 3), generator=g, dtype=torch.float64) * 30)
            opts.update(rope_mode=rope, rope_q=tuple(t.float().contiguous().cuda() for t in tabs))
            ref.update(rope_mode=rope, rope_q=tabs)
        nq, nk = (Sq + 63) // 64, (Sk + 63) // 64
        tm = torch.rand((nq, nk), generator=g) < rng.choice([0.03, 0.1, 0.25, 0.5])
        empty, full = rng.randrange(1, nq - 1), rng.randrange(1, nq - 1)
        tm[empty] = False
        tm[full] = True
        opts.update(block_mask=pk.BlockMask.from_dense(tm, device="cuda"))
        ref.update(tile_map=tm)
        if mode != "bf16":
            opts.update(fp8_qk=True if mode == "fp8" else "pow2")
            ref.update(fp8_qk=True if mode == "fp8" else "pow2")
        qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
        out = pk.attention(qc, kc, vc, **opts)
        again = pk.attention(qc, kc, vc, **opts)
        torch.cuda.synchronize()
        label = (f"seed {seed} case {case}: B={B} H={H} Sq={Sq} ({B * H * groups} workgroups on {cus} CUs) Sk={Sk} {mode} "
                 f"rope={rope} density={float(tm.float().mean()):.3f}")
        assert torch.isfinite(out.float()).all(), label
        assert torch.equal(out, again), label
        if empty != full:
            assert float(out[:, empty * 64:(empty + 1) * 64].float().abs().max()) == 0.0, label   # keeps nothing: zeros
        rows = sorted({0, 63, Sq - 1, (nq - 1) * 64, empty * 64 + 5, full * 64, full * 64 + 37,
                       min(Sq - 1, full * 64 + 63), rng.randrange(Sq), rng.randrange(Sq), rng.randrange(Sq)})
        rows = torch.tensor(rows)
        expect = torch.nan_to_num(O.reference_layer(q[B - 1:, :, H - 1:], k[B - 1:, :, H - 1:], v[B - 1:, :, H - 1:],
                                                    q_rows=rows, **ref), nan=0.0)
        got = out[B - 1:, rows.cuda()][:, :, H - 1:].cpu()
        err, cos = O.max_abs_and_cosine(got, expect)
        print(f"{label}: vs oracle max_abs={err:.3e} cos={cos:.6f}", flush=True)
        if mode != "bf16":
            assert cos >= 0.995, label
        else:
            assert err <= 2e-2 and cos >= 0.9999, label
