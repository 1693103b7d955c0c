"""The entry point that allocates nothing (``pkh3_attn_fwd_noalloc``): same kernels as ``pkh3_attn_fwd`` with the
scratch in an array built into the library.  Its output must equal the workspace entry point's bit for bit, on two
calls in a row that share the array (the second smaller, so stale contents of the first lie behind it), for the
variants whose scratch differs (dense, key mask, block-sparse, fp8); oversized calls are rejected on the host."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu

D = 128


def _inputs(S, Sk, H, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((1, S, H, D), generator=g).to(torch.bfloat16).cuda()
    k, v = (torch.randn((1, Sk, H, D), generator=g).to(torch.bfloat16).cuda() for _ in range(2))
    return q, k, v


def _both(q, k, v, **opts):
    import pika_h3_flex_amd as pk

    w = torch.ones(D, device="cuda")
    opts = dict(q_norm_weight=w, k_norm_weight=w, **opts)
    out_static = torch.empty_like(q)
    pk.attention(q, k, v, out=out_static, static_scratch=True, **opts)
    ref = pk.attention(q, k, v, **opts)
    torch.cuda.synchronize()
    return out_static, ref


@pytest.mark.parametrize("variant", ["dense", "key_mask", "sparse", "fp8", "sparse_fp8"])
def test_noalloc_matches_workspace_entry_point_twice_in_a_row(variant):
    import pika_h3_flex_amd as pk

    for S, Sk, H, seed in ((1500, 1500, 6, 1), (333, 200, 3, 2)):   # the second call is smaller
        if variant == "key_mask":
            Sk = min(Sk, 512)
        if "sparse" in variant:
            Sk = S
        q, k, v = _inputs(S, Sk, H, seed)
        opts = {}
        if variant == "key_mask":
            opts["key_mask"] = (torch.rand((1, Sk), generator=torch.Generator().manual_seed(seed)) < 0.6).cuda()
        if "sparse" in variant:
            n = (S + 63) // 64
            tm = torch.rand((n, n), generator=torch.Generator().manual_seed(seed)) < 0.4
            tm |= torch.eye(n, dtype=torch.bool)
            opts["block_mask"] = pk.BlockMask.from_dense(tm, device="cuda")
        if "fp8" in variant:
            opts["fp8_qk"] = True
        got, ref = _both(q, k, v, **opts)
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, ref), (variant, S, float((got.float() - ref.float()).abs().max()))


def test_noalloc_agrees_with_the_oracle():
    from oracle import attention_oracle as O

    q, k, v = _inputs(700, 700, 4, 5)
    got, _ = _both(q, k, v)
    w = torch.ones(D)
    ref = O.reference_layer(q.cpu(), k.cpu(), v.cpu(), q_norm_weight=w, k_norm_weight=w)
    err, cos = O.max_abs_and_cosine(got.cpu(), ref)
    assert err <= 2e-2 and cos >= 0.9999, (err, cos)   # bf16 bar of the path


def test_noalloc_rejects_calls_beyond_its_scratch():
    import pika_h3_flex_amd as pk
    from pika_h3_flex_amd import _lib

    # 24 heads x 8192 keys x 512 B of K/V images = 96 MiB > 64 MiB; rejected on the host, before any launch
    q = torch.empty((1, 64, 24, D), dtype=torch.bfloat16, device="cuda")
    k = torch.empty((1, 8192, 24, D), dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(q)
    args, _keep = pk.ops.fill_args(q, k, k, out)
    assert pk.ops.workspace_bytes(args) > _lib.NOALLOC_SCRATCH_BYTES
    lib = _lib.load()
    rc = lib.pkh3_attn_fwd_noalloc(C.byref(args), None)
    assert rc == _lib.PKH3_EWORKSPACE and b"scratch" in lib.pkh3_last_error()
    with pytest.raises(_lib.Pkh3Error):
        pk.attention(q, k, k, out=out, static_scratch=True)


def test_noalloc_captured_into_a_hip_graph_replays_the_eager_bits():
    """The entry point is meant for callers under HIP graph capture: after ``pkh3_noalloc_init`` (the look-ups that
    are not stream operations) the call is captured, and every replay -- fresh inputs in the captured buffers, eager
    work of the same entry point in between, which shares the built-in array -- gives the bits of an eager
    ``pkh3_attn_fwd`` call on the same inputs."""
    import pika_h3_flex_amd as pk

    pk.ops.noalloc_init()
    S, H = 700, 3
    gen = torch.Generator().manual_seed(44)
    rnd = lambda: torch.randn((1, S, H, D), generator=gen).to(torch.bfloat16).cuda()
    q, k, v = rnd(), rnd(), rnd()
    w = torch.ones(D, device="cuda")
    pos = torch.rand((S, 3), generator=gen, dtype=torch.float64) * 20.0
    opts = dict(q_norm_weight=w, k_norm_weight=w, rope_mode=1, rope_q=pk.rope_tables(pos.cuda()))
    out = torch.empty_like(q)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pk.attention(q, k, v, out=out, static_scratch=True, **opts)
    for rep in range(3):
        fresh = [rnd() for _ in range(3)]
        eager = pk.attention(*fresh, **opts).clone()
        # eager use of the shared array between the replays, with another shape
        other = pk.attention(fresh[0][:, :200], fresh[1][:, :300], fresh[2][:, :300], static_scratch=True,
                             q_norm_weight=w, k_norm_weight=w)
        torch.cuda.synchronize()
        for dst, src in zip((q, k, v), fresh):
            dst.copy_(src)
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(other.float()).all()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager call"
