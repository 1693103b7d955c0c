"""Host-side logic that runs without a GPU: packed-sequence geometry, the block-sparse tile map
and its CSR form, and the attention processor's argument handling."""
import pytest
import torch

import pika_h3_flex_amd as pk
from pika_h3_flex_amd import layout
from pika_h3_flex_amd.ops import BlockMask


def test_video_positions_are_frame_major_then_row_major():
    pos = layout.video_position_ids(3, 4, 5)
    assert pos.shape == (60, 3) and pos.dtype == torch.float64
    # row n -> (n // 20, (n % 20) // 5, n % 5), the order patchify produces
    assert pos[0].tolist() == [0, 0, 0] and pos[4].tolist() == [0, 0, 4] and pos[5].tolist() == [0, 1, 0]
    assert pos[20].tolist() == [1, 0, 0] and pos[59].tolist() == [2, 3, 4]
    # cross-check against an explicit meshgrid
    t, h, w = torch.meshgrid(torch.arange(3), torch.arange(4), torch.arange(5), indexing="ij")
    assert torch.equal(pos, torch.stack([t, h, w], -1).reshape(-1, 3).double())


def test_audio_positions_channel_major_1d():
    pos = layout.audio_position_ids(7)
    assert pos.shape == (14, 3)
    assert pos[:, 0].tolist() == list(range(7)) * 2 and float(pos[:, 1:].abs().sum()) == 0.0


def test_benchmark_sequence_lengths():
    assert layout.video_position_ids(31, 30, 52).shape[0] == 48360
    assert layout.video_position_ids(31, 48, 84).shape[0] == 124992
    assert 48360 + layout.audio_position_ids(640).shape[0] == 49640


def test_local_window_tile_map_properties():
    S, tpf = 48360, 1560
    tm = layout.local_window_tile_map(S, tpf, window_frames=2, global_fraction=0.10, seed=0)
    n = (S + 63) // 64
    assert tm.shape == (n, n) and tm.dtype == torch.bool
    assert bool(tm.diagonal().all())
    win = layout.local_window_tile_map(S, tpf, window_frames=2, global_fraction=0.0)
    assert torch.equal(win, win.t())  # the window criterion is symmetric
    assert bool((tm | ~win).all())    # the random tiles only add
    # a tile pair is inside the window iff the frame ranges are at most 2 apart
    fr = lambda i: (i * 64 // tpf, min(i * 64 + 63, S - 1) // tpf)
    for i, j in [(0, 0), (0, 80), (100, 149), (100, 175), (400, 300), (755, 700)]:
        (a0, a1), (b0, b1) = fr(i), fr(j)
        gap = max(b0 - a1, a0 - b1)
        assert bool(win[i, j]) == (gap <= 2)
    assert 0.15 < float(win.float().mean()) < 0.22 and 0.20 < float(tm.float().mean()) < 0.32
    # seeded: same seed same map, different seed different map
    assert torch.equal(tm, layout.local_window_tile_map(S, tpf, seed=0))
    assert not torch.equal(tm, layout.local_window_tile_map(S, tpf, seed=1))


def test_block_mask_csr_roundtrip():
    tm = torch.tensor([[1, 0, 1], [0, 0, 0], [1, 1, 1]], dtype=torch.bool)
    bm = BlockMask.from_dense(tm, device="cpu")
    assert bm.row_ptr.tolist() == [0, 2, 2, 5] and bm.col_idx.tolist() == [0, 2, 0, 1, 2]
    assert bm.row_ptr.dtype == torch.int32 and bm.col_idx.dtype == torch.int32
    empty = BlockMask.from_dense(torch.zeros((2, 2), dtype=torch.bool), device="cpu")
    assert empty.row_ptr.tolist() == [0, 0, 0] and empty.col_idx.numel() >= 1


def test_workload_shapes_on_cpu():
    from pika_h3_flex_amd import workloads

    inp = workloads.self_attention_inputs(frames=2, rows_h=3, rows_w=4, heads=2, audio_latents=5, seed=3, device="cpu")
    assert inp.q.shape == (1, 24 + 10, 2, 128) and inp.q.dtype == torch.bfloat16
    assert inp.position_ids.shape == (34, 3) and not inp.q.is_contiguous() or inp.q.stride(3) == 1
    again = workloads.self_attention_inputs(frames=2, rows_h=3, rows_w=4, heads=2, audio_latents=5, seed=3, device="cpu")
    assert torch.equal(inp.q, again.q) and torch.equal(inp.v, again.v)
    cr = workloads.cross_attention_inputs(q_tokens=40, text_tokens=32, valid_range=(5, 20), heads=2, seed=1, device="cpu")
    n_valid = int(cr.key_mask.sum())
    assert 5 <= n_valid <= 20 and bool(cr.key_mask[0, :n_valid].all()) and not bool(cr.key_mask[0, n_valid:].any())
    assert cr.flops == 4.0 * 40 * n_valid * 128 * 2
    pl = workloads.plumbing_inputs(device="cpu")
    assert pl.q.shape == (1, 1024, 4, 128)


def test_fill_args_validation():
    q = torch.zeros((1, 8, 2, 128), dtype=torch.bfloat16)
    with pytest.raises(TypeError):
        pk.ops.fill_args(q.float(), q, q, q)
    with pytest.raises(ValueError):
        pk.ops.fill_args(q[0], q, q, q)


class _FakeAttn(torch.nn.Module):
    def __init__(self, hidden=256, heads=2):
        super().__init__()
        self.heads = heads
        self.to_q = torch.nn.Linear(hidden, hidden, bias=False)
        self.to_k = torch.nn.Linear(hidden, hidden, bias=False)
        self.to_v = torch.nn.Linear(hidden, hidden, bias=False)
        self.to_out = torch.nn.ModuleList([torch.nn.Linear(hidden, hidden), torch.nn.Identity()])
        self.norm_q = torch.nn.RMSNorm(hidden // heads, eps=1e-6)
        self.norm_k = torch.nn.RMSNorm(hidden // heads, eps=1e-6)


def test_processor_rejects_bad_input_and_host_tensors():
    proc = pk.PikaH3AttnProcessor()
    attn = _FakeAttn().to(torch.bfloat16)
    with pytest.raises(ValueError, match=r"\[B, S, C\]"):
        proc(attn, torch.zeros((4, 256), dtype=torch.bfloat16))
    # on a CPU tensor the processor must fail (no CPU fallback), after running the module's own projections
    with pytest.raises(ValueError, match="device memory"):
        proc(attn, torch.zeros((1, 4, 256), dtype=torch.bfloat16))


def test_key_padding_mask_forms():
    from pika_h3_flex_amd.processor import key_padding_mask

    keep = torch.tensor([[True, True, False, False, True], [True, False, False, False, False]])
    additive = torch.zeros((2, 5)).masked_fill(~keep, float("-inf"))
    assert key_padding_mask(None, 2, 5) is None
    assert torch.equal(key_padding_mask(keep, 2, 5), keep)
    assert torch.equal(key_padding_mask(keep.to(torch.int64), 2, 5), keep)
    assert torch.equal(key_padding_mask(additive, 2, 5), keep)
    assert torch.equal(key_padding_mask(additive.to(torch.bfloat16)[:, None, None, :], 2, 5), keep)
    assert torch.equal(key_padding_mask(torch.where(keep, 0.0, -10000.0)[:, None, :], 2, 5), keep)
    assert torch.equal(key_padding_mask(keep[:1], 2, 5), keep[:1].expand(2, 5))
    with pytest.raises(ValueError, match="queries or heads"):
        key_padding_mask(torch.zeros((2, 4, 7, 5)), 2, 5)
    with pytest.raises(ValueError, match="broadcast form"):
        key_padding_mask(keep, 2, 6)
    # a float mask that is not additive {0, large negative}: a 0/1 keep-mask cast to float would keep every key,
    # a soft bias would be collapsed to keep/drop -- both are refused
    with pytest.raises(ValueError, match="additive"):
        key_padding_mask(keep.to(torch.float32), 2, 5)
    with pytest.raises(ValueError, match="additive"):
        key_padding_mask(torch.full((2, 5), -0.5), 2, 5)
    with pytest.raises(ValueError, match="additive"):
        key_padding_mask(additive.to(torch.bfloat16) + 2.0, 2, 5)
    with pytest.raises(ValueError, match="additive"):
        key_padding_mask(torch.full((2, 5), float("nan")), 2, 5)
    assert torch.equal(key_padding_mask(torch.where(keep, 0.0, -1e3), 2, 5), keep)


def test_fp8_option_forms():
    from pika_h3_flex_amd.ops import fp8_mode

    assert fp8_mode(False) is False and fp8_mode(None) is False and fp8_mode(True) is True and fp8_mode(1) is True
    assert fp8_mode("pow2") == "pow2"
    with pytest.raises(ValueError):
        fp8_mode("e5m2")
