"""Packed-sequence formats (CPU only): latents <-> rows by explicit index formulas and round trips, the packed
order and index sets of a document, and the geometry cache."""
import pytest
import torch

from pika_h3_flex_amd import packing as P


def test_video_rows_follow_the_patch_formula():
    B, F, C, H, W = 2, 3, 4, 4, 6
    v = torch.arange(B * F * C * H * W, dtype=torch.float32).reshape(B, F, C, H, W)
    rows = P.video_latents_to_rows(v)
    assert rows.shape == (B, F * (H // 2) * (W // 2), C * 4)
    # brute force: row n = (f, i, j) frame-major then row-major; feature (c*2 + di)*2 + dj
    for b in range(B):
        for f in range(F):
            for i in range(H // 2):
                for j in range(W // 2):
                    n = (f * (H // 2) + i) * (W // 2) + j
                    for c in range(C):
                        for di in range(2):
                            for dj in range(2):
                                assert rows[b, n, (c * 2 + di) * 2 + dj] == v[b, f, c, 2 * i + di, 2 * j + dj]
    assert torch.equal(P.video_rows_to_latents(rows, F, H, W), v)


def test_video_rows_at_benchmark_geometry():
    # 480p: 31 latent frames of 60 x 104 latents -> 31 * 30 * 52 = 48,360 rows of 96 features
    v = torch.zeros(1, 31, P.VIDEO_LATENT_CHANNELS, 60, 104)
    assert P.video_latents_to_rows(v).shape == (1, 48360, 96)


def test_audio_rows_are_channel_major():
    B, T = 2, 5
    a = torch.arange(B * T * 64, dtype=torch.float32).reshape(B, T, 64)
    rows = P.audio_latents_to_rows(a)
    assert rows.shape == (B, 2 * T, 32)
    for b in range(B):
        for ch in range(2):
            for t in range(T):
                assert torch.equal(rows[b, ch * T + t], a[b, t, ch * 32:(ch + 1) * 32])
    assert torch.equal(P.audio_rows_to_latents(rows, T), a)


def test_row_converters_reject_bad_shapes():
    with pytest.raises(ValueError):
        P.video_latents_to_rows(torch.zeros(1, 2, 3, 5, 4))  # odd height
    with pytest.raises(ValueError):
        P.video_latents_to_rows(torch.zeros(2, 3, 4, 4))
    with pytest.raises(ValueError):
        P.audio_latents_to_rows(torch.zeros(1, 4, 63))
    with pytest.raises(ValueError):
        P.video_rows_to_latents(torch.zeros(1, 7, 16), 2, 4, 4)
    with pytest.raises(ValueError):
        P.audio_rows_to_latents(torch.zeros(1, 9, 32), 5)


def test_layout_order_counts_and_indices():
    lay = P.build_layout(num_text_tokens=5, num_latent_frames=3, latent_height=4, latent_width=6,
                         num_audio_latents=7, keyframe_frames=(0, 2), reference_audio_rows=4)
    c = lay.counts
    assert (c.text, c.condition_video, c.condition_audio, c.audio, c.video) == (5, 12, 4, 14, 18)
    assert lay.sequence_length == c.total == 53
    assert lay.position_ids.dtype == torch.float64 and lay.token_tags.dtype == torch.int64
    # packed order: text, condition video, condition audio, audio, video
    assert lay.token_tags.tolist() == [1] * 5 + [0] * 12 + [2] * 4 + [2] * 14 + [0] * 18
    assert lay.text_indices.tolist() == list(range(5))
    # the index sets cover a modality's condition rows first, then its targets (the wrapper concatenates them
    # that way and checks the totals, src/pika_h3/core/wrapper.py:171-179)
    assert lay.audio_indices.tolist() == list(range(17, 35))
    assert lay.video_indices.tolist() == list(range(5, 17)) + list(range(35, 53))
    assert lay.video_indices.numel() == c.condition_video + c.video and lay.audio_indices.numel() == c.condition_audio + c.audio
    every = torch.cat([lay.text_indices, lay.video_indices, lay.audio_indices]).sort().values
    assert every.tolist() == list(range(53))                      # a partition of the rows
    assert lay.num_condition_video_rows == 12 and lay.num_condition_audio_rows == 4 and lay.num_text_tokens == 5
    pos = lay.position_ids
    assert float(pos[:5].abs().sum()) == 0.0                       # text at position 0
    assert set(pos[5:11, 0].tolist()) == {0.0} and set(pos[11:17, 0].tolist()) == {2.0}  # keyframes pin frames 0 and 2
    assert pos[11:17, 1:].tolist() == pos[5:11, 1:].tolist() == [[0, 0], [0, 1], [0, 2], [1, 0], [1, 1], [1, 2]]
    assert pos[21:35, 0].tolist() == list(range(7)) * 2 and float(pos[21:35, 1:].abs().sum()) == 0.0
    assert pos[35].tolist() == [0, 0, 0] and pos[52].tolist() == [2, 1, 2]
    assert lay.rope_row_mask().tolist() == [t != 1 for t in lay.token_tags.tolist()]


def test_joint_benchmark_document_length():
    lay = P.build_layout(num_text_tokens=0, num_latent_frames=31, latent_height=60, latent_width=104, num_audio_latents=640)
    assert lay.sequence_length == 49640 and lay.counts.video == 48360 and lay.counts.audio == 1280


def test_layout_rejects_bad_geometry():
    with pytest.raises(ValueError):
        P.build_layout(num_text_tokens=1, num_latent_frames=2, latent_height=3, latent_width=4, num_audio_latents=0)
    with pytest.raises(ValueError):
        P.build_layout(num_text_tokens=1, num_latent_frames=2, latent_height=4, latent_width=4, num_audio_latents=0,
                       keyframe_frames=(2,))
    with pytest.raises(ValueError):
        P.build_layout(num_text_tokens=-1, num_latent_frames=2, latent_height=4, latent_width=4, num_audio_latents=0)


def test_layout_cache_is_lru_by_geometry():
    cache = P.LayoutCache(capacity=2)
    g = dict(num_text_tokens=3, num_latent_frames=2, latent_height=4, latent_width=4, num_audio_latents=2)
    a = cache.get(**g)
    assert cache.get(**g) is a and (cache.hits, cache.misses) == (1, 1)
    b = cache.get(**{**g, "num_text_tokens": 4})
    assert cache.get(**g) is a                      # a is now the most recent
    cache.get(**{**g, "num_text_tokens": 5})        # evicts b
    assert cache.get(**{**g, "num_text_tokens": 4}) is not b
    assert cache.get(**{**g, "keyframe_frames": [1]}).counts.condition_video == 4


def test_row_timesteps_per_segment():
    """Unique timesteps + per-row index, with the argument list of src/pika_h3/core/packing.py:212-231 and the
    values the wrapper passes (src/pika_h3/core/wrapper.py:182-190)."""
    lay = P.build_layout(num_text_tokens=5, num_latent_frames=3, latent_height=4, latent_width=6,
                         num_audio_latents=7, keyframe_frames=(0, 2), reference_audio_rows=4)
    uniq, idx = P.row_timesteps(lay, video_t=0.25, audio_t=0.5, condition_video_t=max(0.25, 0.75), condition_audio_t=1.0)
    assert uniq.dtype == torch.float32 and idx.dtype == torch.int32 and idx.shape == (53,)
    assert uniq.tolist() == [0.25, 0.5, 0.75, 1.0]
    per_row = uniq[idx.long()].tolist()
    # text (clean), keyframe rows (pinned), condition audio (clean), audio, video
    assert per_row == [1.0] * 5 + [0.75] * 12 + [1.0] * 4 + [0.5] * 14 + [0.25] * 18
    # equal times share one entry: video and audio at the same time, keyframes no noisier than the video
    uniq, idx = P.row_timesteps(lay, video_t=0.5, audio_t=0.5, condition_video_t=0.5)
    assert uniq.tolist() == [0.5, 1.0] and idx.tolist() == [1] * 5 + [0] * 12 + [1] * 4 + [0] * 32
    # the text switch
    uniq, idx = P.row_timesteps(lay, video_t=0.5, audio_t=0.5, condition_video_t=0.5, condition_audio_t=0.5, text_t=0.5)
    assert uniq.tolist() == [0.5] and int(idx.abs().sum()) == 0
