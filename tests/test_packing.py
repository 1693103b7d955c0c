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
    # text (follows the video time, src/pika_h3/core/wrapper.py:22-25), keyframe rows (pinned), condition audio
    # (clean), audio, video
    assert per_row == [0.25] * 5 + [0.75] * 12 + [1.0] * 4 + [0.5] * 14 + [0.25] * 18
    # equal times share one entry: video and audio at the same time, keyframes no noisier than the video
    uniq, idx = P.row_timesteps(lay, video_t=0.5, audio_t=0.5, condition_video_t=0.5)
    assert uniq.tolist() == [0.5, 1.0] and idx.tolist() == [0] * 5 + [0] * 12 + [1] * 4 + [0] * 32
    # the text switch
    uniq, idx = P.row_timesteps(lay, video_t=0.5, audio_t=0.5, condition_video_t=0.5, condition_audio_t=0.5, text_t=1.0)
    assert uniq.tolist() == [0.5, 1.0] and idx.tolist() == [1] * 5 + [0] * 48
    uniq, idx = P.row_timesteps(lay, video_t=0.5, audio_t=0.5, condition_video_t=0.5, condition_audio_t=0.5)
    assert uniq.tolist() == [0.5] and int(idx.abs().sum()) == 0


def test_layout_text_tags_anchors_and_references():
    """Argument list of src/pika_h3/core/packing.py:154-166: prompt tags pass through, "first"/"last" anchors,
    references with their own latent shapes and audio rows; segment sizes as src/pika_h3/core/geometry.py:95-117."""
    tags = torch.tensor([1, 1, 0, 0, 0, 1])          # a vision block inside the prompt (wrapper.py:18)
    lay = P.build_layout(tags, num_latent_frames=3, latent_height=4, latent_width=6, num_audio_latents=2,
                         keyframe_anchors=("first", "last"))
    assert lay.token_tags[:6].tolist() == tags.tolist() and lay.num_text_tokens == 6
    assert lay.counts == P.packed_token_count(num_text_tokens=6, num_latent_frames=3, latent_height=4, latent_width=6,
                                              num_audio_latents=2, num_keyframes=2)
    kf = lay.position_ids[lay.video_indices[:12]]
    assert kf[:6, 0].tolist() == [0.0] * 6 and kf[6:, 0].tolist() == [2.0] * 6
    assert torch.equal(kf[:6, 1:], lay.position_ids[lay.video_indices[12:18], 1:])   # the grid of the pinned frame
    with pytest.raises(ValueError):
        P.build_layout(tags, num_latent_frames=3, latent_height=4, latent_width=6, num_audio_latents=2, keyframe_anchors=("middle",))

    refs = (P.ReferenceSpec("image"), P.ReferenceSpec("video", has_audio=True), P.ReferenceSpec("audio"))
    lay = P.build_layout(num_text_tokens=2, num_latent_frames=3, latent_height=4, latent_width=6, num_audio_latents=2,
                         references=refs, reference_video_shapes=((1, 8, 4), (2, 4, 4)), reference_audio_rows=(6, 4),
                         reference_first_frame=(0.0, 10.0))
    assert lay.counts == P.packed_token_count(num_text_tokens=2, num_latent_frames=3, latent_height=4, latent_width=6,
                                              num_audio_latents=2, reference_video_rows=8 + 8, reference_audio_rows=10)
    assert lay.sequence_length == 2 + 16 + 10 + 4 + 18
    cv = lay.position_ids[lay.video_indices[:16]]
    assert cv[:8, 0].tolist() == [0.0] * 8 and cv[7].tolist() == [0.0, 3.0, 1.0]          # 4 x 2 patches of the image
    assert cv[8:, 0].tolist() == [10.0] * 4 + [11.0] * 4
    ca = lay.position_ids[lay.audio_indices[:10]]
    assert ca[:, 0].tolist() == list(range(6)) + list(range(4)) and float(ca[:, 1:].abs().sum()) == 0
    assert set(lay.token_tags[lay.video_indices].tolist()) == {P.VIDEO_TAG}
    assert set(lay.token_tags[lay.audio_indices].tolist()) == {P.AUDIO_TAG}
    every = torch.cat([lay.text_indices, lay.video_indices, lay.audio_indices]).sort().values
    assert torch.equal(every, torch.arange(lay.sequence_length))
    for bad in (dict(reference_video_shapes=((1, 8, 4),)), dict(reference_audio_rows=(6,)),
                dict(reference_first_frame=(0.0,)), dict(keyframe_anchors=("first",))):
        kw = dict(references=refs, reference_video_shapes=((1, 8, 4), (2, 4, 4)), reference_audio_rows=(6, 4))
        kw.update(bad)
        with pytest.raises(ValueError):
            P.build_layout(num_text_tokens=2, num_latent_frames=3, latent_height=4, latent_width=6, num_audio_latents=2, **kw)


def _document(F=3, H=4, W=6, T=5, L=4):
    g = torch.Generator().manual_seed(3)
    video = torch.randn(1, F, 24, H, W, generator=g)
    audio = torch.randn(1, T, 64, generator=g)
    cond = {"prompt_embeds": torch.randn(L, 16, generator=g), "text_token_tags": torch.ones(1, L, dtype=torch.long)}
    return video, audio, cond, g


def test_prepare_document_keyframes():
    """Mirror of src/pika_h3/core/wrapper.py:96-205 for the first/last-frame task."""
    video, audio, cond, g = _document()
    cond["keyframes"] = [{"anchor": "first", "latents": torch.randn(1, 1, 24, 4, 6, generator=g)},
                         {"anchor": "last", "latents": torch.randn(1, 1, 24, 4, 6, generator=g)}]
    cache = P.LayoutCache()
    mi, tv, ta, ncv, nca = P.prepare_document(video, audio, cond, torch.tensor([0.75]), torch.tensor([[0.5, 0.5]]),
                                              layouts=cache, generator=torch.Generator().manual_seed(1))
    assert (ncv, nca) == (12, 0) and tv.shape == (1, 18, 96) and ta.shape == (1, 10, 32)
    assert set(mi) == {"hidden_states", "audio_hidden_states", "encoder_hidden_states", "timestep", "timestep_indices",
                       "token_tags", "position_ids", "video_indices", "audio_indices", "text_indices", "return_dict"}
    assert mi["hidden_states"].shape == (1, 30, 96) and torch.equal(mi["hidden_states"][:, 12:], tv)
    assert mi["encoder_hidden_states"].shape == (1, 4, 16) and mi["position_ids"].shape == (4 + 12 + 10 + 18, 3)
    # the anchors: t*x0 + (1-t)*eps at t = 0.999, so within 0.1 % noise of the clean rows, and not equal to them
    clean = P.video_latents_to_rows(cond["keyframes"][0]["latents"])
    got = mi["hidden_states"][:, :6]
    assert not torch.equal(got, clean) and float((got - 0.999 * clean).abs().max()) < 0.001 * 6
    # per-row times: text and video at 1 - 0.75, audio at 0.5, anchors pinned at max(0.25, 0.999)
    per_row = mi["timestep"][mi["timestep_indices"].long()]
    want = torch.tensor([0.25] * 4 + [0.999] * 12 + [0.5] * 10 + [0.25] * 18)
    assert torch.allclose(per_row, want) and mi["timestep"].tolist() == sorted(mi["timestep"].tolist())
    # the second denoising step reuses the layout and the same noised anchors
    mi2, *_ = P.prepare_document(video, audio, cond, 0.5, 0.5, layouts=cache)
    assert cache.hits == 1 and torch.equal(mi2["hidden_states"][:, :12], mi["hidden_states"][:, :12])
    assert mi2["timestep"].tolist() == pytest.approx([0.5, 0.999])
    # x0 = x_t + sigma*v on the target rows only
    v = torch.randn(1, 30, 96)
    x0 = P.x0_from_velocity(tv, v, torch.tensor([0.75]), ncv)
    assert torch.allclose(x0, tv + 0.75 * v[:, 12:])
    assert torch.equal(P.video_rows_to_latents(tv, 3, 4, 6), video)
    with pytest.raises(ValueError):
        P.x0_from_velocity(tv, v, 0.75, 0)
    with pytest.raises(ValueError):
        P.prepare_document(video, audio, cond, torch.tensor([[0.1, 0.2]]), 0.5)            # per-frame sigmas differ
    with pytest.raises(ValueError):
        P.prepare_document(video.expand(2, -1, -1, -1, -1), audio, cond, 0.5, 0.5)         # one document per call


def test_prepare_document_references():
    video, audio, cond, g = _document()
    cond["references"] = [{"kind": "image", "video_latents": torch.randn(1, 1, 24, 8, 4, generator=g)},
                          {"kind": "video", "video_latents": torch.randn(1, 2, 24, 4, 4, generator=g),
                           "audio_latents": torch.randn(1, 3, 64, generator=g)},
                          {"kind": "audio", "audio_latents": torch.randn(1, 2, 64, generator=g)}]
    mi, tv, ta, ncv, nca = P.prepare_document(video, audio, cond, 0.5, 0.25)
    assert (ncv, nca) == (8 + 8, 6 + 4)
    assert mi["hidden_states"].shape[1] == ncv + 18 and mi["audio_hidden_states"].shape[1] == nca + 10
    # audio references are packed clean and sit at time 1.0
    assert torch.equal(mi["audio_hidden_states"][:, :6], P.audio_latents_to_rows(cond["references"][1]["audio_latents"]))
    per_row = mi["timestep"][mi["timestep_indices"].long()]
    ai = mi["audio_indices"]
    assert per_row[ai[:nca]].tolist() == [1.0] * nca and per_row[ai[nca:]].tolist() == [0.75] * 10
    assert per_row[mi["video_indices"][:ncv]].tolist() == pytest.approx([0.999] * ncv)


def test_packed_window_tile_map_brute_force():
    """The vectorised map against an explicit per-tile-pair loop over the rows of a document with text, a keyframe,
    audio and video, whose segment boundaries fall inside tiles."""
    lay = P.build_layout(num_text_tokens=37, num_latent_frames=7, latent_height=8, latent_width=12, num_audio_latents=21,
                         keyframe_anchors=("first",))
    S, W = lay.sequence_length, 1
    tm = P.packed_window_tile_map(lay, window_frames=W, global_fraction=0.0)
    nt = (S + 63) // 64
    assert tm.shape == (nt, nt) and tm.dtype == torch.bool
    target = set(lay.video_indices[lay.num_condition_video_rows:].tolist())
    frame = lay.position_ids[:, 0].tolist()
    for i in range(nt):
        for j in range(nt):
            ri, rj = range(i * 64, min(S, i * 64 + 64)), range(j * 64, min(S, j * 64 + 64))
            glob = any(r not in target for r in ri) or any(r not in target for r in rj)
            near = any(abs(frame[a] - frame[b]) <= W for a in ri for b in rj) if not glob else False
            assert bool(tm[i, j]) == (glob or near or i == j), (i, j)
    # every global row sees, and is seen by, everything; a far pair of video tiles is dropped
    first_video_tile = (min(target) + 63) // 64
    assert bool(tm[: first_video_tile].all()) and bool(tm[:, : first_video_tile].all())
    assert not bool(tm[first_video_tile, nt - 1]) and not bool(tm[nt - 1, first_video_tile])
    # symmetric without the random draw; the draw only adds tiles and is seeded
    assert torch.equal(tm, tm.T)
    a = P.packed_window_tile_map(lay, window_frames=W, global_fraction=0.2, seed=5)
    b = P.packed_window_tile_map(lay, window_frames=W, global_fraction=0.2, seed=5)
    assert torch.equal(a, b) and bool((a | ~tm).all()) and int(a.sum()) > int(tm.sum())


def test_packed_window_tile_map_reduces_to_the_video_map():
    """A document of video rows only is the bare grid: the packed map equals layout.local_window_tile_map."""
    from pika_h3_flex_amd import layout as L

    lay = P.build_layout(num_text_tokens=0, num_latent_frames=9, latent_height=6, latent_width=10, num_audio_latents=0)
    per_frame = 3 * 5
    for W in (0, 2):
        got = P.packed_window_tile_map(lay, window_frames=W, global_fraction=0.1, seed=3)
        want = L.local_window_tile_map(lay.sequence_length, per_frame, window_frames=W, global_fraction=0.1, seed=3)
        assert torch.equal(got, want)
    with pytest.raises(ValueError):
        P.packed_window_tile_map(lay, global_fraction=1.5)
