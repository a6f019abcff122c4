"""Pins oracle/qwen_preprocess.py (the step before the encoder: resized uint8 frames -> flat pixel_values)."""

import itertools

import numpy as np
import pytest

from oracle import qwen_preprocess as qp


def _rand_frames(t, h, w, seed):
    return np.random.default_rng(seed).integers(0, 256, (t, h, w, 3), dtype=np.uint8)


def _hf_pil_processor():
    mod = pytest.importorskip("transformers.models.qwen2_vl.image_processing_pil_qwen2_vl")
    pytest.importorskip("PIL")
    return mod.Qwen2VLImageProcessorPil()


@pytest.mark.parametrize("h,w", [(56, 84), (448, 448), (28, 140), (252, 1344)])
def test_numpy_arithmetic_and_layout_match_the_package_bit_for_bit(h, w):
    """Sizes that are multiples of 28 inside the pixel budget: the processor's resize keeps every pixel."""
    proc = _hf_pil_processor()
    img = _rand_frames(1, h, w, seed=h * 7 + w)[0]
    out = proc(images=[img], return_tensors="np")
    got, grid = qp.patchify_frames(img[None], qp.normalization_table(arithmetic="numpy"))
    assert tuple(out["image_grid_thw"][0]) == grid == (1, h // 14, w // 14)
    assert out["pixel_values"].dtype == np.float32
    assert np.array_equal(out["pixel_values"], got)


def test_smart_resize_matches_the_package():
    mod = pytest.importorskip("transformers.models.qwen2_vl.image_processing_pil_qwen2_vl")
    rng = np.random.default_rng(0)
    cases = [(1, 1), (27, 29), (28, 28), (5000, 4000), (100, 19000), (3, 600), (1344, 1344), (10000, 10000)]
    cases += [tuple(int(v) for v in rng.integers(1, 6000, 2)) for _ in range(300)]
    for h, w in cases:
        if max(h, w) / min(h, w) > 200:
            with pytest.raises(ValueError):
                qp.smart_resize(h, w)
            continue
        assert qp.smart_resize(h, w) == mod.smart_resize(h, w)
        assert qp.smart_resize(h, w, 28, 3136, 12845056) == mod.smart_resize(h, w, 28, 3136, 12845056)
    hb, wb = qp.smart_resize(5000, 4000)
    assert hb % 28 == 0 and wb % 28 == 0 and hb * wb <= 14 * 14 * 4 * 1280


def test_tables():
    a, b = qp.normalization_table(arithmetic="numpy"), qp.normalization_table(arithmetic="fused")
    assert a.shape == b.shape == (3, 256) and a.dtype == b.dtype == np.float32
    # worked values: byte 0 and byte 255 of the red channel
    assert a[0, 0] == np.float32(-0.48145466) / np.float32(0.26862954)
    assert a[0, 255] == (np.float32(1.0) - np.float32(0.48145466)) / np.float32(0.26862954)
    assert np.all(np.diff(a, axis=1) > 0) and np.all(np.diff(b, axis=1) > 0)          # monotone in the byte value
    # the two arithmetic sequences agree to 2 units in the last place of the largest values ...
    assert np.all(np.abs(a - b) <= 2 * np.spacing(np.float32(2.0)))
    # ... so after the encoder's cast to bfloat16 they agree for (nearly) all byte values
    import torch
    ta, tb = torch.from_numpy(a).bfloat16(), torch.from_numpy(b).bfloat16()
    assert (ta != tb).sum().item() <= 3


def _rn32(x):
    """Round an exact rational to the nearest float32, ties to even -- what one IEEE-754 binary32 operation returns
    for an exact result x -- by exact comparison with the two neighbouring float32 values."""
    from fractions import Fraction

    c = np.float32(float(x))                       # within one float32 ulp of x
    cands = sorted({np.nextafter(c, np.float32(-np.inf)), c, np.nextafter(c, np.float32(np.inf))}, key=float)
    best = min(cands, key=lambda f: (abs(Fraction(float(f)) - x), int(np.float32(f).view(np.uint32)) & 1))
    return np.float32(best)


def test_fused_table_is_the_ieee_evaluation_of_the_published_sequence():
    """The "fused" arithmetic of the torch image processor is four binary32 operations per value -- mean * (1/scale),
    std * (1/scale), u - mean', (.) / std' (transformers `_fuse_mean_std_and_rescale_factor` followed by torchvision's
    normalize: subtract, then divide) -- and IEEE-754 fixes the result of each: the exact value rounded to nearest
    even.  Evaluated with exact rationals and that rounding, every one of the 768 entries must come out bit for bit;
    float64 intermediates, a multiply by the reciprocal or the "numpy" order of operations each change some entry."""
    from fractions import Fraction

    for mean, std in ((qp.OPENAI_CLIP_MEAN, qp.OPENAI_CLIP_STD), ((0.5, 0.5, 0.5), (0.5, 0.5, 0.5))):
        table = qp.normalization_table(mean, std, arithmetic="fused")
        inv = _rn32(Fraction(1.0 / (1 / 255)))     # the Python float 1/scale enters the float32 multiply as float32
        assert inv == np.float32(255.0)
        for c in range(3):
            m = _rn32(Fraction(float(np.float32(mean[c]))) * Fraction(float(inv)))
            s = _rn32(Fraction(float(np.float32(std[c]))) * Fraction(float(inv)))
            for u in range(256):
                d = _rn32(Fraction(u) - Fraction(float(m)))
                want = _rn32(Fraction(float(d)) / Fraction(float(s)))
                assert table[c, u].view(np.uint32) == want.view(np.uint32), (c, u, table[c, u], want)
    # the near-misses this evaluation tells apart from the published sequence
    clip = qp.normalization_table(arithmetic="fused")
    u = np.arange(256, dtype=np.float64)[None, :]
    m64, s64 = np.asarray(qp.OPENAI_CLIP_MEAN, np.float32).astype(np.float64)[:, None], np.asarray(qp.OPENAI_CLIP_STD, np.float32).astype(np.float64)[:, None]
    assert (((u - m64 * 255.0) / (s64 * 255.0)).astype(np.float32) != clip).any()        # float64 intermediates
    assert (qp.normalization_table(arithmetic="numpy") != clip).any()                     # the other order
    # the library's own table (what the GPU kernel looks bytes up in) is the same array
    from cornserve_amd.eric import frames
    assert np.array_equal(frames.byte_table(arithmetic="fused").numpy(), clip)
    assert np.array_equal(frames.byte_table(arithmetic="numpy").numpy(), qp.normalization_table(arithmetic="numpy"))


def _brute_force(frames, table, patch, merge, temporal):
    """Every output element from its definition, with plain index arithmetic (no reshape / transpose)."""
    T, H, W, _ = frames.shape
    gt, gh, gw = -(-T // temporal), H // patch, W // patch
    out = np.zeros((gt * gh * gw, 3 * temporal * patch * patch), np.float32)
    for t, by, bx, my, mx in itertools.product(range(gt), range(gh // merge), range(gw // merge), range(merge), range(merge)):
        row = (((t * (gh // merge) + by) * (gw // merge) + bx) * merge + my) * merge + mx
        for c, tt, py, px in itertools.product(range(3), range(temporal), range(patch), range(patch)):
            f = min(t * temporal + tt, T - 1)
            y, x = (by * merge + my) * patch + py, (bx * merge + mx) * patch + px
            out[row, ((c * temporal + tt) * patch + py) * patch + px] = table[c, frames[f, y, x, c]]
    return out


@pytest.mark.parametrize("t,h,w,patch,merge,temporal", [(1, 8, 12, 2, 2, 2), (3, 8, 4, 2, 2, 2), (4, 12, 12, 2, 3, 2),
                                                        (5, 4, 8, 2, 2, 3), (2, 28, 56, 14, 2, 2)])
def test_layout_against_brute_force(t, h, w, patch, merge, temporal):
    frames = _rand_frames(t, h, w, seed=t + h + w)
    table = qp.normalization_table()
    got, grid = qp.patchify_frames(frames, table, patch, merge, temporal)
    assert grid == (-(-t // temporal), h // patch, w // patch)
    assert np.array_equal(got, _brute_force(frames, table, patch, merge, temporal))


def test_video_of_repeated_frames_is_the_image():
    img = _rand_frames(1, 56, 84, seed=9)
    table = qp.normalization_table()
    one, _ = qp.patchify_frames(img, table)
    vid, grid = qp.patchify_frames(np.repeat(img, 4, axis=0), table)
    assert grid == (2, 4, 6)
    assert np.array_equal(vid[:24], one) and np.array_equal(vid[24:], one)
    odd, grid = qp.patchify_frames(np.repeat(img, 3, axis=0), table)   # 3 frames: the last one is repeated
    assert grid == (2, 4, 6) and np.array_equal(odd, vid)


def test_rejects_bad_input():
    with pytest.raises(ValueError):
        qp.patchify_frames(np.zeros((1, 30, 28, 3), np.uint8), qp.normalization_table())
    with pytest.raises(ValueError):
        qp.patchify_frames(np.zeros((1, 28, 28, 3), np.float32), qp.normalization_table())


def _test_image(kind, h, w, rng):
    if kind == 0:
        return rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    if kind == 1:   # black / white only: the negative lobes overshoot and the clamp at 0 and 255 is exercised
        return (rng.integers(0, 2, (h, w, 3)) * 255).astype(np.uint8)
    return np.clip(np.cumsum(rng.integers(-9, 10, (h, w, 3)), axis=1) + 128, 0, 255).astype(np.uint8)   # smooth


def test_pillow_bicubic_resize_matches_the_package_bit_for_bit():
    Image = pytest.importorskip("PIL.Image")
    rng = np.random.default_rng(11)
    sizes = [tuple(int(v) for v in rng.integers(3, 200, 4)) for _ in range(24)]
    sizes += [(97, 64, 97, 140), (97, 64, 28, 64), (40, 40, 40, 40), (600, 450, 196, 140), (30, 45, 112, 168), (2, 2, 56, 56)]
    for i, (h, w, oh, ow) in enumerate(sizes):
        img = _test_image(i % 3, h, w, rng)
        ref = np.asarray(Image.fromarray(img).resize((ow, oh), resample=Image.Resampling.BICUBIC))
        got = qp.pillow_bicubic_resize(img, oh, ow)
        assert got.shape == ref.shape and np.array_equal(got, ref), (h, w, oh, ow)
    video = _test_image(0, 3 * 50, 70, rng).reshape(3, 50, 70, 3)
    got = qp.pillow_bicubic_resize(video, 84, 112)
    for f, g in zip(video, got):
        assert np.array_equal(g, np.asarray(Image.fromarray(f).resize((112, 84), resample=Image.Resampling.BICUBIC)))


def test_pillow_bicubic_taps_properties():
    """What the construction fixes whatever the package: taps of a position sum to 2^22 within rounding, a pass over a
    constant image returns the constant, and the same size in and out is the identity (centre tap 2^22, others 0)."""
    for a, b in [(100, 37), (37, 100), (1000, 28), (5, 5), (3, 300)]:
        bounds, taps = qp.pillow_bicubic_taps(a, b)
        assert taps.shape[1] == int(np.ceil(2.0 * max(a / b, 1.0))) * 2 + 1
        assert np.all(np.abs(taps.sum(axis=1) - (1 << 22)) <= taps.shape[1])
        assert np.all(bounds[:, 0] >= 0) and np.all(bounds[:, 0] + bounds[:, 1] <= a) and np.all(bounds[:, 1] > 0)
    bounds, taps = qp.pillow_bicubic_taps(5, 5)
    for i in range(5):
        row = np.zeros(5, dtype=np.int64)
        row[bounds[i, 0]:bounds[i, 0] + bounds[i, 1]] = taps[i, :bounds[i, 1]]
        assert row[i] == 1 << 22 and row.sum() == 1 << 22
    flat = np.full((9, 13, 3), 201, dtype=np.uint8)
    assert np.all(qp.pillow_bicubic_resize(flat, 31, 5) == 201)
