"""ORACLE (test infrastructure, never on the product path): the step BEFORE the encoder — resized uint8 frames
to the flat `pixel_values` layout the Qwen2.5-VL encoder consumes.

The reference calls the Hugging Face image processor (`AutoImageProcessor.from_pretrained`, qwen2_5_vl.py:488-512,
run in the router's thread pool, router/processor.py:46-131); the arithmetic lives in the third-party package
`transformers` (the reference pins 4.57.1), not in the reference's tree.  This file restates the published algorithm
of its Qwen2-VL processors:

* `smart_resize`          target size: both sides multiples of patch*merge, area inside [min_pixels, max_pixels]
                          (transformers models/qwen2_vl/image_processing_qwen2_vl.py, `smart_resize`);
* `normalization_table`   what rescale (1/255) followed by normalize (mean, std) makes of each of the 256 byte values,
                          per channel, in the two arithmetic sequences the package has:
                            "numpy"  float32(float64(u) * scale), then (v - mean32) / std32 in float32
                                     (image_transforms.rescale / normalize: the PIL / "slow" processor);
                            "fused"  (float32(u) - mean32 * (1/scale)) / (std32 * (1/scale)) in float32
                                     (`_fuse_mean_std_and_rescale_factor` + torchvision normalize: the "fast" processor,
                                     the default of the pinned version);
* `patchify_frames`       the layout: rows in (t, block-row, block-col, row-in-block, col-in-block) order, columns in
                          (channel, temporal, y, x) order; an image is one frame repeated temporal_patch_size times,
                          a video whose frame count is not a multiple repeats its last frame
                          (image processor `patchify`; video_processing_qwen2_vl.py `patchify`).

Pinned by tests/test_oracle_preprocess.py: `smart_resize` and the "numpy" table + layout bit-for-bit against the
installed package's PIL processor on images whose size needs no resampling; the layout also against an index formula
written independently (brute force over every output element of small cases); videos through the identity "a video
of repeated frames == the image"; the "fused" table entry by entry against an exact-rational evaluation of its four
binary32 operations with IEEE round-to-nearest-even after each (what the standard fixes for that sequence; float64
intermediates or the other order of operations fail it).  PARITY UNPINNED: that torchvision's normalize -- absent here
-- is exactly "subtract, then divide" in float32 (taken from its published source).

* `pillow_bicubic_resize` the resampling the PIL processor applies before all of the above (`image.resize(size,
                          resample=BICUBIC)`): the third-party package Pillow (the reference's pyproject lists it
                          without a version; 12.2.0 is installed here), libImaging/Resample.c: per-axis taps
                          (`precompute_coeffs` with the cubic a = -0.5 filter, `normalize_coeffs_8bpc`: 22 fractional
                          bits) and the two 8-bit passes (`ImagingResampleHorizontal_8bpc`, then
                          `ImagingResampleVertical_8bpc`, a uint8 image between them).  Pinned bit for bit against the
                          installed Pillow itself on random, binary and smooth images over random size pairs (up- and
                          down-scaling, one axis unchanged).  The torch processor resamples with torchvision (absent
                          here, different integer weights): its resampling is PARITY UNPINNED and not restated.
"""

from __future__ import annotations

import math

import numpy as np

OPENAI_CLIP_MEAN = (0.48145466, 0.4578275, 0.40821073)
OPENAI_CLIP_STD = (0.26862954, 0.26130258, 0.27577711)


def smart_resize(height: int, width: int, factor: int = 28, min_pixels: int = 56 * 56,
                 max_pixels: int = 14 * 14 * 4 * 1280) -> tuple[int, int]:
    if max(height, width) / min(height, width) > 200:
        raise ValueError("absolute aspect ratio must be smaller than 200")
    h_bar = round(height / factor) * factor
    w_bar = round(width / factor) * factor
    if h_bar * w_bar > max_pixels:
        beta = math.sqrt((height * width) / max_pixels)
        h_bar = max(factor, math.floor(height / beta / factor) * factor)
        w_bar = max(factor, math.floor(width / beta / factor) * factor)
    elif h_bar * w_bar < min_pixels:
        beta = math.sqrt(min_pixels / (height * width))
        h_bar = math.ceil(height * beta / factor) * factor
        w_bar = math.ceil(width * beta / factor) * factor
    return h_bar, w_bar


def normalization_table(mean=OPENAI_CLIP_MEAN, std=OPENAI_CLIP_STD, scale: float = 1 / 255,
                        arithmetic: str = "fused") -> np.ndarray:
    """float32 [3, 256]: table[c, u] = normalised value of byte u in channel c."""
    u = np.arange(256)
    mean32 = np.asarray(mean, dtype=np.float32)[:, None]
    std32 = np.asarray(std, dtype=np.float32)[:, None]
    if arithmetic == "numpy":
        v = (u.astype(np.float64) * scale).astype(np.float32)[None, :]
        return ((v - mean32) / std32).astype(np.float32)
    if arithmetic == "fused":
        inv = np.float32(1.0 / scale)
        return ((u.astype(np.float32)[None, :] - mean32 * inv) / (std32 * inv)).astype(np.float32)
    raise ValueError(f"unknown arithmetic {arithmetic!r}")


def patchify_frames(frames: np.ndarray, table: np.ndarray, patch: int = 14, merge: int = 2,
                    temporal: int = 2) -> tuple[np.ndarray, tuple[int, int, int]]:
    """frames: uint8 [T, H, W, 3] (already resized: H and W multiples of patch*merge).
    Returns (float32 [grid_t*grid_h*grid_w, 3*temporal*patch*patch], (grid_t, grid_h, grid_w))."""
    frames = np.asarray(frames)
    if frames.dtype != np.uint8 or frames.ndim != 4 or frames.shape[-1] != 3:
        raise ValueError("frames must be uint8 [T, H, W, 3]")
    T, H, W, C = frames.shape
    if H % (patch * merge) or W % (patch * merge) or T < 1:
        raise ValueError("frame size must be a multiple of patch*merge")
    pad = -T % temporal
    if pad:
        frames = np.concatenate([frames, np.repeat(frames[-1:], pad, axis=0)], axis=0)
    grid_t, grid_h, grid_w = (T + pad) // temporal, H // patch, W // patch
    # normalise: channels-first float32 through the per-channel table
    chw = np.stack([table[c][frames[..., c]] for c in range(C)], axis=1)  # [T', C, H, W]
    x = chw.reshape(grid_t, temporal, C, grid_h // merge, merge, patch, grid_w // merge, merge, patch)
    x = x.transpose(0, 3, 6, 4, 7, 2, 1, 5, 8)
    return np.ascontiguousarray(x.reshape(grid_t * grid_h * grid_w, C * temporal * patch * patch)), (grid_t, grid_h, grid_w)


PILLOW_PRECISION_BITS = 32 - 8 - 2


def _cubic(x: float) -> float:
    a = -0.5
    if x < 0.0:
        x = -x
    if x < 1.0:
        return ((a + 2.0) * x - (a + 3.0)) * x * x + 1
    if x < 2.0:
        return (((x - 5) * x + 8) * x - 4) * a
    return 0.0


def pillow_bicubic_taps(in_size: int, out_size: int) -> tuple[np.ndarray, np.ndarray]:
    """(bounds int32 [out_size,2] = (first input position, count), taps int32 [out_size,ksize]) of one axis:
    Resample.c `precompute_coeffs` (doubles, the box [0, in_size) held as floats) + `normalize_coeffs_8bpc`."""
    scale = float(np.float32(in_size) - np.float32(0.0)) / out_size
    filterscale = max(scale, 1.0)
    support = 2.0 * filterscale
    ksize = int(math.ceil(support)) * 2 + 1
    taps = np.zeros((out_size, ksize), dtype=np.int32)
    bounds = np.zeros((out_size, 2), dtype=np.int32)
    inv = 1.0 / filterscale
    for i in range(out_size):
        center = 0.0 + (i + 0.5) * scale
        first = max(int(center - support + 0.5), 0)
        n = max(min(int(center + support + 0.5), in_size) - first, 0)
        w = [_cubic((x + first - center + 0.5) * inv) for x in range(n)]
        total = 0.0
        for v in w:
            total += v
        for x, v in enumerate(w):
            if total != 0.0:
                v = v / total
            taps[i, x] = int(-0.5 + v * (1 << PILLOW_PRECISION_BITS)) if v < 0 else int(0.5 + v * (1 << PILLOW_PRECISION_BITS))
        bounds[i] = (first, n)
    return bounds, taps


def _pillow_pass(img: np.ndarray, out_size: int, axis: int) -> np.ndarray:
    img = np.moveaxis(img, axis, 0)
    bounds, taps = pillow_bicubic_taps(img.shape[0], out_size)
    out = np.empty((out_size,) + img.shape[1:], dtype=np.uint8)
    for i in range(out_size):
        first, n = bounds[i]
        acc = np.tensordot(taps[i, :n].astype(np.int64), img[first:first + n].astype(np.int64), axes=(0, 0))
        acc = (acc + (1 << (PILLOW_PRECISION_BITS - 1))).astype(np.int32)   # the C code accumulates in INT32
        out[i] = np.clip(acc >> PILLOW_PRECISION_BITS, 0, 255)
    return np.moveaxis(out, 0, axis)


def pillow_bicubic_resize(frames: np.ndarray, out_h: int, out_w: int) -> np.ndarray:
    """uint8 [..., H, W, C] -> [..., out_h, out_w, C]: along x first, then along y, an unchanged axis skipped."""
    frames = np.asarray(frames)
    if frames.dtype != np.uint8 or frames.ndim < 3:
        raise ValueError("frames must be uint8 [..., H, W, C]")
    if frames.shape[-2] != out_w:
        frames = _pillow_pass(frames, out_w, frames.ndim - 2)
    if frames.shape[-3] != out_h:
        frames = _pillow_pass(frames, out_h, frames.ndim - 3)
    return frames
