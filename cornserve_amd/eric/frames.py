"""Host side of the uint8-frame input format of the Qwen2-VL family encoders.

The reference's router runs the Hugging Face image processor on the CPU and ships float `pixel_values`
(1176 floats per patch; ModalityProcessor at eric/models/qwen2_5_vl.py:488-512, called from
eric/router/processor.py:46-131).  With this format the router only RESIZES (the processor's `smart_resize` target
size and its PIL bicubic resampling) and ships the uint8 frames, 8x fewer bytes; rescale, normalise and the patch
layout happen on the GPU (`cs_qwen_patchify_u8`), reproducing the processor's float arithmetic exactly through a
table of the 256 byte values per channel.  The router can also ship the frames as decoded: the same resampling then
runs on the GPU (`cs_resize_u8_pass`, Pillow's fixed-point bicubic bit for bit) at the target size computed here.
"""

from __future__ import annotations

import math

import numpy as np
import torch

CLIP_MEAN = (0.48145466, 0.4578275, 0.40821073)   # the processor's defaults (OPENAI_CLIP_MEAN / _STD)
CLIP_STD = (0.26862954, 0.26130258, 0.27577711)


def target_size(height: int, width: int, factor: int = 28, min_pixels: int = 56 * 56,
                max_pixels: int = 14 * 14 * 4 * 1280) -> tuple[int, int]:
    """The processor's `smart_resize`: sides rounded to multiples of `factor`, area clamped to the pixel budget
    with the aspect ratio kept."""
    if max(height, width) / min(height, width) > 200:
        raise ValueError(f"absolute aspect ratio must be smaller than 200, got {max(height, width) / min(height, width)}")
    h, w = round(height / factor) * factor, round(width / factor) * factor
    if h * w > max_pixels:
        shrink = math.sqrt((height * width) / max_pixels)
        h = max(factor, math.floor(height / shrink / factor) * factor)
        w = max(factor, math.floor(width / shrink / factor) * factor)
    elif h * w < min_pixels:
        grow = math.sqrt(min_pixels / (height * width))
        h = math.ceil(height * grow / factor) * factor
        w = math.ceil(width * grow / factor) * factor
    return h, w


def byte_table(mean=CLIP_MEAN, std=CLIP_STD, scale: float = 1 / 255, arithmetic: str = "fused") -> torch.Tensor:
    """fp32 [3,256]: what rescale + normalise make of every byte value per channel, in the processor's arithmetic.

    "fused": the torch processor (mean and std pre-multiplied by 1/scale, one subtract and one divide on the
    float32 byte value); "numpy": the PIL processor (float64 multiply by scale, cast to float32, subtract, divide)."""
    if arithmetic == "fused":
        inv = 1.0 / scale
        m = torch.tensor(mean, dtype=torch.float32) * inv
        s = torch.tensor(std, dtype=torch.float32) * inv
        return ((torch.arange(256, dtype=torch.float32)[None, :] - m[:, None]) / s[:, None]).contiguous()
    if arithmetic == "numpy":
        v = (np.arange(256).astype(np.float64) * scale).astype(np.float32)
        m = np.asarray(mean, dtype=np.float32)
        s = np.asarray(std, dtype=np.float32)
        return torch.from_numpy(((v[None, :] - m[:, None]) / s[:, None]).astype(np.float32))
    raise ValueError(f"unknown arithmetic {arithmetic!r}")


def as_frames(frames) -> np.ndarray:
    """uint8 [H,W,3] or [T,H,W,3] -> contiguous uint8 [T,H,W,3]; anything else is refused."""
    frames = np.asarray(frames)
    if frames.ndim == 3:
        frames = frames[None]
    if frames.dtype != np.uint8 or frames.ndim != 4 or frames.shape[-1] != 3:
        raise ValueError("frames must be uint8 [H,W,3] or [T,H,W,3] (RGB)")
    return np.ascontiguousarray(frames)


def resize_frames(frames: np.ndarray, factor: int = 28, min_pixels: int = 56 * 56,
                  max_pixels: int = 14 * 14 * 4 * 1280) -> np.ndarray:
    """uint8 [H,W,3] or [T,H,W,3] -> uint8 [T,H',W',3] at the processor's target size (PIL bicubic, as the
    processor's PIL backend resamples)."""
    from PIL import Image

    frames = as_frames(frames)
    h, w = target_size(frames.shape[1], frames.shape[2], factor, min_pixels, max_pixels)
    return np.stack([np.asarray(Image.fromarray(f).resize((w, h), resample=Image.Resampling.BICUBIC)) for f in frames])
