"""ORACLE (test infrastructure, never on the product path): LLaVA-OneVision vision encoder on the CPU.

A plain-PyTorch restatement of eric/models/llava_onevision.py:

* tower          the SigLIP tower of oracle/gemma3.py built up to `vision_feature_layer`, without the final
                 LayerNorm (layers/vit.py:10-62, llava_onevision.py:46), every token kept ("full", :69-76);
* projector      linear_1 -> act -> linear_2 (:21-37);
* image merge    `_merge_image_patch_embeddings`, strategy "spatial_unpad" (:78-153): tile 0 is the base image;
                 the other tiles form a (tiles_h*side) x (tiles_w*side) grid, the padding that the preprocessor
                 added around the image is cropped, a grid above the token budget ("anyres_max_9") is shrunk by
                 bilinear interpolation, every grid row gets the newline embedding appended;
* video          `apply_pooling` (:169-183): bilinear resize of every frame's side x side grid to
                 ceil(side/2) x ceil(side/2); `_add_image_newline` (:155-167): one newline behind the whole video;
                 the result keeps a leading axis of size 1 (:254-258).

Three helpers live in the third-party package `transformers` (the reference pins 4.57.1), not in the reference's tree,
and are restated here from their published algorithm: `select_best_resolution` (image_processing_utils.py),
`get_anyres_image_grid_shape` and `unpad_image` (models/llava_onevision/modeling_llava_onevision.py).
`torch.nn.functional.interpolate(mode="bilinear", align_corners=False)` is restated as `bilinear_resize`: source
position max(scale*(i+0.5)-0.5, 0) with scale = in/out, two taps per axis, value
(1-ly)*((1-lx)*a00 + lx*a01) + ly*((1-lx)*a10 + lx*a11) in fp32, rounded once to the feature dtype.

Pinned by tests/test_oracle_models.py: the three helpers against the installed package's functions over a sweep of
image sizes; `bilinear_resize` against torch.nn.functional.interpolate in fp32; the whole forward against the
committed golden sample tests/golden/llava_onevision_small.npz, written by tests/golden/make_golden.py from the
installed Hugging Face LlavaOnevisionModel (get_image_features + pack_image_features, get_video_features), and live
against that implementation when it is importable.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch
import torch.nn.functional as F

from . import gemma3 as siglip

MM = "multi_modal_projector."


@dataclass
class LlavaOneVisionConfig:
    vision: siglip.SiglipConfig = field(default_factory=lambda: siglip.SiglipConfig(
        num_hidden_layers=26, image_size=384, hidden_act="gelu_pytorch_tanh"))
    text_hidden_size: int = 3584
    projector_hidden_act: str = "gelu"
    vision_feature_layer: int = -1
    vision_aspect_ratio: str = "anyres_max_9"
    image_grid_pinpoints: list = field(default_factory=lambda: [[384 * i, 384 * j] for i in range(1, 7) for j in range(1, 7)])


def num_tower_layers(cfg: LlavaOneVisionConfig) -> int:
    """layers/vit.py:10-40: a negative feature layer counts from the end, hidden state k is the output of layer k."""
    n = cfg.vision.num_hidden_layers
    return n + cfg.vision_feature_layer + 1 if cfg.vision_feature_layer < 0 else cfg.vision_feature_layer


def select_best_resolution(original_size, possible_resolutions) -> tuple[int, int]:
    oh, ow = original_size
    best, max_eff, min_waste = None, 0, float("inf")
    for h, w in possible_resolutions:
        scale = min(w / ow, h / oh)
        dw, dh = int(ow * scale), int(oh * scale)
        eff = min(dw * dh, ow * oh)
        waste = w * h - eff
        if eff > max_eff or (eff == max_eff and waste < min_waste):
            best, max_eff, min_waste = (h, w), eff, waste
    return best


def anyres_grid_shape(image_size, grid_pinpoints, tile: int) -> tuple[int, int]:
    h, w = select_best_resolution(tuple(int(v) for v in image_size), grid_pinpoints)
    return h // tile, w // tile


def unpad_bounds(cur_h: int, cur_w: int, orig_h: int, orig_w: int) -> tuple[int, int, int, int]:
    """(y0, y1, x0, x1) of the region `unpad_image` keeps of a [*, cur_h, cur_w] grid."""
    if orig_w / orig_h > cur_w / cur_h:
        new_h = int(round(orig_h * (cur_w / orig_w), 7))
        pad = (cur_h - new_h) // 2
        return pad, cur_h - pad, 0, cur_w
    new_w = int(round(orig_w * (cur_h / orig_h), 7))
    pad = (cur_w - new_w) // 2
    return 0, cur_h, pad, cur_w - pad


def bilinear_axis(n_in: int, n_out: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(first tap, second tap, fraction of the second tap) per output position, fp32 arithmetic."""
    scale = torch.tensor(n_in, dtype=torch.float32) / torch.tensor(n_out, dtype=torch.float32)
    pos = scale * (torch.arange(n_out, dtype=torch.float32) + 0.5) - 0.5
    pos = torch.clamp(pos, min=0.0)
    i0 = pos.to(torch.int64)
    i1 = i0 + (i0 < n_in - 1).to(torch.int64)
    return i0, i1, pos - i0.to(torch.float32)


def bilinear_resize(x: torch.Tensor, out_h: int, out_w: int) -> torch.Tensor:
    """x: [C, H, W] -> [C, out_h, out_w], arithmetic in fp32, one rounding to x.dtype."""
    y0, y1, ly = bilinear_axis(x.shape[1], out_h)
    x0, x1, lx = bilinear_axis(x.shape[2], out_w)
    xf = x.float()
    ly, lx = ly[None, :, None], lx[None, None, :]
    hy, hx = 1.0 - ly, 1.0 - lx
    top = hx * xf[:, y0][:, :, x0] + lx * xf[:, y0][:, :, x1]
    bot = hx * xf[:, y1][:, :, x0] + lx * xf[:, y1][:, :, x1]
    return (hy * top + ly * bot).to(x.dtype)


def act_fn(name: str):
    if name == "gelu":
        return F.gelu
    if name == "gelu_pytorch_tanh":
        return lambda x: F.gelu(x, approximate="tanh")
    raise NotImplementedError(name)


def projector(sd: dict, cfg: LlavaOneVisionConfig, feats: torch.Tensor, dtype) -> torch.Tensor:
    h = F.linear(feats, sd[MM + "linear_1.weight"].to(dtype), sd[MM + "linear_1.bias"].to(dtype))
    h = act_fn(cfg.projector_hidden_act)(h)
    return F.linear(h, sd[MM + "linear_2.weight"].to(dtype), sd[MM + "linear_2.bias"].to(dtype))


def merge_image(cfg: LlavaOneVisionConfig, tiles: torch.Tensor, image_size, newline: torch.Tensor) -> torch.Tensor:
    """tiles: [n_tiles, side*side, C] -> [tokens, C]."""
    side = cfg.vision.image_size // cfg.vision.patch_size
    base = tiles[0]
    if side * side != base.shape[0]:
        raise ValueError("The number of patches is not consistent with the image size.")
    if tiles.shape[0] == 1:
        return torch.cat([base, newline[None].to(base.dtype)], dim=0)
    oh, ow = (int(v) for v in image_size)
    th, tw = anyres_grid_shape((oh, ow), cfg.image_grid_pinpoints, cfg.vision.image_size)
    other = tiles[1 : 1 + th * tw].view(th, tw, side, side, -1)
    other = other.permute(4, 0, 2, 1, 3).contiguous().flatten(1, 2).flatten(2, 3)  # [C, th*side, tw*side]
    y0, y1, x0, x1 = unpad_bounds(other.shape[1], other.shape[2], oh, ow)
    other = other[:, y0:y1, x0:x1]
    max_tiles = int(cfg.vision_aspect_ratio.removeprefix("anyres_max_"))
    _, ch, cw = other.shape
    ratio = math.sqrt(ch * cw / (max_tiles * side**2))
    if ratio > 1.1:
        other = bilinear_resize(other, int(ch // ratio), int(cw // ratio))
    other = torch.cat([other, newline.to(other.dtype)[:, None, None].expand(*other.shape[:-1], 1)], dim=-1)
    return torch.cat([base, other.flatten(1, 2).transpose(0, 1)], dim=0)


def pool_video(cfg: LlavaOneVisionConfig, frames: torch.Tensor, newline: torch.Tensor) -> torch.Tensor:
    """frames: [n_frames, side*side, C] -> [1, n_frames * ceil(side/2)^2 + 1, C]."""
    side = cfg.vision.image_size // cfg.vision.patch_size
    n, _, C = frames.shape
    if n == 1:
        # (:254-258 squeezes the frame axis away and the reshape of :162 then misreads the tensor)
        raise RuntimeError("a video of one frame is not supported")
    out_side = math.ceil(side / 2)
    grid = frames.view(n, side, side, C).permute(0, 3, 1, 2)
    pooled = torch.stack([bilinear_resize(g, out_side, out_side) for g in grid])
    pooled = pooled.permute(0, 2, 3, 1).reshape(1, n * out_side * out_side, C)
    return torch.cat([pooled, newline.to(pooled.dtype)[None, None, :]], dim=1)


def features(sd: dict, cfg: LlavaOneVisionConfig, pixel_values: torch.Tensor, dtype) -> torch.Tensor:
    x = siglip.vision_tower(sd, cfg.vision, pixel_values, dtype, num_layers=num_tower_layers(cfg), post_norm=False)
    return projector(sd, cfg, x, dtype)


def forward_images(sd: dict, cfg: LlavaOneVisionConfig, pixel_values: list, image_sizes: list,
                   dtype=torch.float32) -> list:
    feats = features(sd, cfg, torch.cat(list(pixel_values), dim=0), dtype)
    newline = sd["image_newline"].to(dtype)
    per_image = feats.split([int(p.shape[0]) for p in pixel_values])
    return [merge_image(cfg, t, torch.as_tensor(s).reshape(-1).tolist(), newline) for t, s in zip(per_image, image_sizes)]


def forward_videos(sd: dict, cfg: LlavaOneVisionConfig, pixel_values_videos: list, dtype=torch.float32) -> list:
    feats = features(sd, cfg, torch.cat(list(pixel_values_videos), dim=0), dtype)
    newline = sd["image_newline"].to(dtype)
    per_video = feats.split([int(p.shape[0]) for p in pixel_values_videos])
    return [pool_video(cfg, f, newline) for f in per_video]
