"""LLaVA-OneVision vision encoder (SigLIP tower + two-layer projector + anyres merge) on hand-written gfx950 kernels.

Drop-in for `LlavaOneVisionEncoder` (reference: eric/models/llava_onevision.py:40-285).  Parameter names follow the
checkpoint (`vision_tower.vision_model....`, `multi_modal_projector.linear_{1,2}`, `image_newline`).

Forward = the SigLIP tower's launch sequence (built up to `vision_feature_layer`, no final LayerNorm; layers/vit.py:43-62),
two GEMMs for the projector, and ONE weighted row gather that replaces the reference's view / permute / crop /
interpolate / concatenate program (:78-183): the host turns each item's geometry into, per output row, four source rows
and two interpolation fractions, and `cs_rows_bilinear` writes every item's sequence in one launch.  The newline
embedding is kept as one extra row behind the projector's output so that the same gather places it.
"""

from __future__ import annotations

import math
from collections.abc import Callable
from typing import Any

import numpy as np
import torch
import torch.nn as nn

from cornserve_amd import ops
from cornserve_amd.eric.api import Modality
from cornserve_amd.eric.models.base import BaseModalityProcessor
from cornserve_amd.eric.models.gemma3 import SiglipEncoderBase, SiglipVisionModel
from cornserve_amd.eric.models.qwen2_5_vl import _Linear


# ---- geometry (host side) ---------------------------------------------------------------------------------------
def select_best_resolution(original_size: tuple[int, int], possible_resolutions: list) -> tuple[int, int]:
    """The (height, width) among `possible_resolutions` that keeps most of the image after downscaling and wastes
    least (transformers image_processing_utils.select_best_resolution, which the reference reaches through
    get_anyres_image_grid_shape, llava_onevision.py:102-106)."""
    oh, ow = original_size
    best, max_eff, min_waste = None, 0, float("inf")
    for h, w in possible_resolutions:
        scale = min(w / ow, h / oh)
        eff = min(int(ow * scale) * int(oh * scale), ow * oh)
        waste = w * h - eff
        if eff > max_eff or (eff == max_eff and waste < min_waste):
            best, max_eff, min_waste = (h, w), eff, waste
    return best


def anyres_grid_shape(image_size: tuple[int, int], grid_pinpoints: list, tile: int) -> tuple[int, int]:
    """(tiles along the height, tiles along the width) of the grid the preprocessor cut the image into."""
    if not isinstance(grid_pinpoints, list):
        raise TypeError("grid_pinpoints should be a list of tuples or lists")
    h, w = select_best_resolution((int(image_size[0]), int(image_size[1])), grid_pinpoints)
    return h // tile, w // tile


def _unpad_bounds(cur_h: int, cur_w: int, orig_h: int, orig_w: int) -> tuple[int, int, int, int]:
    """Rows and columns that `unpad_image` (llava_onevision.py:121) keeps of a cur_h x cur_w grid."""
    if orig_w / orig_h > cur_w / cur_h:
        new_h = int(round(orig_h * (cur_w / orig_w), 7))
        pad = (cur_h - new_h) // 2
        return pad, cur_h - pad, 0, cur_w
    new_w = int(round(orig_w * (cur_h / orig_h), 7))
    pad = (cur_w - new_w) // 2
    return 0, cur_h, pad, cur_w - pad


def _bilinear_axis(n_in: int, n_out: int) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """torch's bilinear resize along one axis (align_corners=False): first tap, second tap, fraction (fp32)."""
    scale = np.float32(n_in) / np.float32(n_out)
    pos = scale * (np.arange(n_out, dtype=np.float32) + np.float32(0.5)) - np.float32(0.5)
    pos = np.maximum(pos, np.float32(0.0)).astype(np.float32)
    i0 = pos.astype(np.int64)
    i1 = i0 + (i0 < n_in - 1)
    return i0, i1, (pos - i0.astype(np.float32)).astype(np.float32)


def _resize_taps(rows: np.ndarray, out_h: int, out_w: int) -> tuple[np.ndarray, np.ndarray]:
    """rows: [h, w] source row of every grid position -> taps [out_h*out_w, 4], frac [out_h*out_w, 2]."""
    y0, y1, ly = _bilinear_axis(rows.shape[0], out_h)
    x0, x1, lx = _bilinear_axis(rows.shape[1], out_w)
    taps = np.stack([rows[y0][:, x0], rows[y0][:, x1], rows[y1][:, x0], rows[y1][:, x1]], axis=-1)
    frac = np.stack(np.broadcast_arrays(ly[:, None], lx[None, :]), axis=-1)
    return taps.reshape(-1, 4), frac.reshape(-1, 2)


def _copy_taps(rows: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    rows = rows.reshape(-1)
    return np.repeat(rows[:, None], 4, axis=1), np.zeros((rows.size, 2), dtype=np.float32)


def image_merge_plan(n_tiles: int, image_size: tuple[int, int], first_row: int, newline_row: int, side: int,
                     grid_pinpoints: list, tile_px: int, vision_aspect_ratio: str = "anyres_max_9",
                     tokens_per_tile: int | None = None) -> tuple[np.ndarray, np.ndarray]:
    """Gather records of one image (strategy "spatial_unpad", llava_onevision.py:78-153): `first_row` is the row of
    the image's first token in the projector's output, tiles follow each other with `side*side` rows each."""
    per = side * side
    if (per if tokens_per_tile is None else tokens_per_tile) != per:
        raise ValueError("The number of patches is not consistent with the image size.")
    base = first_row + np.arange(per, dtype=np.int64)
    if n_tiles == 1:
        taps, frac = _copy_taps(np.concatenate([base, [newline_row]]))
        return taps, frac
    oh, ow = int(image_size[0]), int(image_size[1])
    th, tw = anyres_grid_shape((oh, ow), grid_pinpoints, tile_px)
    if th * tw > n_tiles - 1:
        raise RuntimeError(f"an image of size {(oh, ow)} needs {th * tw} tiles next to the base tile, got {n_tiles - 1}")
    # row of grid position (Y, X): tile (Y // side, X // side), patch (Y % side, X % side)
    Y, X = np.meshgrid(np.arange(th * side), np.arange(tw * side), indexing="ij")
    grid = first_row + (1 + (Y // side) * tw + (X // side)) * per + (Y % side) * side + (X % side)
    y0, y1, x0, x1 = _unpad_bounds(th * side, tw * side, oh, ow)
    grid = grid[y0:y1, x0:x1]
    ch, cw = grid.shape
    max_tiles = int(vision_aspect_ratio.removeprefix("anyres_max_"))
    ratio = math.sqrt(ch * cw / (max_tiles * side**2))
    if ratio > 1.1:
        out_h, out_w = int(ch // ratio), int(cw // ratio)
        taps, frac = _resize_taps(grid, out_h, out_w)
    else:
        out_h, out_w = ch, cw
        taps, frac = _copy_taps(grid)
    # one newline behind every row of the grid
    taps = np.concatenate([taps.reshape(out_h, out_w, 4), np.full((out_h, 1, 4), newline_row, dtype=np.int64)], axis=1)
    frac = np.concatenate([frac.reshape(out_h, out_w, 2), np.zeros((out_h, 1, 2), dtype=np.float32)], axis=1)
    bt, bf = _copy_taps(base)
    return np.concatenate([bt, taps.reshape(-1, 4)]), np.concatenate([bf, frac.reshape(-1, 2)])


def video_pool_plan(n_frames: int, first_row: int, newline_row: int, side: int) -> tuple[np.ndarray, np.ndarray]:
    """Gather records of one video (llava_onevision.py:155-183): every frame's side x side grid resized to
    ceil(side/2) squared, one newline behind the last frame."""
    out_side = math.ceil(side / 2)
    taps, frac = [], []
    for f in range(n_frames):
        rows = first_row + f * side * side + np.arange(side * side, dtype=np.int64).reshape(side, side)
        t, fr = _resize_taps(rows, out_side, out_side)
        taps.append(t)
        frac.append(fr)
    t, fr = _copy_taps(np.array([newline_row], dtype=np.int64))
    return np.concatenate(taps + [t]), np.concatenate(frac + [fr])


# ---- modules ----------------------------------------------------------------------------------------------------
class LlavaOneVisionMultiModalProjector(nn.Module):
    """linear_1 -> activation -> linear_2 (reference: llava_onevision.py:21-37); run by the encoder's forward."""

    def __init__(self, config: Any) -> None:
        super().__init__()
        bias = getattr(config, "multimodal_projector_bias", True)
        self.linear_1 = _Linear(config.vision_config.hidden_size, config.text_config.hidden_size, bias=bias)
        self.linear_2 = _Linear(config.text_config.hidden_size, config.text_config.hidden_size, bias=bias)


def _num_tower_layers(config: Any) -> int:
    """Layers needed for `vision_feature_layer` (reference: layers/vit.py:10-40)."""
    total = config.vision_config.num_hidden_layers
    feature = config.vision_feature_layer
    if isinstance(feature, int):
        layers = [feature]
    elif isinstance(feature, (list, tuple)):
        layers = list(feature)
    else:
        raise TypeError(f"vision_layer_feature type: {type(feature)} is not supported")
    return max(total + f + 1 if f < 0 else f for f in layers)


class LlavaOneVisionEncoder(SiglipEncoderBase):
    def __init__(self, config: Any, fold_norm: bool = False) -> None:
        """`fold_norm`: see Gemma3VisionEncoder (the same tower): off by default."""
        super().__init__()
        self.config = config
        self.vision_tower = SiglipVisionModel(config.vision_config, num_hidden_layers_override=_num_tower_layers(config),
                                              require_post_norm=False)
        self.multi_modal_projector = LlavaOneVisionMultiModalProjector(config)
        self.image_newline = nn.Parameter(torch.empty(config.text_config.hidden_size), requires_grad=False)
        act = config.projector_hidden_act
        if act == "gelu":
            self._proj_epi = ops.EPI_GELU_ERF
        elif act == "gelu_pytorch_tanh":
            self._proj_epi = ops.EPI_GELU_TANH
        elif act == "quick_gelu":
            self._proj_epi = ops.EPI_QUICK_GELU
        else:
            raise NotImplementedError(f"Activation function {act!r} is not implemented.")
        self._init_tower(fold_norm)

    @property
    def dtype(self) -> torch.dtype:
        return self.multi_modal_projector.linear_1.weight.dtype

    @property
    def device(self) -> torch.device:
        return self.multi_modal_projector.linear_1.weight.device

    @property
    def chunk_shape(self) -> tuple[int, ...]:
        # Tiles are merged into sequences of varying length, so a chunk is one token (reference: :55-63).
        return (1, self.config.text_config.hidden_size)

    def _side(self) -> int:
        vc = self.config.vision_config
        return vc.image_size // vc.patch_size

    def _projected(self, pixel_values: list[torch.Tensor]) -> torch.Tensor:
        """Tower + projector over all tiles of the batch: bf16 [tiles*tokens + 1, T]; the last row is the newline."""
        strategy = self.config.vision_feature_select_strategy
        if strategy not in ("default", "full"):
            raise ValueError(f"Unexpected select feature strategy: {strategy}")
        stacked = ops.cat_to_device(pixel_values, self.device, self.dtype)
        feats = self.vision_tower_forward(stacked)            # [tiles, tokens, H]
        if strategy == "default":
            feats = feats[:, 1:].contiguous()
        M = feats.shape[0] * feats.shape[1]
        mp = self.multi_modal_projector
        T = self.config.text_config.hidden_size
        hidden = ops.gemm(feats.view(M, -1), mp.linear_1.weight, mp.linear_1.bias, epilogue=self._proj_epi)
        out = torch.empty((M + 1, T), dtype=torch.bfloat16, device=self.device)
        ops.gemm(hidden, mp.linear_2.weight, mp.linear_2.bias, out=out[:M])
        out[M].copy_(self.image_newline)
        return out

    def _gather(self, projected: torch.Tensor, plans: list[tuple[np.ndarray, np.ndarray]]) -> list[torch.Tensor]:
        taps = np.concatenate([p[0] for p in plans]).astype(np.int32)
        frac = np.concatenate([p[1] for p in plans]).astype(np.float32)
        merged = ops.rows_bilinear(projected, ops.host_to_device(taps, self.device),
                                   ops.host_to_device(frac, self.device))
        return list(merged.split([p[0].shape[0] for p in plans]))

    def _check_pixels(self, items: list[torch.Tensor]) -> None:
        size = self.config.vision_config.image_size
        assert isinstance(items, list)
        for item in items:
            assert isinstance(item, torch.Tensor)
            assert item.ndim == 4
            assert item.shape[1] == 3
            assert item.shape[2] == item.shape[3] == size

    def get_image_embeddings(self, pixel_values: list[torch.Tensor], image_sizes: list[torch.Tensor]) -> list[torch.Tensor]:
        """Reference: llava_onevision.py:185-227."""
        assert isinstance(image_sizes, list)
        assert len(pixel_values) == len(image_sizes)
        self._check_pixels(pixel_values)
        for item in image_sizes:
            assert isinstance(item, torch.Tensor)
        side, per = self._side(), self._side() ** 2
        tokens = per - (1 if self.config.vision_feature_select_strategy == "default" else 0)
        total_tiles = sum(int(p.shape[0]) for p in pixel_values)
        newline_row = total_tiles * tokens
        plans, first = [], 0
        for px, size in zip(pixel_values, image_sizes):
            hw = [int(v) for v in size.reshape(-1).tolist()]
            plans.append(image_merge_plan(int(px.shape[0]), (hw[0], hw[1]), first, newline_row, side,
                                          self.config.image_grid_pinpoints, self.config.vision_config.image_size,
                                          getattr(self.config, "vision_aspect_ratio", "anyres_max_9"),
                                          tokens_per_tile=tokens))
            first += int(px.shape[0]) * tokens
        return self._gather(self._projected(pixel_values), plans)

    def get_video_embeddings(self, pixel_values_videos: list[torch.Tensor]) -> list[torch.Tensor]:
        """Reference: llava_onevision.py:229-258; every result keeps the reference's leading axis of size 1."""
        self._check_pixels(pixel_values_videos)
        side = self._side()
        if self.config.vision_feature_select_strategy != "full":
            raise RuntimeError("video pooling needs every token of a frame (vision_feature_select_strategy='full')")
        for px in pixel_values_videos:
            if px.shape[0] == 1:
                # the reference squeezes the frame axis of a one-frame video away and its reshape then fails (:162, :257)
                raise RuntimeError("a video of one frame is not supported")
        newline_row = sum(int(p.shape[0]) for p in pixel_values_videos) * side * side
        plans, first = [], 0
        for px in pixel_values_videos:
            plans.append(video_pool_plan(int(px.shape[0]), first, newline_row, side))
            first += int(px.shape[0]) * side * side
        return [v.unsqueeze(0) for v in self._gather(self._projected(pixel_values_videos), plans)]

    @torch.inference_mode()
    def forward(self, modality: Modality, adapter_name: str, batch: dict[str, list[torch.Tensor]]) -> list[torch.Tensor]:
        """Images: `pixel_values` (each [tiles, 3, S, S]) and `image_sizes` (each [2]: height, width of the original);
        videos: `pixel_values_videos` (each [frames, 3, S, S]).  Reference: llava_onevision.py:260-285."""
        match modality:
            case Modality.IMAGE:
                return self.get_image_embeddings(batch["pixel_values"], batch["image_sizes"])
            case Modality.VIDEO:
                return self.get_video_embeddings(batch["pixel_values_videos"])
            case _:
                raise ValueError(f"Unsupported modality: {modality}.")


class ModalityProcessor(BaseModalityProcessor):
    """LLaVA-OneVision modality processor (reference: llava_onevision.py:288-318); needs the model files locally."""

    def __init__(self, model_id: str) -> None:
        super().__init__(model_id=model_id)
        from transformers import AutoProcessor  # deferred

        hf_processor = AutoProcessor.from_pretrained(model_id)
        self.image_processor = hf_processor.image_processor
        self.video_processor = hf_processor.video_processor

    def get_image_processor(self) -> Callable | None:
        def processor(image) -> dict[str, torch.Tensor]:
            out = self.image_processor.preprocess(images=[image], return_tensors="pt")
            return {k: v.squeeze(0) for k, v in out.data.items()}  # batch size is 1

        return processor

    def get_video_processor(self) -> Callable | None:
        def processor(video) -> dict[str, torch.Tensor]:
            out = self.video_processor.preprocess(videos=[video], return_tensors="pt")
            return {k: v.squeeze(0) for k, v in out.data.items()}

        return processor
