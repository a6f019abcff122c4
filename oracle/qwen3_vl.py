"""ORACLE (test infrastructure, never on the product path): Qwen3-VL vision encoder on the CPU.

A plain-PyTorch restatement of eric/models/qwen3_vl.py:

* patch embed      a Linear with bias on the flat patch rows (:30-86; the checkpoint's Conv3d weight reshaped);
* position embed   `fast_pos_embed_interpolate` (:364-420): bilinear interpolation of the learned
                   num_grid_per_side^2 table at `linspace(0, side-1, h)` x `linspace(0, side-1, w)`, weights cast to
                   the model dtype, weighted rows summed, rows reordered into 2x2-block-major patch order and
                   repeated per frame;
* rotary           :320-362 (position (row, col) of every patch in block-major order times inv_freq), applied
                   as in the Qwen2.5-VL attention module the reference reuses (:126-136);
* block            :111-153: LayerNorm, attention (one segment per frame, :288-291), LayerNorm, fc2(act(fc1));
* mergers          :156-186: the main one normalises the rows (width E) before the 2x2 merge, the deepstack ones
                   (use_postshuffle_norm) normalise the merged rows (width 4E); :300-311: their outputs are
                   concatenated along the feature axis behind the main output.

`dtype=torch.float32` is the exact-arithmetic form; `dtype=torch.bfloat16` rounds after every op as the reference
does with a bf16 model.  Pinned by tests/test_oracle_models.py against the committed golden sample
tests/golden/qwen3_vl_small.npz, which tests/golden/make_golden.py wrote from the installed third-party Hugging
Face implementation of the same network (the reference's own test oracle), live against that implementation when
it is importable, and by closed forms of the interpolation (a grid of the table's own size returns the table; two
points per side return its corners).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
import torch
import torch.nn.functional as F

from . import vit_index
from .qwen2_5_vl import apply_rotary, varlen_attention


@dataclass
class Qwen3VisionConfig:
    depth: int = 27
    hidden_size: int = 1152
    intermediate_size: int = 4304
    num_heads: int = 16
    in_channels: int = 3
    patch_size: int = 16
    temporal_patch_size: int = 2
    spatial_merge_size: int = 2
    out_hidden_size: int = 4096
    num_position_embeddings: int = 2304
    deepstack_visual_indexes: list = field(default_factory=lambda: [8, 16, 24])
    hidden_act: str = "gelu_pytorch_tanh"
    norm_eps: float = 1e-6


def act_fn(name: str):
    if name == "gelu_pytorch_tanh":
        return lambda x: F.gelu(x, approximate="tanh")
    if name == "gelu":
        return F.gelu
    if name == "silu":
        return F.silu
    raise NotImplementedError(name)


def pos_embed_interpolate(table: torch.Tensor, grid: np.ndarray, merge: int) -> torch.Tensor:
    """table: [side*side, E] in the model dtype -> [L, E] position rows in patch order."""
    side = int(math.sqrt(table.shape[0]))
    dtype, E = table.dtype, table.shape[1]
    outs = []
    for t, h, w in grid:
        t, h, w = int(t), int(h), int(w)
        h_idxs = torch.linspace(0, side - 1, h, dtype=torch.float32)
        w_idxs = torch.linspace(0, side - 1, w, dtype=torch.float32)
        h_floor, w_floor = h_idxs.to(torch.long), w_idxs.to(torch.long)
        h_ceil = torch.clamp(h_floor + 1, max=side - 1)
        w_ceil = torch.clamp(w_floor + 1, max=side - 1)
        dh, dw = h_idxs - h_floor, w_idxs - w_floor
        dh_g, dw_g = torch.meshgrid(dh, dw, indexing="ij")
        hf_g, wf_g = torch.meshgrid(h_floor, w_floor, indexing="ij")
        hc_g, wc_g = torch.meshgrid(h_ceil, w_ceil, indexing="ij")
        w11 = dh_g * dw_g
        w10 = dh_g - w11
        w01 = dw_g - w11
        w00 = 1 - dh_g - dw_g + w11
        idx = torch.stack([hf_g * side + wf_g, hf_g * side + wc_g, hc_g * side + wf_g, hc_g * side + wc_g]).reshape(4, -1)
        weights = torch.stack([w00, w01, w10, w11]).reshape(4, -1, 1).to(dtype)
        combined = (table[idx] * weights).sum(dim=0).view(h * w, E)
        rep = combined.unsqueeze(0).expand(t, -1, -1).contiguous()
        rep = rep.view(t, h // merge, merge, w // merge, merge, E).permute(0, 1, 3, 2, 4, 5).reshape(-1, E)
        outs.append(rep)
    return torch.cat(outs, dim=0)


def rotary_angles(cfg: Qwen3VisionConfig, grid: np.ndarray) -> torch.Tensor:
    pos_ids = torch.from_numpy(vit_index.rot_pos_ids(grid, cfg.spatial_merge_size))
    dim = cfg.hidden_size // cfg.num_heads // 2
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))
    freqs = torch.outer(torch.arange(int(grid[:, 1:].max()), dtype=inv_freq.dtype), inv_freq)
    return freqs[pos_ids].flatten(1)


def _merger(W: dict, prefix: str, x: torch.Tensor, E: int, unit: int, eps: float, postshuffle: bool) -> torch.Tensor:
    if postshuffle:
        x = F.layer_norm(x.view(-1, E * unit), (E * unit,), W[prefix + "norm.weight"], W[prefix + "norm.bias"], eps)
    else:
        x = F.layer_norm(x, (E,), W[prefix + "norm.weight"], W[prefix + "norm.bias"], eps).view(-1, E * unit)
    x = F.gelu(F.linear(x, W[prefix + "linear_fc1.weight"], W[prefix + "linear_fc1.bias"]))
    return F.linear(x, W[prefix + "linear_fc2.weight"], W[prefix + "linear_fc2.bias"])


def forward(sd: dict, cfg: Qwen3VisionConfig, pixel_values: list, grid_thw: list, dtype=torch.float32,
            collect: dict | None = None) -> list:
    W = {k: v.to(dtype) for k, v in sd.items()}
    E, nh = cfg.hidden_size, cfg.num_heads
    d = E // nh
    unit = cfg.spatial_merge_size**2
    act = act_fn(cfg.hidden_act)
    grid = np.concatenate([np.asarray(g, dtype=np.int64).reshape(-1, 3) for g in grid_thw], axis=0)
    x = torch.cat(list(pixel_values), dim=0).to(dtype)
    L = x.shape[0]
    x = F.linear(x, W["patch_embed.proj.weight"].reshape(E, -1), W["patch_embed.proj.bias"])
    x = x + pos_embed_interpolate(W["pos_embed.weight"], grid, cfg.spatial_merge_size)
    rotary = rotary_angles(cfg, grid)
    cu = vit_index.full_cu_seqlens(grid)
    if collect is not None:
        collect["embed"] = x.clone()
    kept = []
    for i in range(cfg.depth):
        p = f"blocks.{i}."
        n1 = F.layer_norm(x, (E,), W[p + "norm1.weight"], W[p + "norm1.bias"], cfg.norm_eps)
        qkv = F.linear(n1, W[p + "attn.qkv.weight"], W[p + "attn.qkv.bias"])
        q, k, v = (t.reshape(L, nh, d) for t in qkv.chunk(3, dim=-1))
        q, k = apply_rotary(q, rotary), apply_rotary(k, rotary)
        o = varlen_attention(q, k, v, cu, d**-0.5).reshape(L, E)
        x = x + F.linear(o, W[p + "attn.proj.weight"], W[p + "attn.proj.bias"])
        n2 = F.layer_norm(x, (E,), W[p + "norm2.weight"], W[p + "norm2.bias"], cfg.norm_eps)
        h = act(F.linear(n2, W[p + "mlp.linear_fc1.weight"], W[p + "mlp.linear_fc1.bias"]))
        x = x + F.linear(h, W[p + "mlp.linear_fc2.weight"], W[p + "mlp.linear_fc2.bias"])
        if i in cfg.deepstack_visual_indexes:
            kept.append(x)
        if collect is not None:
            collect[f"block{i}"] = x.clone()
    outs = [_merger(W, "merger.", x, E, unit, cfg.norm_eps, False)]
    for j, hs in enumerate(kept):
        outs.append(_merger(W, f"deepstack_merger_list.{j}.", hs, E, unit, cfg.norm_eps, True))
    y = torch.cat(outs, dim=1)
    seqlens = (grid[:, 0] * grid[:, 1] * grid[:, 2]) // unit
    return list(y.split([int(s) for s in seqlens], dim=0))
