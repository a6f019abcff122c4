"""ORACLE (test infrastructure, never on the product path): Qwen2-VL vision encoder on the CPU.

A plain-PyTorch restatement of eric/models/qwen2_vl.py (the sibling of the Qwen2.5-VL encoder that shares its
patch layout, rotary table and merger, with LayerNorm instead of RMSNorm, a two-layer QuickGELU MLP instead of
the gated one, and full attention per frame in every block instead of windows):

* patch embed      Conv3d with kernel == stride, no bias (:25-51);
* LayerNorm        nn.LayerNorm(eps) with affine parameters (:263-266, :328-330);
* attention        :170-251; rotary as apply_rotary_emb_torch :140-157 (non-interleaved, fp32) on q and k,
                   flash_attn_varlen_func (third party, not vendored) restated as per-segment
                   softmax(q k^T / sqrt(d)) v in fp32 on the stored-precision q, k, v;
* MLP              :112-128: fc2(QuickGELU(fc1(x))), QuickGELU = x * sigmoid(1.702 x) (layers/activations.py:9-12);
* block            :277-291;  merger :54-83 (LayerNorm, Linear, GELU(erf), Linear);
* forward          :386-439: rotary table :354-384, one attention segment per frame (:423-426).

`dtype=torch.float32` is the exact-arithmetic form; `dtype=torch.bfloat16` rounds after every op as the reference
does with a bf16 model.  Pinned by tests/test_oracle_models.py against the committed golden sample
tests/golden/qwen2_vl_small.npz, which tests/golden/make_golden.py wrote from the installed third-party Hugging
Face implementation of the same network (the reference's own test oracle, python/tests/task_executors/eric/models/),
and live against that implementation when it is importable.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch
import torch.nn.functional as F

from . import vit_index
from .qwen2_5_vl import apply_rotary, varlen_attention


@dataclass
class Qwen2VisionConfig:
    depth: int = 32
    embed_dim: int = 1280
    hidden_size: int = 3584          # output width of the merger (the language model's hidden size)
    num_heads: int = 16
    mlp_ratio: float = 4.0
    in_channels: int = 3
    patch_size: int = 14
    temporal_patch_size: int = 2
    spatial_merge_size: int = 2
    norm_eps: float = 1e-6


def quick_gelu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(1.702 * x)


def rotary_angles(cfg: Qwen2VisionConfig, grid: np.ndarray) -> torch.Tensor:
    """[L, head_dim/2] angles: (h, w) position of every patch (2x2-block-major order) times inv_freq."""
    pos_ids = torch.from_numpy(vit_index.rot_pos_ids(grid, cfg.spatial_merge_size))
    dim = cfg.embed_dim // cfg.num_heads // 2
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))
    freqs = torch.outer(torch.arange(int(grid[:, 1:].max()), dtype=inv_freq.dtype), inv_freq)
    return freqs[pos_ids].flatten(1)


def forward(sd: dict, cfg: Qwen2VisionConfig, pixel_values: list, grid_thw: list, dtype=torch.float32,
            collect: dict | None = None) -> list:
    W = {k: v.to(dtype) for k, v in sd.items()}
    E, nh = cfg.embed_dim, cfg.num_heads
    d = E // nh
    unit = cfg.spatial_merge_size**2
    grid = np.concatenate([np.asarray(g, dtype=np.int64).reshape(-1, 3) for g in grid_thw], axis=0)
    x = torch.cat(list(pixel_values), dim=0).to(dtype)
    L = x.shape[0]
    pw = W["patch_embed.proj.weight"]
    x = F.conv3d(x.view(L, cfg.in_channels, cfg.temporal_patch_size, cfg.patch_size, cfg.patch_size), pw,
                 stride=pw.shape[2:]).view(L, E)
    rotary = rotary_angles(cfg, grid)
    cu = vit_index.full_cu_seqlens(grid)
    if collect is not None:
        collect["embed"] = x.clone()
    for i in range(cfg.depth):
        p = f"blocks.{i}."
        n1 = F.layer_norm(x, (E,), W[p + "norm1.weight"], W[p + "norm1.bias"], cfg.norm_eps)
        qkv = F.linear(n1, W[p + "attn.qkv.weight"], W[p + "attn.qkv.bias"])
        q, k, v = (t.reshape(L, nh, d) for t in qkv.chunk(3, dim=-1))
        q, k = apply_rotary(q, rotary), apply_rotary(k, rotary)
        o = varlen_attention(q, k, v, cu, d**-0.5).reshape(L, E)
        x = x + F.linear(o, W[p + "attn.proj.weight"], W[p + "attn.proj.bias"])
        n2 = F.layer_norm(x, (E,), W[p + "norm2.weight"], W[p + "norm2.bias"], cfg.norm_eps)
        h = quick_gelu(F.linear(n2, W[p + "mlp.fc1.weight"], W[p + "mlp.fc1.bias"]))
        x = x + F.linear(h, W[p + "mlp.fc2.weight"], W[p + "mlp.fc2.bias"])
        if collect is not None:
            collect[f"block{i}"] = x.clone()
    x = F.layer_norm(x, (E,), W["merger.ln_q.weight"], W["merger.ln_q.bias"], cfg.norm_eps).view(-1, E * unit)
    x = F.gelu(F.linear(x, W["merger.mlp.0.weight"], W["merger.mlp.0.bias"]))
    x = F.linear(x, W["merger.mlp.2.weight"], W["merger.mlp.2.bias"])
    seqlens = (grid[:, 0] * grid[:, 1] * grid[:, 2]) // unit
    return list(x.split([int(s) for s in seqlens], dim=0))
