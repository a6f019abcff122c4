"""ORACLE (test infrastructure, never on the product path): Qwen2.5-VL vision encoder on the CPU.

A plain-PyTorch restatement of eric/models/qwen2_5_vl.py with the third-party device kernels replaced by
their published definitions:

* patch embed      Conv3d with kernel == stride (:181-201) == F.conv3d on the [L,3,2,14,14] view;
* RMSNorm          eric/models/layers/norm.py:35-70 (fp32 statistics, cast, then weight);
* attention        :86-126; flash_attn_varlen_func (third party, flash-attn 2.7.4.post1, not vendored) is
                   restated as per-segment softmax(q k^T / sqrt(d)) v in fp32 on the stored-precision q,k,v;
* rotary           :26-33; flash_attn.layers.rotary.apply_rotary_emb (non-interleaved) restated as
                   o1 = x1 cos - x2 sin, o2 = x1 sin + x2 cos on fp32 copies, as the reference's own
                   torch version does (eric/models/qwen2_vl.py:131-157);
* MLP              :129-148 (gate/up/down with bias, SiLU);
* merger           :204-233 (RMSNorm, Linear, GELU(erf), Linear);
* forward          :396-485 including the window permutation and its inverse.

`dtype=torch.float32` is the exact-arithmetic form; `dtype=torch.bfloat16` performs every step in bf16
the way the reference does when the model is loaded in bf16 (each op rounds its output), which is the
comparator for the device kernels.  Pinned by tests/test_oracle_models.py against the committed golden
sample tests/golden/qwen2_5_vl_cfg1.npz, which tests/golden/make_golden.py wrote from the installed
third-party Hugging Face implementation of the same network (the reference's own test oracle,
python/tests/task_executors/eric/models/test_qwen2_5_vl.py:63-105), and against closed-form checks of
the pieces (rotary at angle 0, one-token segments, norm of constant rows).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch
import torch.nn.functional as F

from . import vit_index


@dataclass
class QwenVisionConfig:
    depth: int = 32
    hidden_size: int = 1280
    intermediate_size: int = 3420
    num_heads: int = 16
    in_channels: int = 3
    patch_size: int = 14
    temporal_patch_size: int = 2
    spatial_merge_size: int = 2
    window_size: int = 112
    out_hidden_size: int = 3584
    fullatt_block_indexes: list = field(default_factory=lambda: [7, 15, 23, 31])
    rms_norm_eps: float = 1e-6
    hidden_act: str = "silu"


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    orig = x.dtype
    xf = x.to(torch.float32)
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    xf = xf * torch.rsqrt(var + eps)
    return xf.to(orig) * w


def apply_rotary(t: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """t: [L, heads, d]; freqs: [L, d/2] angles."""
    tf = t.float()
    cos = freqs.cos()[:, None, :]
    sin = freqs.sin()[:, None, :]
    half = freqs.shape[-1]
    x1, x2 = tf[..., :half], tf[..., half : 2 * half]
    out = torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos, tf[..., 2 * half :]], dim=-1)
    return out.type_as(t)


def varlen_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens, scale: float) -> torch.Tensor:
    """q,k,v: [L, heads, d]; block-diagonal non-causal attention; fp32 math, output in q.dtype."""
    out = torch.empty_like(q)
    cu = [int(c) for c in cu_seqlens]
    for s, e in zip(cu[:-1], cu[1:]):
        qs = q[s:e].float().transpose(0, 1)
        ks = k[s:e].float().transpose(0, 1)
        vs = v[s:e].float().transpose(0, 1)
        p = torch.softmax(torch.matmul(qs, ks.transpose(1, 2)) * scale, dim=-1)
        out[s:e] = torch.matmul(p, vs).transpose(0, 1).to(q.dtype)
    return out


def rot_pos_emb(cfg: QwenVisionConfig, grid_thw) -> torch.Tensor:
    pos_ids = torch.from_numpy(vit_index.rot_pos_ids(grid_thw, cfg.spatial_merge_size))
    dim = cfg.hidden_size // cfg.num_heads // 2
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))
    max_grid = int(np.asarray(grid_thw).reshape(-1, 3)[:, 1:].max())
    seq = torch.arange(max_grid, dtype=inv_freq.dtype)
    freqs = torch.outer(seq, inv_freq)
    return freqs[pos_ids].flatten(1)  # [L, dim]


def forward(sd: dict, cfg: QwenVisionConfig, pixel_values: list, grid_thw: list, dtype=torch.float32,
            collect: dict | None = None, linear_mode: str = "native") -> list:
    """sd: state dict with the checkpoint's names (after `visual.` is stripped), any float dtype.
    pixel_values: list of [L_i, 1176]; grid_thw: list of [1,3] (or [3]) integer arrays.

    `linear_mode`: "native" runs every linear layer as F.linear in `dtype`; "fp32_accumulate" (meaningful for
    bf16) computes it on fp32 copies of the same bf16 operands and rounds the result to `dtype` once -- the same
    definition (fp32 accumulation, one rounding, as the reference's GEMM library does), evaluated in a different
    summation order.  The distance between the two is what the order of accumulation alone is worth."""
    W = {k: v.to(dtype) for k, v in sd.items()}
    if linear_mode == "native":
        linear = F.linear
    elif linear_mode == "fp32_accumulate":
        def linear(a, w, b=None):
            return F.linear(a.float(), w.float(), None if b is None else b.float()).to(a.dtype)
    else:
        raise ValueError(f"unknown linear_mode {linear_mode}")
    H, nh = cfg.hidden_size, cfg.num_heads
    d = H // nh
    unit = cfg.spatial_merge_size**2
    grid = np.concatenate([np.asarray(g, dtype=np.int64).reshape(-1, 3) for g in grid_thw], axis=0)
    x = torch.cat([p for p in pixel_values], dim=0).to(dtype)
    L = x.shape[0]

    # patch embed (Conv3d, no bias)
    pw = W["patch_embed.proj.weight"]
    x = F.conv3d(x.view(L, cfg.in_channels, cfg.temporal_patch_size, cfg.patch_size, cfg.patch_size), pw,
                 stride=pw.shape[2:]).view(L, H)

    rotary = rot_pos_emb(cfg, grid)
    window_index, cu_window = vit_index.get_window_index(grid, cfg.window_size, cfg.spatial_merge_size,
                                                         cfg.patch_size)
    wi = torch.from_numpy(window_index)
    x = x.reshape(L // unit, unit, -1)[wi].reshape(L, -1)
    rotary = rotary.reshape(L // unit, unit, -1)[wi].reshape(L, -1)
    cu_full = vit_index.full_cu_seqlens(grid)
    if collect is not None:
        collect["embed"] = x.clone()

    for i in range(cfg.depth):
        cu = cu_full if i in cfg.fullatt_block_indexes else cu_window
        p = f"blocks.{i}."
        n1 = rms_norm(x, W[p + "norm1.weight"], cfg.rms_norm_eps)
        qkv = linear(n1, W[p + "attn.qkv.weight"], W[p + "attn.qkv.bias"])
        q, k, v = (t.reshape(L, nh, d) for t in qkv.chunk(3, dim=-1))
        q = apply_rotary(q, rotary)
        k = apply_rotary(k, rotary)
        o = varlen_attention(q, k, v, cu, d**-0.5).reshape(L, H)
        x = x + linear(o, W[p + "attn.proj.weight"], W[p + "attn.proj.bias"])
        n2 = rms_norm(x, W[p + "norm2.weight"], cfg.rms_norm_eps)
        g = F.silu(linear(n2, W[p + "mlp.gate_proj.weight"], W[p + "mlp.gate_proj.bias"]))
        u = linear(n2, W[p + "mlp.up_proj.weight"], W[p + "mlp.up_proj.bias"])
        x = x + linear(g * u, W[p + "mlp.down_proj.weight"], W[p + "mlp.down_proj.bias"])
        if collect is not None:
            collect[f"block{i}"] = x.clone()

    x = rms_norm(x, W["merger.ln_q.weight"], cfg.rms_norm_eps).view(-1, H * unit)
    x = linear(x, W["merger.mlp.0.weight"], W["merger.mlp.0.bias"])
    x = F.gelu(x)
    x = linear(x, W["merger.mlp.2.weight"], W["merger.mlp.2.bias"])
    x = x[torch.argsort(wi)]
    seqlens = (grid[:, 0] * grid[:, 1] * grid[:, 2]) // unit
    return list(x.split([int(s) for s in seqlens], dim=0))


def dequantized_state_dict(sd: dict, linear_keys) -> dict:
    """Config 5 comparator: the same network with fp8-e4m3 weights de-quantised (per-output-channel fp32
    scale amax/448).  The reference has no fp8 path; this is the definition the build tests against."""
    out = dict(sd)
    for k in linear_keys:
        w = sd[k].float()
        w2 = w.reshape(w.shape[0], -1)
        scale = w2.abs().amax(dim=1).clamp_min(1e-12) / 448.0
        q = (w2 / scale[:, None]).to(torch.float8_e4m3fn).float()
        out[k] = (q * scale[:, None]).reshape(w.shape)
    return out
