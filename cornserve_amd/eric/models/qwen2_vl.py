"""Qwen2-VL vision transformer on the same gfx950 kernels as the Qwen2.5-VL encoder.

Drop-in for `Qwen2VisionTransformer` (reference: eric/models/qwen2_vl.py:294-439): same constructor argument (the
HF config, of which `vision_config` and `rms_norm_eps` are read), the checkpoint's parameter names after `visual.`
is stripped, the same `forward(modality, adapter_name, batch)` contract and output list.

Against its successor this encoder has LayerNorm where that has RMSNorm, a two-layer MLP with QuickGELU where that
has the gated one, and full attention inside every frame in every block (no windows, so no row permutation).  The
forward pass is a fixed sequence of C-ABI launches:

    patch-embed GEMM                                                          :47-51
    per block:  LayerNorm -> QKV GEMM(+bias) -> varlen MFMA attention with rotary fused into the q/k load
                -> proj GEMM(+bias,+residual) -> LayerNorm -> fc1 GEMM(+bias, QuickGELU)
                -> fc2 GEMM(+bias,+residual)                                  :277-291
    merger:     LayerNorm -> GEMM(+bias, GELU) -> GEMM(+bias)                  :75-83
"""

from __future__ import annotations

from typing import Any

import numpy as np
import torch
import torch.nn as nn

from cornserve_amd import ops
from cornserve_amd.eric.models.base import fold_layernorm
from cornserve_amd.eric.models.qwen2_5_vl import (  # noqa: F401  (the processors are this module's too)
    FrameModalityProcessor,
    ModalityProcessor,
    QwenVisionBase,
    _Attn,
    _Linear,
    _no_mark,
    _PatchEmbed,
)


class _LayerNorm(nn.Module):
    def __init__(self, dim: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(dim), requires_grad=False)


class _MLP(nn.Module):
    def __init__(self, dim: int, hidden: int) -> None:
        super().__init__()
        self.fc1 = _Linear(dim, hidden)
        self.fc2 = _Linear(hidden, dim)


class _Block(nn.Module):
    def __init__(self, dim: int, hidden: int) -> None:
        super().__init__()
        self.norm1 = _LayerNorm(dim)
        self.norm2 = _LayerNorm(dim)
        self.attn = _Attn(dim)
        self.mlp = _MLP(dim, hidden)


class _Merger(nn.Module):
    def __init__(self, out_dim: int, context_dim: int, merge: int) -> None:
        super().__init__()
        hidden = context_dim * merge * merge
        self.ln_q = _LayerNorm(context_dim)
        self.mlp = nn.ModuleList([_Linear(hidden, hidden), nn.Identity(), _Linear(hidden, out_dim)])


class Qwen2VisionTransformer(QwenVisionBase):
    def __init__(self, config: Any, weight_format: str = "bf16", fold_norm: bool = False) -> None:
        """`fold_norm`: norm1 / norm2 of every block are applied inside the GEMM that follows them (see
        Qwen2_5_VisionTransformer; here the norms are LayerNorms: the residual GEMMs also emit the row sums).
        Off by default: the folded LayerNorm GEMM exists for the 256x160 tile only, which costs the wide QKV
        projection more than the norm kernels take (measured: 12.82 against 12.77 ms per 8192 patches)."""
        super().__init__()
        vc = config.vision_config if hasattr(config, "vision_config") else config
        if weight_format not in ("bf16", "fp8_e4m3"):
            raise ValueError(f"Unknown weight_format: {weight_format}")
        self.weight_format = weight_format
        E = vc.embed_dim
        hidden = int(vc.embed_dim * vc.mlp_ratio)
        # (the folded forms exist in the direct-to-LDS GEMM only: K a multiple of 64 and at least 192 on both sides)
        self.fold_norm = (bool(fold_norm) and weight_format == "bf16" and E % 64 == 0 and 192 <= E <= 160 * ops.SUMSQ_PARTS
                          and hidden % 64 == 0 and hidden >= 192)
        self.hidden_size = vc.hidden_size          # width of the merger's output (:307)
        self.embed_dim = vc.embed_dim
        self.num_heads = vc.num_heads
        self.mlp_hidden = int(vc.embed_dim * vc.mlp_ratio)
        self.patch_size = vc.patch_size
        self.temporal_patch_size = vc.temporal_patch_size
        self.in_channels = getattr(vc, "in_channels", getattr(vc, "in_chans", 3))
        self.spatial_merge_size = vc.spatial_merge_size
        self.spatial_merge_unit = self.spatial_merge_size**2
        self.norm_eps = getattr(config, "rms_norm_eps", 1e-6)   # the reference reads this name for its LayerNorms (:326-327)
        self.head_dim = self.embed_dim // self.num_heads
        if self.mlp_hidden % 8:
            raise ValueError("the MLP width must be a multiple of 8")

        self.patch_embed = _PatchEmbed(self.in_channels, self.embed_dim, self.temporal_patch_size, self.patch_size)
        self.blocks = nn.ModuleList([_Block(self.embed_dim, self.mlp_hidden) for _ in range(vc.depth)])
        self.merger = _Merger(self.hidden_size, self.embed_dim, self.spatial_merge_size)

    @property
    def chunk_shape(self) -> tuple[int, ...]:
        return (1, self.hidden_size)

    @torch.no_grad()
    def _pack(self) -> dict:
        pk: dict = {"pe_w": self.patch_embed.proj.weight.reshape(self.embed_dim, -1).contiguous()}
        def folded(lin: _Linear, norm: _LayerNorm) -> dict:
            w, b, colsum = fold_layernorm(lin.weight, lin.bias, norm.weight, norm.bias)
            return {"w": w, "s": None, "b": b, "colsum": colsum}

        fold = self.fold_norm
        pk["blocks"] = [
            {
                "n1": (b.norm1.weight, b.norm1.bias),
                "n2": (b.norm2.weight, b.norm2.bias),
                "qkv": folded(b.attn.qkv, b.norm1) if fold else self._lin(b.attn.qkv.weight, b.attn.qkv.bias),
                "proj": self._lin(b.attn.proj.weight, b.attn.proj.bias),
                "fc1": folded(b.mlp.fc1, b.norm2) if fold else self._lin(b.mlp.fc1.weight, b.mlp.fc1.bias),
                "fc2": self._lin(b.mlp.fc2.weight, b.mlp.fc2.bias),
            }
            for b in self.blocks
        ]
        pk["ln_q"] = (self.merger.ln_q.weight, self.merger.ln_q.bias)
        pk["m1"] = self._lin(self.merger.mlp[0].weight, self.merger.mlp[0].bias)
        pk["m2"] = self._lin(self.merger.mlp[2].weight, self.merger.mlp[2].bias)
        dim = self.head_dim // 2
        pk["inv_freq"] = (1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))).to(self.device)
        return pk

    def forward_device(self, pixel_values: torch.Tensor, grid_thw: np.ndarray, mark=None) -> list[torch.Tensor]:
        """pixel_values: bf16 [L, C*T*P*P] already on the device; grid_thw: host int64 [n,3]."""
        if mark is None:
            mark = _no_mark
        pk = self._ensure_packed()
        E, nh, d, unit, dev = self.embed_dim, self.num_heads, self.head_dim, self.spatial_merge_unit, self.device
        eps = self.norm_eps
        if self.fold_norm:   # 32-bit operand offsets in the folded-norm GEMMs: a batch beyond them runs as several
            groups = self._addressable_groups(grid_thw, (2**32 - 1) // (2 * max(3 * E, self.mlp_hidden)))
            if len(groups) > 1:
                return self._forward_in_groups(pixel_values, grid_thw, groups, mark)

        # Rotary table (rot_pos_emb, :354-384) and one attention segment per frame (:423-426).  The index routines
        # are the Qwen2.5-VL ones with a window larger than any grid: one window per frame, i.e. no permutation.
        mark("index")
        merge = self.spatial_merge_size
        no_window = 1 << 20
        sl = ops.vit_seqlens_host(grid_thw, merge, no_window)
        meta = ops.host_to_device(sl.item_meta, dev)
        ix = ops.vit_index(meta, sl.total_patches, sl.max_units_per_item, merge, no_window, pk["inv_freq"])
        plan = ops.attn_plan(sl.cu_full, dev)
        L = sl.total_patches
        if pixel_values.shape[0] != L:
            raise ValueError(f"pixel_values has {pixel_values.shape[0]} rows but grid_thw describes {L} patches")

        mark("patch_embed")
        x = ops.gemm(pixel_values, pk["pe_w"], None)
        n = torch.empty_like(x)
        qkv = torch.empty((L, 3 * E), dtype=torch.bfloat16, device=dev)
        att = torch.empty((L, E), dtype=torch.bfloat16, device=dev)
        hmid = torch.empty((L, self.mlp_hidden), dtype=torch.bfloat16, device=dev)
        scale = d**-0.5
        fold = self.fold_norm
        res = {}
        if self.split_residual:   # the byte plane of the residual stream; zero = "x is exact"
            lo = torch.zeros(x.shape, dtype=torch.uint8, device=dev)
            res = {"residual_lo": lo, "out_lo": lo}
        if fold:
            mark("norm")
            ss = torch.zeros((L, ops.SUMSQ_PARTS), dtype=torch.float32, device=dev)
            sm = torch.zeros_like(ss)
            ops.row_stats(x, ss, sm)
            stats_in = lambda lin: {"a_row_sumsq": ss, "a_row_sum": sm, "w_col_sum": lin["colsum"], "norm_eps": eps}  # noqa: E731
            stats_out = {"c_row_sumsq": ss, "c_row_sum": sm}
        # few rows: each launch names the weights of the launch after next for its idle compute units to read
        hint = L <= self.prefetch_rows
        for i, b in enumerate(pk["blocks"]):
            after = pk["blocks"][i + 1]["qkv"] if i + 1 < len(pk["blocks"]) else pk["m1"]
            after_proj = pk["blocks"][i + 1]["proj"]["w"] if i + 1 < len(pk["blocks"]) else None
            pf_qkv, pf_proj, pf_fc1, pf_fc2 = ((b["fc1"]["w"], b["fc2"]["w"], after["w"], after_proj) if hint
                                               else (None, None, None, None))
            if fold:
                mark("gemm_qkv")
                ops.gemm(x, b["qkv"]["w"], b["qkv"]["b"], out=qkv, prefetch=pf_qkv, **stats_in(b["qkv"]))
            else:
                mark("norm")
                ops.layernorm(x, *b["n1"], eps, out=n)
                mark("gemm_qkv")
                self._g(n, b["qkv"], out=qkv, prefetch=pf_qkv)
            mark("attn_full")
            ops.attn_varlen_rotary_(qkv, plan, nh, d, scale, ix.cos_sin, out=att)
            mark("gemm_proj")
            self._g(att, b["proj"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, prefetch=pf_proj, **res,
                    **(stats_out if fold else {}))
            if fold:
                mark("gemm_fc1")
                ops.gemm(x, b["fc1"]["w"], b["fc1"]["b"], epilogue=ops.EPI_QUICK_GELU, out=hmid, prefetch=pf_fc1,
                         **stats_in(b["fc1"]))
            else:
                mark("norm")
                ops.layernorm(x, *b["n2"], eps, out=n)
                mark("gemm_fc1")
                self._g(n, b["fc1"], epilogue=ops.EPI_QUICK_GELU, out=hmid, prefetch=pf_fc1)
            mark("gemm_fc2")
            self._g(hmid, b["fc2"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, prefetch=pf_fc2, **res,
                    **(stats_out if fold else {}))
        mark("norm")
        ops.layernorm(x, *pk["ln_q"], eps, out=n)
        mark("gemm_merger")
        y = self._g(n.view(L // unit, E * unit), pk["m1"], epilogue=ops.EPI_GELU_ERF)
        out = self._g(y, pk["m2"])
        mark("end")
        g = grid_thw.reshape(-1, 3)
        seqlens = (g[:, 0] * g[:, 1] * g[:, 2]) // unit
        return list(out.split([int(s) for s in seqlens], dim=0))
