"""Qwen3-VL vision transformer on the same gfx950 kernels as the other Qwen encoders.

Drop-in for `Qwen3_VisionTransformer` (reference: eric/models/qwen3_vl.py:189-420): same constructor argument (the HF
config, of which `vision_config` is read), the checkpoint's parameter names after `visual.` is stripped (the patch
embedding accepts the checkpoint's Conv3d-shaped weight), the same `forward(modality, adapter_name, batch)` contract
and output list: per item `[tokens, out_hidden_size * (1 + number of deepstack layers)]`.

The forward pass is a fixed sequence of C-ABI launches:

    position rows: bilinear interpolation of the learned table, in patch order      :364-420  cs_pos_embed_interp
    patch-embed GEMM (+bias, + position rows in the epilogue)                        :85-86, :283-284
    per block:  LayerNorm -> QKV GEMM(+bias) -> rotary on q and k in place -> varlen MFMA attention (one segment per
                frame) -> proj GEMM(+bias,+residual) -> LayerNorm -> fc1 GEMM(+bias, GELU tanh)
                -> fc2 GEMM(+bias,+residual)                                          :139-153
    mergers:    LayerNorm (per row for the main merger, per merged row for the deepstack ones) -> GEMM(+bias, GELU)
                -> GEMM(+bias) straight into its column block of the output           :176-186, :300-311

The head dimension is 72: its rotary halves (36) are not multiples of the 8-element chunks the attention kernel
rotates while staging, so rotary runs as its own in-place kernel and attention takes the direct-to-LDS path.
"""

from __future__ import annotations

import math
from collections.abc import Callable
from typing import Any

import numpy as np
import torch
import torch.nn as nn

from cornserve_amd import ops
from cornserve_amd.eric.models.base import BaseModalityProcessor, fold_layernorm
from cornserve_amd.eric.models.qwen2_5_vl import FrameModalityProcessor, QwenVisionBase, _Attn, _Linear, _no_mark  # noqa: F401
from cornserve_amd.eric.models.qwen2_vl import _LayerNorm

_ACTIVATIONS = {"gelu_pytorch_tanh": ops.EPI_GELU_TANH, "gelu": ops.EPI_GELU_ERF, "quick_gelu": ops.EPI_QUICK_GELU}


class _PatchLinear(nn.Module):
    """Linear patch embedding with bias (:30-86); takes the checkpoint's Conv3d-shaped weight [E, C, T, P, P]."""

    def __init__(self, in_dim: int, embed_dim: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(embed_dim, in_dim), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(embed_dim), requires_grad=False)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        key = prefix + "weight"
        if key in state_dict and state_dict[key].dim() == 5:
            state_dict[key] = state_dict[key].reshape(state_dict[key].shape[0], -1)
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)


class _PatchEmbed(nn.Module):
    def __init__(self, in_dim: int, embed_dim: int) -> None:
        super().__init__()
        self.proj = _PatchLinear(in_dim, embed_dim)


class _PosEmbed(nn.Module):
    def __init__(self, n: int, dim: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(n, dim), requires_grad=False)


class _MLP(nn.Module):
    def __init__(self, dim: int, hidden: int) -> None:
        super().__init__()
        self.linear_fc1 = _Linear(dim, hidden)
        self.linear_fc2 = _Linear(hidden, dim)


class _Block(nn.Module):
    def __init__(self, dim: int, hidden: int) -> None:
        super().__init__()
        self.norm1 = _LayerNorm(dim)
        self.norm2 = _LayerNorm(dim)
        self.attn = _Attn(dim)
        self.mlp = _MLP(dim, hidden)


class _Merger(nn.Module):
    def __init__(self, out_dim: int, context_dim: int, merge: int, postshuffle: bool) -> None:
        super().__init__()
        hidden = context_dim * merge * merge
        self.norm = _LayerNorm(hidden if postshuffle else context_dim)
        self.linear_fc1 = _Linear(hidden, hidden)
        self.linear_fc2 = _Linear(hidden, out_dim)


class Qwen3_VisionTransformer(QwenVisionBase):
    image_mean = (0.5, 0.5, 0.5)   # the Qwen3-VL checkpoints' preprocessor_config.json
    image_std = (0.5, 0.5, 0.5)

    def __init__(self, config: Any, weight_format: str = "bf16", fold_norm: bool = True) -> None:
        """`fold_norm`: norm1 / norm2 of every block are applied inside the GEMM that follows them (see
        Qwen2_5_VisionTransformer; here the norms are LayerNorms: the residual GEMMs also emit the row sums).  On by
        default (measured: 10.09 against 10.17 ms per 8192 patches)."""
        super().__init__()
        vc = config.vision_config if hasattr(config, "vision_config") else config
        if weight_format not in ("bf16", "fp8_e4m3"):
            raise ValueError(f"Unknown weight_format: {weight_format}")
        self.weight_format = weight_format
        E = vc.hidden_size
        self.fold_norm = (bool(fold_norm) and weight_format == "bf16" and E % 64 == 0 and 192 <= E <= 160 * ops.SUMSQ_PARTS
                          and vc.hidden_act in ("gelu_pytorch_tanh", "quick_gelu") and vc.intermediate_size > 128)
        self.in_channels = vc.in_channels
        self.embed_dim = vc.hidden_size
        self.num_heads = vc.num_heads
        self.intermediate_size = vc.intermediate_size
        self.patch_size = vc.patch_size
        self.temporal_patch_size = vc.temporal_patch_size
        self.spatial_merge_size = vc.spatial_merge_size
        self.spatial_merge_unit = self.spatial_merge_size**2
        self.deepstack_visual_indexes = list(vc.deepstack_visual_indexes or [])
        self.out_hidden_size = vc.out_hidden_size
        self.num_position_embeddings = vc.num_position_embeddings
        self.num_grid_per_side = int(math.sqrt(self.num_position_embeddings))
        self.norm_eps = getattr(vc, "rms_norm_eps", 1e-6)      # the name the reference reads (:221)
        self.head_dim = self.embed_dim // self.num_heads
        if vc.hidden_act not in _ACTIVATIONS:
            raise NotImplementedError(f"Activation function {vc.hidden_act!r} is not implemented.")
        self.act_epilogue = _ACTIVATIONS[vc.hidden_act]
        self.mlp_pad = -self.intermediate_size % 64    # zero columns so that fc2's K loop has no tail

        in_dim = self.in_channels * self.temporal_patch_size * self.patch_size * self.patch_size
        self.patch_embed = _PatchEmbed(in_dim, self.embed_dim)
        self.pos_embed = _PosEmbed(self.num_position_embeddings, self.embed_dim)
        self.blocks = nn.ModuleList([_Block(self.embed_dim, self.intermediate_size) for _ in range(vc.depth)])
        self.merger = _Merger(self.out_hidden_size, self.embed_dim, self.spatial_merge_size, postshuffle=False)
        self.deepstack_merger_list = (
            nn.ModuleList([_Merger(self.out_hidden_size, self.embed_dim, self.spatial_merge_size, postshuffle=True)
                           for _ in self.deepstack_visual_indexes])
            if self.deepstack_visual_indexes else None
        )

    @property
    def chunk_shape(self) -> tuple[int, ...]:
        return (1, self.out_hidden_size * (1 + len(self.deepstack_visual_indexes)))

    @torch.no_grad()
    def _pack(self) -> dict:
        pad = self.mlp_pad

        def pad_rows(w: torch.Tensor) -> torch.Tensor:     # [I, E] -> [I + pad, E]
            return torch.cat([w, w.new_zeros((pad,) + tuple(w.shape[1:]))]) if pad else w

        def pad_cols(w: torch.Tensor) -> torch.Tensor:     # [E, I] -> [E, I + pad]
            return torch.cat([w, w.new_zeros((w.shape[0], pad))], dim=1) if pad else w

        def merger(m: _Merger) -> dict:
            return {"norm": (m.norm.weight, m.norm.bias),
                    "fc1": self._lin(m.linear_fc1.weight, m.linear_fc1.bias),
                    "fc2": self._lin(m.linear_fc2.weight, m.linear_fc2.bias)}

        # (the patch embedding stays bf16 also with fp8 weights, like the other Qwen encoders')
        pk: dict = {"pe": {"w": self.patch_embed.proj.weight.contiguous(), "s": None, "b": self.patch_embed.proj.bias},
                    "pos": self.pos_embed.weight.contiguous()}
        def folded(w: torch.Tensor, b: torch.Tensor, norm: _LayerNorm, padded: bool) -> dict:
            w, b, colsum = fold_layernorm(w, b, norm.weight, norm.bias)
            if padded:   # pad AFTER folding: the pad rows stay exactly zero (weight, bias and column sum)
                w, b, colsum = pad_rows(w), pad_rows(b), pad_rows(colsum)
            return {"w": w.contiguous(), "s": None, "b": b.contiguous(), "colsum": colsum.contiguous()}

        fold = self.fold_norm
        pk["blocks"] = [
            {
                "n1": (b.norm1.weight, b.norm1.bias),
                "n2": (b.norm2.weight, b.norm2.bias),
                "qkv": folded(b.attn.qkv.weight, b.attn.qkv.bias, b.norm1, False) if fold
                else self._lin(b.attn.qkv.weight, b.attn.qkv.bias),
                "proj": self._lin(b.attn.proj.weight, b.attn.proj.bias),
                # gelu(0) = 0 and the padded fc2 columns are zero: the padding contributes exactly nothing
                "fc1": folded(b.mlp.linear_fc1.weight, b.mlp.linear_fc1.bias, b.norm2, True) if fold
                else self._lin(pad_rows(b.mlp.linear_fc1.weight), pad_rows(b.mlp.linear_fc1.bias)),
                "fc2": self._lin(pad_cols(b.mlp.linear_fc2.weight), b.mlp.linear_fc2.bias),
            }
            for b in self.blocks
        ]
        pk["merger"] = merger(self.merger)
        pk["deepstack"] = [merger(m) for m in (self.deepstack_merger_list or [])]
        dim = self.head_dim // 2
        pk["inv_freq"] = (1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))).to(self.device)
        return pk

    def forward_device(self, pixel_values: torch.Tensor, grid_thw: np.ndarray, mark=None) -> list[torch.Tensor]:
        """pixel_values: bf16 [L, C*T*P*P] already on the device; grid_thw: host int64 [n,3]."""
        if mark is None:
            mark = _no_mark
        pk = self._ensure_packed()
        E, nh, d, unit, dev = self.embed_dim, self.num_heads, self.head_dim, self.spatial_merge_unit, self.device
        eps, O = self.norm_eps, self.out_hidden_size
        if self.fold_norm:   # 32-bit operand offsets in the folded-norm GEMMs: a batch beyond them runs as several
            groups = self._addressable_groups(grid_thw, (2**32 - 1) // (2 * max(3 * E, self.intermediate_size + self.mlp_pad)))
            if len(groups) > 1:
                return self._forward_in_groups(pixel_values, grid_thw, groups, mark)

        # rotary table (:320-362) and one attention segment per frame (:288-291): the Qwen2.5-VL index routines
        # with a window larger than any grid, i.e. without the window permutation
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
        pos = ops.pos_embed_interp(pk["pos"], meta, L, sl.max_units_per_item, merge)
        x = self._g(pixel_values, pk["pe"], pos=pos)           # (m % L) == m: one position row per patch row
        n = torch.empty_like(x)
        qkv = torch.empty((L, 3 * E), dtype=torch.bfloat16, device=dev)
        att = torch.empty((L, E), dtype=torch.bfloat16, device=dev)
        hmid = torch.empty((L, self.intermediate_size + self.mlp_pad), dtype=torch.bfloat16, device=dev)
        n_out = 1 + len(self.deepstack_visual_indexes)
        out = torch.empty((L // unit, O * n_out), dtype=torch.bfloat16, device=dev)
        scale = d**-0.5
        kept: list[torch.Tensor] = []
        fold = self.fold_norm
        if fold:
            mark("norm")
            ss = torch.zeros((L, ops.SUMSQ_PARTS), dtype=torch.float32, device=dev)
            sm = torch.zeros_like(ss)
            ops.row_stats(x, ss, sm)
            stats_in = lambda lin: {"a_row_sumsq": ss, "a_row_sum": sm, "w_col_sum": lin["colsum"], "norm_eps": eps}  # noqa: E731
            stats_out = {"c_row_sumsq": ss, "c_row_sum": sm}
        else:
            stats_out = {}
        if self.split_residual:   # the byte plane of the residual stream; zero = "x is exact".  It is updated in place
            lo = torch.zeros(x.shape, dtype=torch.uint8, device=dev)   # even when the bf16 plane moves to a new buffer
            stats_out = dict(stats_out, residual_lo=lo, out_lo=lo)
        # few rows: each launch names the weights of the launch after next for its idle compute units to read
        hint = L <= self.prefetch_rows
        for i, b in enumerate(pk["blocks"]):
            after = pk["blocks"][i + 1]["qkv"] if i + 1 < len(pk["blocks"]) else pk["merger"]["fc1"]
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
            mark("rope")
            ops.rope_qk_(qkv, ix.cos_sin, nh, d)
            mark("attn_full")
            ops.attn_varlen(qkv[:, :E], qkv[:, E : 2 * E], qkv[:, 2 * E :], plan, nh, d, scale, out=att)
            mark("gemm_proj")
            # a hidden state kept for a deepstack merger must survive: the next update goes to a new buffer
            x_next = torch.empty_like(x) if kept and kept[-1] is x else x
            self._g(att, b["proj"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x_next, prefetch=pf_proj, **stats_out)
            x = x_next
            if fold:
                mark("gemm_fc1")
                ops.gemm(x, b["fc1"]["w"], b["fc1"]["b"], epilogue=self.act_epilogue, out=hmid, prefetch=pf_fc1,
                         **stats_in(b["fc1"]))
            else:
                mark("norm")
                ops.layernorm(x, *b["n2"], eps, out=n)
                mark("gemm_fc1")
                self._g(n, b["fc1"], epilogue=self.act_epilogue, out=hmid, prefetch=pf_fc1)
            mark("gemm_fc2")
            self._g(hmid, b["fc2"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, prefetch=pf_fc2, **stats_out)
            if i in self.deepstack_visual_indexes:
                kept.append(x)

        mark("gemm_merger")
        mergers = [(pk["merger"], x, False)] + [(m, h, True) for m, h in zip(pk["deepstack"], kept)]
        for j, (m, h, postshuffle) in enumerate(mergers):
            if postshuffle:
                nm = ops.layernorm(h.view(L // unit, E * unit), *m["norm"], eps)
            else:
                nm = ops.layernorm(h, *m["norm"], eps, out=n).view(L // unit, E * unit)
            y = self._g(nm, m["fc1"], epilogue=ops.EPI_GELU_ERF)
            self._g(y, m["fc2"], out=out[:, j * O : (j + 1) * O])
        mark("end")
        g = grid_thw.reshape(-1, 3)
        seqlens = (g[:, 0] * g[:, 1] * g[:, 2]) // unit
        return list(out.split([int(s) for s in seqlens], dim=0))


class ModalityProcessor(BaseModalityProcessor):
    """Qwen3-VL modality processor (reference: :428-461): wraps the Hugging Face processor's image and video
    processors, which have to be available locally; preprocessing is outside the accelerated path.

    The reference's video processor passes the metadata (fps, duration, frame indices) that its own video loader
    recorded for the clip; a caller that has such a record sets `video_metadata_provider` to a callable returning
    it (a `transformers.video_utils.VideoMetadata`), otherwise the clip is processed without metadata."""

    def __init__(self, model_id: str) -> None:
        super().__init__(model_id=model_id)
        from transformers import AutoProcessor  # deferred: needs the model files

        self.hf_processor = AutoProcessor.from_pretrained(model_id, trust_remote_code=True)
        self.video_metadata_provider: Callable | None = None

    def get_image_processor(self) -> Callable | None:
        def processor(image) -> dict[str, torch.Tensor]:
            return self.hf_processor.image_processor(images=[image], videos=None, return_tensors="pt").data

        return processor

    def get_video_processor(self) -> Callable | None:
        def processor(video) -> dict[str, torch.Tensor]:
            kwargs = {}
            if self.video_metadata_provider is not None:
                kwargs["video_metadata"] = [self.video_metadata_provider()]
            return self.hf_processor.video_processor(videos=[video], do_sample_frames=False, return_tensors="pt",
                                                     **kwargs).data

        return processor
