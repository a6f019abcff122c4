"""Qwen2.5-VL vision transformer on hand-written gfx950 kernels.

Drop-in for `Qwen2_5_VisionTransformer` (reference: eric/models/qwen2_5_vl.py:262-485): same constructor
argument (the HF config, of which only `vision_config` is read), same parameter names as the checkpoint
after `visual.` is stripped, same `forward(modality, adapter_name, batch)` contract and output list.

What differs is everything underneath.  The forward pass is a fixed sequence of C-ABI kernel launches
on torch's current stream:

    patch-embed GEMM (window permutation fused as a row gather of A)        :424,:438-440
    per block:  RMSNorm -> QKV GEMM(+bias) -> varlen MFMA attention with rotary fused into the q/k load
                -> proj GEMM(+bias,+residual) -> RMSNorm -> gate|up GEMM(+bias, SiLU*mul)
                -> down GEMM(+bias,+residual)                                :168-178
                (by default the two RMSNorms are folded into the GEMMs around them: see `fold_norm`)
    merger:     RMSNorm -> GEMM(+bias, GELU) -> GEMM(+bias) with the inverse window permutation fused
                as a row scatter of C                                        :225-233,:478-479

Weights are repacked once after loading: gate and up rows are interleaved (so SiLU(gate)*up is a
lane-local epilogue), the MLP intermediate size is zero-padded to a multiple of 64 so K loops have no
tail, and optionally every linear weight is quantised to fp8-e4m3 with per-output-channel scales.
"""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import numpy as np
import torch
import torch.nn as nn

from cornserve_amd import ops
from cornserve_amd.eric import frames as frame_ops
from cornserve_amd.eric.api import Modality
from cornserve_amd.eric.models.base import BaseModalityProcessor, EricModel


class _Linear(nn.Module):
    """Parameter holder with nn.Linear's names; arithmetic happens in the fused kernels."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(out_features, in_features), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(out_features), requires_grad=False) if bias else None


class _Scale(nn.Module):
    def __init__(self, dim: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim), requires_grad=False)


class _PatchProj(nn.Module):
    def __init__(self, in_channels: int, hidden: int, t: int, p: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(hidden, in_channels, t, p, p), requires_grad=False)


class _PatchEmbed(nn.Module):
    def __init__(self, in_channels: int, hidden: int, t: int, p: int) -> None:
        super().__init__()
        self.proj = _PatchProj(in_channels, hidden, t, p)


class _Attn(nn.Module):
    def __init__(self, dim: int) -> None:
        super().__init__()
        self.qkv = _Linear(dim, 3 * dim)
        self.proj = _Linear(dim, dim)


class _MLP(nn.Module):
    def __init__(self, dim: int, inter: int) -> None:
        super().__init__()
        self.gate_proj = _Linear(dim, inter)
        self.up_proj = _Linear(dim, inter)
        self.down_proj = _Linear(inter, dim)


class _Block(nn.Module):
    def __init__(self, dim: int, inter: int) -> None:
        super().__init__()
        self.norm1 = _Scale(dim)
        self.norm2 = _Scale(dim)
        self.attn = _Attn(dim)
        self.mlp = _MLP(dim, inter)


class _Merger(nn.Module):
    def __init__(self, out_dim: int, context_dim: int, merge: int) -> None:
        super().__init__()
        hidden = context_dim * merge * merge
        self.ln_q = _Scale(context_dim)
        self.mlp = nn.ModuleList([_Linear(hidden, hidden), nn.Identity(), _Linear(hidden, out_dim)])


def _no_mark(name: str) -> None:
    return None


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def quantize_fp8_rows(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-output-channel e4m3 quantisation: scale = amax/448 (fp32), q = rne(w/scale)."""
    wf = w.float()
    scale = wf.abs().amax(dim=1).clamp_min(1e-12) / 448.0
    q = (wf / scale[:, None]).to(torch.float8_e4m3fn)
    return q, scale.contiguous()


class QwenVisionBase(EricModel):
    """What the Qwen2-VL family encoders share: parameter placement, lazy repacking of the weights into their
    device form, the batch formats of `forward` and the uint8-frame input path.  Subclasses provide `_pack`,
    `forward_device`, `chunk_shape` and the attributes patch_size, temporal_patch_size, spatial_merge_size,
    in_channels, weight_format and patch_embed."""

    # Batches of at most this many patches pass the GEMM launches a weight-prefetch hint (0: never): such launches
    # leave compute units idle, and those read the weights a later launch of the block needs into the last-level cache.
    prefetch_rows = 6144

    # what the checkpoint's image processor normalises with (preprocessor_config.json): CLIP statistics for
    # Qwen2-VL and Qwen2.5-VL; subclasses override
    # carry the residual stream with 16 significant bits (see Qwen2_5_VisionTransformer.__init__)
    split_residual: bool = True
    image_mean: tuple = frame_ops.CLIP_MEAN
    image_std: tuple = frame_ops.CLIP_STD

    def __init__(self) -> None:
        super().__init__()
        self._packed: dict | None = None
        self.register_load_state_dict_post_hook(lambda module, incompatible: module._invalidate())

    # ------------------------------------------------------------------ EricModel properties
    @property
    def dtype(self) -> torch.dtype:
        return self.patch_embed.proj.weight.dtype

    @property
    def device(self) -> torch.device:
        return self.patch_embed.proj.weight.device

    # ------------------------------------------------------------------ weight repacking
    def _invalidate(self) -> None:
        self._packed = None

    def _apply(self, fn, recurse=True):  # .to()/.cuda()/.bfloat16() move the parameters: repack lazily
        self._packed = None
        return super()._apply(fn, recurse)

    def _lin(self, w: torch.Tensor, b: torch.Tensor | None) -> dict:
        """Device form of one linear layer: bf16 [N,K] or fp8 [N,K] + fp32 scale [N]."""
        w = w.contiguous()
        if self.weight_format == "fp8_e4m3":
            q, s = quantize_fp8_rows(w)
            return {"w": q.contiguous(), "s": s, "b": b}
        return {"w": w, "s": None, "b": b}

    def _ensure_packed(self) -> dict:
        if self._packed is None:
            if self.dtype != torch.bfloat16 or self.device.type != "cuda":
                raise RuntimeError(
                    "the gfx950 kernels need the model in bfloat16 on a GPU "
                    f"(got {self.dtype} on {self.device}); there is no CPU path"
                )
            self._packed = self._pack()
        return self._packed

    # ------------------------------------------------------------------ forward
    @staticmethod
    def _g(a: torch.Tensor, lin: dict, **kw) -> torch.Tensor:
        return ops.gemm(a, lin["w"], lin["b"], w_scale=lin["s"], **kw)

    def _plain_qkv(self, block: dict) -> dict:
        """The qkv layer of a block in the form the separate kernels take.  A window block keeps only the per-head
        packed form of its weight (one copy in HBM); the plain rows are the same bits in another order and are put back
        together the first time an item takes the separate kernels."""
        if block["qkv"] is None:
            wp, bp, *sp = block["qkv_wattn"]
            w, b, *s = ops.unpack_qkv_window_attn(wp, bp, self.num_heads, w_scale=sp[0] if sp else None)
            block["qkv"] = {"w": w, "b": b, "s": s[0] if s else None}
        return block["qkv"]

    def patchify_frames(self, frames: list[torch.Tensor], arithmetic: str = "fused",
                        pixel_budgets: list | None = None) -> tuple[torch.Tensor, np.ndarray]:
        """uint8 frames of every item ([T,H,W,3] or [H,W,3], on the host or the device) -> (pixel_values
        [L, C*T*P*P] in the model dtype on the device, grid_thw int64 [n,3]): what the Hugging Face processor the
        reference runs (:488-512) produces from the same frames, with rescale, normalise and the patch layout done on
        the GPU.  Without `pixel_budgets` the frames are already at the processor's target size; with it (one
        (min_pixels, max_pixels) pair per item) they are as decoded and the processor's resize runs on the GPU too
        (`frames.target_size`, then `ops.resize_bicubic_u8`: Pillow's bicubic, bit for bit)."""
        p, m, tps, dev = self.patch_size, self.spatial_merge_size, self.temporal_patch_size, self.device
        key = ("byte_table", arithmetic)   # (a model's mean / std are fixed)
        pk = self._ensure_packed()
        if key not in pk:
            pk[key] = frame_ops.byte_table(self.image_mean, self.image_std, arithmetic=arithmetic).to(dev)
        items, grids = [], []
        for f in frames:
            f = torch.as_tensor(f)
            if f.dim() == 3:
                f = f[None]
            if f.dtype != torch.uint8 or f.dim() != 4 or f.shape[-1] != 3:
                raise ValueError("frames must be uint8 [T,H,W,3] or [H,W,3] (RGB)")
            f = f.contiguous().to(dev, non_blocking=True)
            if pixel_budgets is not None:
                lo, hi = (int(v) for v in torch.as_tensor(pixel_budgets[len(items)]).reshape(-1).tolist())
                f = ops.resize_bicubic_u8(f, *frame_ops.target_size(f.shape[1], f.shape[2], p * m, lo, hi))
            T, H, W, _ = f.shape
            if H % (p * m) or W % (p * m) or T < 1:
                raise ValueError(f"frame size {H}x{W} is not a multiple of {p * m}: resize first (frames.resize_frames)")
            items.append(f)
            grids.append((-(-T // tps), H // p, W // p))
        grid = np.asarray(grids, dtype=np.int64).reshape(-1, 3)
        L = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
        px = torch.empty((L, self.in_channels * tps * p * p), dtype=self.dtype, device=dev)
        row = 0
        for f, (gt, gh, gw) in zip(items, grids):
            ops.qwen_patchify_u8(f, pk[key], p, m, tps, out=px[row : row + gt * gh * gw])
            row += gt * gh * gw
        return px, grid

    @staticmethod
    def _addressable_groups(grid_thw: np.ndarray, max_rows: int) -> list[tuple[int, int]]:
        """Consecutive item ranges [first, last) of at most `max_rows` patches each (items are independent, so a batch
        can run as several); one range when the whole batch fits.  An item above the limit on its own is refused."""
        g = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)
        rows = g[:, 0] * g[:, 1] * g[:, 2]
        if int(rows.sum()) <= max_rows:
            return [(0, len(rows))]
        groups, first, acc = [], 0, 0
        for i, r in enumerate(rows.tolist()):
            if r > max_rows:
                raise ValueError(f"item {i} has {r} patches, more than the {max_rows} the folded-norm GEMMs address; "
                                 "construct the model with fold_norm=False")
            if acc + r > max_rows:
                groups.append((first, i))
                first, acc = i, 0
            acc += r
        groups.append((first, len(rows)))
        return groups

    def _forward_in_groups(self, pixel_values: torch.Tensor, grid_thw: np.ndarray, groups, mark) -> list[torch.Tensor]:
        g = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)
        starts = np.concatenate([[0], np.cumsum(g[:, 0] * g[:, 1] * g[:, 2])])
        out: list[torch.Tensor] = []
        for first, last in groups:
            out += self.forward_device(pixel_values[int(starts[first]):int(starts[last])], g[first:last], mark)
        return out

    @torch.inference_mode()
    def forward(self, modality: Modality, adapter_name: str, batch: dict[str, list[torch.Tensor]]) -> list[torch.Tensor]:
        """See the reference docstring (:402-413): `pixel_values` + `image_grid_thw` for images,
        `pixel_values_videos` + `video_grid_thw` for videos.  In addition to the reference's format, a batch
        may carry `pixel_frames` / `pixel_frames_videos` instead: one uint8 [T,H,W,3] tensor of resized frames
        per item (see `FrameModalityProcessor`); the grids follow from the shapes.  With `raw_frames` /
        `raw_frames_videos` the frames are as decoded, and `raw_frames_budget` holds each item's
        (min_pixels, max_pixels): the resize runs on the GPU as well."""
        if modality == Modality.IMAGE:
            px_key, grid_key, frame_key, raw_key = "pixel_values", "image_grid_thw", "pixel_frames", "raw_frames"
        elif modality == Modality.VIDEO:
            px_key, grid_key, frame_key, raw_key = ("pixel_values_videos", "video_grid_thw", "pixel_frames_videos",
                                                    "raw_frames_videos")
        else:
            raise ValueError(f"Unsupported modality: {modality}")
        if raw_key in batch:
            if len(batch.get("raw_frames_budget", ())) != len(batch[raw_key]):
                raise ValueError(f"`{raw_key}` needs one `raw_frames_budget` entry (min_pixels, max_pixels) per item")
            return self.forward_device(*self.patchify_frames(batch[raw_key], pixel_budgets=batch["raw_frames_budget"]))
        if frame_key in batch:
            return self.forward_device(*self.patchify_frames(batch[frame_key]))
        pixel_values = ops.cat_to_device(batch[px_key], self.device, self.dtype)
        grid = torch.cat([g.reshape(-1, 3) for g in batch[grid_key]], dim=0).cpu().numpy().astype(np.int64)
        return self.forward_device(pixel_values, grid)


class Qwen2_5_VisionTransformer(QwenVisionBase):
    def __init__(self, config: Any, weight_format: str = "bf16", fold_norm: bool = True,
                 split_residual: bool = True, fuse_window_attn: bool = True, fuse_min_rows: int = 0,
                 fuse_min_fill: float | None = None) -> None:
        """`fuse_window_attn`: run qkv projection + rotary + window attention of a block (:93-120) as ONE launch
        (`ops.qkv_window_attn`: q, k and v stay in registers, the [L, 3*hidden] tensor is never written).  Every window
        takes a 64-row slot of that launch, so an ITEM takes it when its windows fill their slots to `fuse_min_fill` or
        more on average (an image whose sides are multiples of 8 patches fills them completely; edge windows of other
        sizes are shorter, and a slot's empty rows cost the projection as much as full ones: below about 0.75 the
        separate kernels are cheaper -- 0.92 with fp8 weights, whose projection costs more per row; None selects these
        measured break-even points).  Other items of the same batch and head dims other than 80 take the separate
        kernels.  The one launch rounds q and k to bf16 once (after the rotation) instead of twice, so the two
        routes agree within the parity tolerance, not bit for bit; since the route depends on the item alone, an item's
        embedding is the same bits whatever it is batched with (setting the attribute to False afterwards selects the
        separate kernels for every item).  `fuse_min_rows` > 0 is a deployment knob that gives this up for latency: a
        batch with fewer one-launch rows than that takes the separate kernels throughout, whose GEMM has narrower tiles
        for few rows (one 1024-patch image alone: 3.99 against 4.28 ms; 3072 is where the one launch starts to pay).

        `split_residual`: carry the residual stream (:175,177) with 16 significant bits -- the bf16 tensor every
        kernel reads plus a byte plane with the next 8 mantissa bits, joined and re-split inside the two residual GEMMs
        of a block -- so that the 2 x depth additions do not each round the stream to 8 bits.  A bf16 stream (False:
        the reference's arithmetic when loaded in bf16) drifts from the exact result by about 2e-2 of the output range
        over 32 blocks, which is the whole parity tolerance; the split stream stays near 1e-2.

        `fold_norm`: apply norm1 / norm2 of every block inside the GEMM that follows them (the norm weight is
        folded into that GEMM's weight columns at pack time, the per-row rsqrt is applied to the fp32
        accumulators, and the row sums of squares come out of the GEMM that wrote the residual stream).  The
        normalised activations are then never rounded to bf16 on their own, unlike the reference
        (norm.py:35-70 followed by F.linear): results stay inside the parity tolerance but are not
        bit-identical to the unfolded path.  Only with bf16 weights and a hidden size the fast GEMM takes."""
        super().__init__()
        vc = config.vision_config if hasattr(config, "vision_config") else config
        if weight_format not in ("bf16", "fp8_e4m3"):
            raise ValueError(f"Unknown weight_format: {weight_format}")
        self.weight_format = weight_format
        self.split_residual = bool(split_residual)
        self.fuse_min_rows = int(fuse_min_rows)
        self.fuse_min_fill = float(fuse_min_fill) if fuse_min_fill is not None else (0.75 if weight_format == "bf16" else 0.92)
        self.hidden_size = vc.hidden_size
        self.out_hidden_size = vc.out_hidden_size
        self.num_heads = vc.num_heads
        self.intermediate_size = vc.intermediate_size
        self.window_size = vc.window_size
        self.patch_size = vc.patch_size
        self.temporal_patch_size = vc.temporal_patch_size
        self.in_channels = getattr(vc, "in_channels", getattr(vc, "in_chans", 3))
        self.spatial_merge_size = vc.spatial_merge_size
        self.fullatt_block_indexes = list(vc.fullatt_block_indexes)
        self.spatial_merge_unit = self.spatial_merge_size**2
        self.norm_eps = getattr(config, "rms_norm_eps", 1e-6)
        if getattr(vc, "hidden_act", "silu") != "silu":
            raise NotImplementedError("only the SiLU-gated MLP of Qwen2.5-VL is implemented")
        self.head_dim = self.hidden_size // self.num_heads
        H = self.hidden_size
        # (the folded forms exist in the direct-to-LDS GEMM only: bf16 weights, K a multiple of 64 and at least 192 for
        # both the hidden and the padded intermediate size, hidden size within the row-sum parts)
        self.fold_norm = (bool(fold_norm) and weight_format == "bf16" and H % 64 == 0 and 192 <= H <= 160 * ops.SUMSQ_PARTS
                          and _round_up(self.intermediate_size, 64) >= 192)

        # (one launch for qkv + rotary + window attention: heads of 80, K a multiple of 64 from 192 up,
        # windows of 64 rows)
        win_rows = (self.window_size // self.spatial_merge_size // self.patch_size) ** 2 * self.spatial_merge_unit
        self.fuse_window_attn = (bool(fuse_window_attn) and H % 64 == 0 and H >= 192
                                 and self.head_dim == ops.QKV_WATTN_HEAD_DIM and win_rows == ops.QKV_WATTN_WINDOW)

        self.patch_embed = _PatchEmbed(self.in_channels, self.hidden_size, self.temporal_patch_size, self.patch_size)
        self.blocks = nn.ModuleList([_Block(self.hidden_size, self.intermediate_size) for _ in range(vc.depth)])
        self.merger = _Merger(self.out_hidden_size, self.hidden_size, self.spatial_merge_size)

    # ------------------------------------------------------------------ EricModel properties
    @property
    def chunk_shape(self) -> tuple[int, ...]:
        return (1, self.out_hidden_size)

    # ------------------------------------------------------------------ weight repacking
    @torch.no_grad()
    def _pack(self) -> dict:
        dev, H, I = self.device, self.hidden_size, self.intermediate_size
        Ip = _round_up(I, 64)
        pk: dict = {"Ip": Ip}
        pk["pe_w"] = self.patch_embed.proj.weight.reshape(H, -1).contiguous()
        blocks = []
        for i, blk in enumerate(self.blocks):
            gu_w = torch.zeros((2 * Ip, H), dtype=self.dtype, device=dev)
            gu_b = torch.zeros(2 * Ip, dtype=self.dtype, device=dev)
            gu_w[0 : 2 * I : 2] = blk.mlp.gate_proj.weight
            gu_w[1 : 2 * I : 2] = blk.mlp.up_proj.weight
            gu_b[0 : 2 * I : 2] = blk.mlp.gate_proj.bias
            gu_b[1 : 2 * I : 2] = blk.mlp.up_proj.bias
            down_w = torch.zeros((H, Ip), dtype=self.dtype, device=dev)
            down_w[:, :I] = blk.mlp.down_proj.weight
            qkv_w = blk.attn.qkv.weight
            if self.fold_norm:
                qkv_w = (qkv_w.float() * blk.norm1.weight.float()[None, :]).to(self.dtype)
                gu_w = (gu_w.float() * blk.norm2.weight.float()[None, :]).to(self.dtype)
            blocks.append(
                {
                    "n1": blk.norm1.weight,
                    "n2": blk.norm2.weight,
                    "qkv": self._lin(qkv_w, blk.attn.qkv.bias),
                    "proj": self._lin(blk.attn.proj.weight, blk.attn.proj.bias),
                    "gu": self._lin(gu_w, gu_b),
                    "down": self._lin(down_w, blk.mlp.down_proj.bias),
                }
            )
            if self.fuse_window_attn and i not in self.fullatt_block_indexes:
                # (fp8: the very bytes and scales of the plain form, reordered)
                lin = blocks[-1]["qkv"]
                blocks[-1]["qkv_wattn"] = ops.pack_qkv_window_attn(lin["w"], lin["b"].to(self.dtype), self.num_heads, w_scale=lin["s"])
                blocks[-1]["qkv"] = None   # the plain form comes back from the packed one if a batch ever needs it
        pk["blocks"] = blocks
        pk["ln_q"] = self.merger.ln_q.weight
        pk["fc1"] = self._lin(self.merger.mlp[0].weight, self.merger.mlp[0].bias)
        pk["fc2"] = self._lin(self.merger.mlp[2].weight, self.merger.mlp[2].bias)
        dim = self.head_dim // 2
        inv_freq = 1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))
        pk["inv_freq"] = inv_freq.to(dev)
        return pk

    # ------------------------------------------------------------------ forward
    def get_window_index(self, grid_thw) -> tuple[torch.Tensor, list[int]]:
        """Same results as the reference method (:357-386) followed by unique_consecutive (:436)."""
        g = np.asarray(torch.as_tensor(grid_thw).cpu(), dtype=np.int64).reshape(-1, 3)
        win = self.window_size // self.spatial_merge_size // self.patch_size
        sl = ops.vit_seqlens_host(g, self.spatial_merge_size, win)
        pk = self._ensure_packed()
        meta = torch.from_numpy(sl.item_meta).to(self.device)
        ix = ops.vit_index(meta, sl.total_patches, sl.max_units_per_item, self.spatial_merge_size, win, pk["inv_freq"])
        return ix.window_index, sl.cu_window.tolist()

    def _index(self, grid_thw: np.ndarray):
        """Everything that depends on the grids only: window permutation, rotary table, attention work lists
        (reference: rot_pos_emb :325-355, get_window_index :357-386, cu_seqlens :445-448), and the route of every item
        through the window blocks.

        An item whose windows fill their 64-row slots well enough (`fuse_min_fill`; whole windows fill them completely)
        takes the one-launch form of qkv + rotary + window attention, every other item the separate kernels.  The choice
        depends on the item alone, so an item's embedding does not depend on what it is batched with.  The items are
        PROCESSED with the one-launch items first (a stable reordering: their rows are then one leading block of the
        batch); the index kernel takes each item's place in the caller's patch matrix separately from its place in the
        processing order, and `order` maps processing position to the caller's item number.  `win_start` is None when
        every one-launch window has 64 rows, else the starts of those windows on the device."""
        merge = self.spatial_merge_size
        win = self.window_size // merge // self.patch_size
        dev = self.device
        g = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)
        n = g.shape[0]
        units = g[:, 0] * (g[:, 1] // merge) * (g[:, 2] // merge)
        if self.fuse_window_attn and n:
            slots = g[:, 0] * -(-(g[:, 1] // merge) // win) * -(-(g[:, 2] // merge) // win)   # windows of the item
            one_launch = units >= self.fuse_min_fill * slots * (win * win)
        else:
            one_launch = np.zeros(n, dtype=bool)
        fused_rows = int(units[one_launch].sum()) * merge * merge
        if fused_rows < self.fuse_min_rows:
            one_launch[:] = False
            fused_rows = 0
        order = np.concatenate([np.flatnonzero(one_launch), np.flatnonzero(~one_launch)]) if n else np.zeros(0, np.int64)
        sl = ops.vit_seqlens_host(g[order], merge, win)
        if n:
            caller_unit_base = np.concatenate([[0], np.cumsum(units)[:-1]])
            sl.item_meta[:, 7] = caller_unit_base[order]
        # the separate kernels' work list covers the windows behind the one-launch rows (absolute row numbers)
        first_sep = int(np.searchsorted(sl.cu_window, fused_rows))
        work_win, max_win = ops.attn_work_host(sl.cu_window[first_sep:])
        work_full, max_full = ops.attn_work_host(sl.cu_full)
        # the one-launch windows' starts, when any of them is short of 64 rows
        cu_fused = np.ascontiguousarray(sl.cu_window[:first_sep + 1], dtype=np.int32)
        ragged = bool(first_sep) and bool(np.any(np.diff(cu_fused) != ops.QKV_WATTN_WINDOW))
        # one host-to-device copy for the small arrays
        meta, dwin, dfull, dcu = ops.host_to_device_packed([sl.item_meta, work_win, work_full, cu_fused], dev)
        ix = ops.vit_index(meta, sl.total_patches, sl.max_units_per_item, merge, win, self._ensure_packed()["inv_freq"])
        return (ix, ops.AttnPlan(dwin, work_win.shape[0], max_win), ops.AttnPlan(dfull, work_full.shape[0], max_full),
                sl.total_patches, fused_rows, order, dcu if ragged else None)

    def forward_device(self, pixel_values: torch.Tensor, grid_thw: np.ndarray, mark=None) -> list[torch.Tensor]:
        """pixel_values: bf16 [L, C*T*P*P] already on the device; grid_thw: host int64 [n,3].

        `mark`, if given, is called as mark(name) right before the kernels of each named stage are
        enqueued (profiling hook: the caller records a stream event there)."""
        if mark is None:
            mark = _no_mark
        pk = self._ensure_packed()
        H, nh, d = self.hidden_size, self.num_heads, self.head_dim
        unit = self.spatial_merge_unit
        merge = self.spatial_merge_size
        win = self.window_size // merge // self.patch_size
        dev = self.device

        # the folded-norm GEMMs address their operands with 32-bit byte offsets: a batch beyond that runs as several
        if self.fold_norm:
            groups = self._addressable_groups(grid_thw, (2**32 - 1) // (2 * max(3 * H, pk["Ip"])))
            if len(groups) > 1:
                return self._forward_in_groups(pixel_values, grid_thw, groups, mark)
        mark("index")
        ix, plan_win, plan_full, L, fused_rows, order, win_start = self._index(grid_thw)
        if pixel_values.shape[0] != L:
            raise ValueError(f"pixel_values has {pixel_values.shape[0]} rows but grid_thw describes {L} patches")

        # patch embed; rows come out already in window order
        mark("patch_embed")
        x = ops.gemm(pixel_values, pk["pe_w"], None, a_rows=ix.src_rows)
        # the low-order plane of the residual stream; zero = "x is exact"
        res = {"residual_lo": (lo := torch.zeros(x.shape, dtype=torch.uint8, device=dev)), "out_lo": lo} if self.split_residual else {}
        n = torch.empty_like(x)
        # the folded-norm GEMMs exist in the fast kernel only, whose per-lane byte offsets are 32-bit
        fold = self.fold_norm
        eps = self.norm_eps
        if fold:
            mark("norm")
            ss = ops.row_sumsq(x, out=torch.zeros((L, ops.SUMSQ_PARTS), dtype=torch.float32, device=dev))
        qkv = torch.empty((L, 3 * H), dtype=torch.bfloat16, device=dev)
        att = torch.empty((L, H), dtype=torch.bfloat16, device=dev)
        hmid = torch.empty((L, pk["Ip"]), dtype=torch.bfloat16, device=dev)
        scale = d**-0.5
        # rows [0, fused_rows) belong to the items whose window blocks run as one launch, the rest to the others
        xf = x[:fused_rows]
        # A batch of few rows leaves most compute units idle in the N = hidden GEMMs, and what bounds those launches is
        # the latency of weights that nothing has touched since the previous forward pass: the one-launch window block
        # has its idle units read the gate|up weights, the attention-output projection the down-projection's, the
        # down-projection the next block's qkv weights.
        hint = L <= self.prefetch_rows

        def next_qkv(i: int) -> torch.Tensor | None:
            if i + 1 >= len(pk["blocks"]):
                return pk["fc1"]["w"]
            nb = pk["blocks"][i + 1]
            return nb["qkv"]["w"] if nb["qkv"] is not None else nb["qkv_wattn"][0]

        for i, b in enumerate(pk["blocks"]):
            full = i in self.fullatt_block_indexes
            pf_qkv = b["gu"]["w"] if hint else None   # (from the one-launch window block only: the plain QKV GEMM of a
            # small batch leaves too few compute units idle to read 18 MB in its own time -- measured slower)
            pf_proj = b["down"]["w"] if hint else None
            pf_down = next_qkv(i) if hint else None
            if not full and fused_rows:
                wp, bp, *sp = b["qkv_wattn"]      # (a third entry with fp8 weights: their scales)
                wsc = sp[0] if sp else None
                if fold:
                    mark("gemm_qkv_attn_window")
                    ops.qkv_window_attn(xf, wp, bp, ix.cos_sin[:fused_rows], nh, scale, a_row_sumsq=ss[:fused_rows], norm_eps=eps,
                                        out=att[:fused_rows], win_start=win_start, prefetch=pf_qkv)
                else:
                    mark("norm")
                    ops.rmsnorm(xf, b["n1"], eps, out=n[:fused_rows])
                    mark("gemm_qkv_attn_window")
                    ops.qkv_window_attn(n[:fused_rows], wp, bp, ix.cos_sin[:fused_rows], nh, scale, out=att[:fused_rows],
                                        win_start=win_start, w_scale=wsc, prefetch=pf_qkv)
            if full or fused_rows < L:
                lo = 0 if full else fused_rows           # first row the separate kernels work on in this block
                if fold:
                    mark("gemm_qkv")
                    self._g(x[lo:], self._plain_qkv(b), out=qkv[lo:], a_row_sumsq=ss[lo:], norm_eps=eps)
                else:
                    mark("norm")
                    ops.rmsnorm(x[lo:], b["n1"], eps, out=n[lo:])
                    mark("gemm_qkv")
                    self._g(n[lo:], self._plain_qkv(b), out=qkv[lo:])
                mark("attn_full" if full else "attn_window")
                ops.attn_varlen_rotary_(qkv, plan_full if full else plan_win, nh, d, scale, ix.cos_sin, out=att)
            mark("gemm_proj")
            if fold:
                self._g(att, b["proj"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, c_row_sumsq=ss, prefetch=pf_proj, **res)
                mark("gemm_gate_up")
                self._g(x, b["gu"], epilogue=ops.EPI_SWIGLU, out=hmid, a_row_sumsq=ss, norm_eps=eps)
                mark("gemm_down")
                self._g(hmid, b["down"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, c_row_sumsq=ss, prefetch=pf_down, **res)
            else:
                self._g(att, b["proj"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, prefetch=pf_proj, **res)
                mark("norm")
                ops.rmsnorm(x, b["n2"], eps, out=n)
                mark("gemm_gate_up")
                self._g(n, b["gu"], epilogue=ops.EPI_SWIGLU, out=hmid)
                mark("gemm_down")
                self._g(hmid, b["down"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, prefetch=pf_down, **res)

        mark("norm")
        ops.rmsnorm(x, pk["ln_q"], self.norm_eps, out=n)
        mark("gemm_merger")
        y = self._g(n.view(L // unit, H * unit), pk["fc1"], epilogue=ops.EPI_GELU_ERF)
        out = torch.empty((L // unit, self.out_hidden_size), dtype=torch.bfloat16, device=dev)
        # merged row m sits at window-order position m; it belongs at row window_index[m]
        self._g(y, pk["fc2"], c_rows=ix.window_index32, out=out)
        mark("end")
        g = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)[order]
        seqlens = (g[:, 0] * g[:, 1] * g[:, 2]) // unit
        parts = out.split([int(s) for s in seqlens], dim=0)     # in processing order
        result: list = [None] * len(parts)
        for pos, item in enumerate(order.tolist()):
            result[item] = parts[pos]
        return result

class ModalityProcessor(BaseModalityProcessor):
    """Qwen2.5-VL modality processor (reference: :488-512). Wraps the HF image processor, which has to be
    available locally; preprocessing is outside the accelerated path."""

    def __init__(self, model_id: str) -> None:
        super().__init__(model_id=model_id)
        from transformers import AutoImageProcessor  # deferred: needs the model files

        self.hf_processor = AutoImageProcessor.from_pretrained(model_id)

    def get_image_processor(self) -> Callable | None:
        def processor(image) -> dict[str, torch.Tensor]:
            return self.hf_processor(images=[image], return_tensors="pt").data

        return processor

    def get_video_processor(self) -> Callable | None:
        def processor(video) -> dict[str, torch.Tensor]:
            return self.hf_processor(images=None, videos=[video], return_tensors="pt").data

        return processor


class FrameModalityProcessor(BaseModalityProcessor):
    """Processor for the uint8-frame input formats.  With `resize_on="router"` it resizes only (the Hugging Face
    processor's target size and PIL bicubic resampling) and emits `pixel_frames` / `pixel_frames_videos`; rescale,
    normalise and the patch layout run on the GPU inside the model's forward.  With `resize_on="gpu"` it only checks
    the frames and emits them as decoded (`raw_frames` / `raw_frames_videos` plus the pixel budget); the model resizes
    them on the GPU to the same bytes.  Needs no model files."""

    def __init__(self, model_id: str, min_pixels: int = 56 * 56, max_pixels: int = 14 * 14 * 4 * 1280,
                 factor: int = 28, resize_on: str = "router") -> None:
        """`factor` = patch size x merge size of the encoder (28 for Qwen2-VL / Qwen2.5-VL, 32 for Qwen3-VL)."""
        super().__init__(model_id=model_id)
        if resize_on not in ("router", "gpu"):
            raise ValueError(f"resize_on must be 'router' or 'gpu', got {resize_on!r}")
        self.min_pixels, self.max_pixels, self.factor, self.resize_on = min_pixels, max_pixels, factor, resize_on

    def _frames(self, frames, key: str) -> dict[str, torch.Tensor]:
        if self.resize_on == "router":
            resized = frame_ops.resize_frames(frames, self.factor, self.min_pixels, self.max_pixels)
            return {"pixel_frames" + key: torch.from_numpy(resized)}
        raw = frame_ops.as_frames(frames)
        frame_ops.target_size(raw.shape[1], raw.shape[2], self.factor, self.min_pixels, self.max_pixels)   # aspect check
        return {"raw_frames" + key: torch.from_numpy(raw),
                "raw_frames_budget": torch.tensor([self.min_pixels, self.max_pixels], dtype=torch.int64)}

    def get_image_processor(self) -> Callable | None:
        return lambda image: self._frames(image, "")

    def get_video_processor(self) -> Callable | None:
        return lambda video: self._frames(video, "_videos")
