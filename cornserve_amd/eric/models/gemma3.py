"""Gemma-3 vision encoder (SigLIP tower + multimodal projector adapters) on hand-written gfx950 kernels.

Drop-in for `Gemma3VisionEncoder` (reference: eric/models/gemma3.py:58-136) with the SigLIP tower of
eric/models/layers/siglip.py.  Parameter names follow the checkpoint (`vision_tower.vision_model....`,
separate q/k/v projections, which the reference fuses at load time, eric/models/layers/linear.py:339-371);
the adapter container and its error behaviour follow eric/models/base.py:57-90.

Forward = one fixed sequence of C-ABI launches:

    strided patch gather -> patch-embed GEMM (+bias, +learned position embedding)  siglip.py:91-101
    per layer: LayerNorm -> fused QKV GEMM -> full MFMA attention (d=72) -> out GEMM(+residual)
               LayerNorm -> fc1 GEMM(+GELU-tanh) -> fc2 GEMM(+residual)            siglip.py:166-189
    post LayerNorm                                                                 siglip.py:275-279
    AvgPool(4x4)+GemmaRMSNorm -> projection GEMM                                   gemma3.py:33-49
"""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import numpy as np
import torch
import torch.nn as nn

from cornserve_amd import ops
from cornserve_amd.eric.api import Modality
from cornserve_amd.eric.models.base import BaseAdapterModule, BaseModalityProcessor, EricModel, fold_layernorm
from cornserve_amd.eric.models.qwen2_5_vl import _Linear, _round_up


class _LN(nn.Module):
    def __init__(self, dim: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(dim), requires_grad=False)


class _Conv(nn.Module):
    def __init__(self, cin: int, cout: int, k: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(cout, cin, k, k), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(cout), requires_grad=False)


class _Embedding(nn.Module):
    def __init__(self, n: int, dim: int) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(n, dim), requires_grad=False)


class _Embeddings(nn.Module):
    def __init__(self, cfg: Any) -> None:
        super().__init__()
        self.patch_embedding = _Conv(cfg.num_channels, cfg.hidden_size, cfg.patch_size)
        self.position_embedding = _Embedding((cfg.image_size // cfg.patch_size) ** 2, cfg.hidden_size)


class _SelfAttn(nn.Module):
    def __init__(self, dim: int) -> None:
        super().__init__()
        self.q_proj = _Linear(dim, dim)
        self.k_proj = _Linear(dim, dim)
        self.v_proj = _Linear(dim, dim)
        self.out_proj = _Linear(dim, dim)


class _SiglipMLP(nn.Module):
    def __init__(self, dim: int, inter: int) -> None:
        super().__init__()
        self.fc1 = _Linear(dim, inter)
        self.fc2 = _Linear(inter, dim)


class _EncoderLayer(nn.Module):
    def __init__(self, dim: int, inter: int) -> None:
        super().__init__()
        self.self_attn = _SelfAttn(dim)
        self.layer_norm1 = _LN(dim)
        self.mlp = _SiglipMLP(dim, inter)
        self.layer_norm2 = _LN(dim)


class _Encoder(nn.Module):
    def __init__(self, cfg: Any, num_layers: int) -> None:
        super().__init__()
        self.layers = nn.ModuleList([_EncoderLayer(cfg.hidden_size, cfg.intermediate_size) for _ in range(num_layers)])


class SiglipVisionTransformer(nn.Module):
    """The tower, optionally built only up to a feature layer and then without its final LayerNorm (reference:
    siglip.py:301-335)."""

    def __init__(self, cfg: Any, num_hidden_layers_override: int | None = None,
                 require_post_norm: bool | None = None) -> None:
        super().__init__()
        num_layers = cfg.num_hidden_layers if num_hidden_layers_override is None else num_hidden_layers_override
        if num_layers > cfg.num_hidden_layers:
            raise ValueError(f"The original encoder only has {cfg.num_hidden_layers} layers, "
                             f"but you requested {num_layers} layers.")
        self.embeddings = _Embeddings(cfg)
        self.encoder = _Encoder(cfg, num_layers)
        if require_post_norm is None:
            require_post_norm = num_layers == cfg.num_hidden_layers
        self.post_layernorm = _LN(cfg.hidden_size) if require_post_norm else None


class SiglipVisionModel(nn.Module):
    def __init__(self, cfg: Any, num_hidden_layers_override: int | None = None,
                 require_post_norm: bool | None = None) -> None:
        super().__init__()
        self.vision_model = SiglipVisionTransformer(cfg, num_hidden_layers_override, require_post_norm)


class Gemma3MultiModalProjector(nn.Module):
    """Adapter: AvgPool2d -> GemmaRMSNorm -> projection (reference: gemma3.py:18-49)."""

    def __init__(self, config: Any) -> None:
        super().__init__()
        vc = config.vision_config
        self.mm_input_projection_weight = nn.Parameter(
            torch.zeros(vc.hidden_size, config.text_config.hidden_size), requires_grad=False
        )
        self.mm_soft_emb_norm = nn.Module()
        self.mm_soft_emb_norm.weight = nn.Parameter(torch.zeros(vc.hidden_size), requires_grad=False)
        self.eps = vc.layer_norm_eps
        self.patches_per_image = int(vc.image_size // vc.patch_size)
        self.tokens_per_side = int(config.mm_tokens_per_image**0.5)
        self.kernel_size = self.patches_per_image // self.tokens_per_side
        self._wt: torch.Tensor | None = None
        self.register_load_state_dict_post_hook(lambda module, incompatible: setattr(module, "_wt", None))

    def _apply(self, fn, recurse=True):
        self._wt = None
        return super()._apply(fn, recurse)

    def forward(self, vision_outputs: torch.Tensor) -> torch.Tensor:
        if self._wt is None:  # GEMM wants the weight as [N=T, K=H]
            self._wt = self.mm_input_projection_weight.t().contiguous()
        B = vision_outputs.shape[0]
        normed = ops.avgpool_gemma_rmsnorm(
            vision_outputs, self.mm_soft_emb_norm.weight, self.patches_per_image, self.kernel_size, self.eps
        )
        out = ops.gemm(normed.view(-1, normed.shape[-1]), self._wt, None)
        return out.view(B, -1, out.shape[-1])


class Gemma3MultiModalProjectorAdapter(BaseAdapterModule):
    def __init__(self) -> None:
        super().__init__(adapter_cls=Gemma3MultiModalProjector)


class SiglipEncoderBase(EricModel):
    """What the encoders built on the SigLIP tower share: the packed weights and the tower's launch sequence.
    A subclass sets `self.config` (with `.vision_config`), `self.vision_tower` (a SiglipVisionModel) and calls
    `_init_tower(fold_norm)`."""
    # the residual stream (siglip.py:178,188) is carried with 16 significant bits, as in Qwen2_5_VisionTransformer
    split_residual: bool = True

    def _init_tower(self, fold_norm: bool) -> None:
        vc = self.config.vision_config
        self.fold_norm = (bool(fold_norm) and vc.hidden_size % 64 == 0 and 192 <= vc.hidden_size <= 160 * ops.SUMSQ_PARTS
                          and getattr(vc, "hidden_act", "gelu_pytorch_tanh") == "gelu_pytorch_tanh"
                          and vc.intermediate_size > 128)   # fc2's K, padded to a multiple of 64, must be at least 192
        self._packed: dict | None = None
        self.register_load_state_dict_post_hook(lambda module, incompatible: setattr(module, "_packed", None))

    @property
    def dtype(self) -> torch.dtype:
        return self.vision_tower.vision_model.embeddings.patch_embedding.weight.dtype

    @property
    def device(self) -> torch.device:
        return self.vision_tower.vision_model.embeddings.patch_embedding.weight.device

    def _apply(self, fn, recurse=True):
        self._packed = None
        return super()._apply(fn, recurse)

    @torch.no_grad()
    def _pack(self) -> dict:
        vm = self.vision_tower.vision_model
        vc = self.config.vision_config
        H = vc.hidden_size
        kraw = vc.num_channels * vc.patch_size * vc.patch_size
        kp = _round_up(kraw, 8)    # K of the strided-gather patch-embedding GEMM: a multiple of 8, zero columns behind kraw
        pe_w = torch.zeros((H, kp), dtype=self.dtype, device=self.device)
        pe_w[:, :kraw] = vm.embeddings.patch_embedding.weight.reshape(H, kraw)
        # The MLP intermediate size (4304 for SigLIP-so400m) is padded to a multiple of 64 so that fc2's K loop is
        # tail-free: the pad rows of fc1 (and their bias) are zero, GELU(0) = 0, and fc2's pad columns are zero,
        # so the padded activations are exactly zero and the result is unchanged.
        inter = vc.intermediate_size
        ip = _round_up(inter, 64)

        def pad_rows(w: torch.Tensor) -> torch.Tensor:
            out = torch.zeros((ip, *w.shape[1:]), dtype=w.dtype, device=w.device)
            out[:inter] = w
            return out

        def pad_cols(w: torch.Tensor) -> torch.Tensor:
            out = torch.zeros((w.shape[0], ip), dtype=w.dtype, device=w.device)
            out[:, :inter] = w
            return out

        layers = []
        for lyr in vm.encoder.layers:
            a = lyr.self_attn
            entry = {
                "ln1": (lyr.layer_norm1.weight, lyr.layer_norm1.bias),
                "ln2": (lyr.layer_norm2.weight, lyr.layer_norm2.bias),
                "qkv_w": torch.cat([a.q_proj.weight, a.k_proj.weight, a.v_proj.weight], dim=0).contiguous(),
                "qkv_b": torch.cat([a.q_proj.bias, a.k_proj.bias, a.v_proj.bias], dim=0).contiguous(),
                "out": (a.out_proj.weight, a.out_proj.bias),
                "fc1": (pad_rows(lyr.mlp.fc1.weight), pad_rows(lyr.mlp.fc1.bias)),
                "fc2": (pad_cols(lyr.mlp.fc2.weight), lyr.mlp.fc2.bias),
            }
            if self.fold_norm:
                w, b, cs = fold_layernorm(entry["qkv_w"], entry["qkv_b"], *entry["ln1"])
                entry["qkv_w"], entry["qkv_b"], entry["qkv_colsum"] = w, b, cs
                w, b, cs = fold_layernorm(lyr.mlp.fc1.weight, lyr.mlp.fc1.bias, *entry["ln2"])
                # pad AFTER folding: the pad rows stay exactly zero (weight, bias and column sum)
                entry["fc1"], entry["fc1_colsum"] = (pad_rows(w), pad_rows(b)), pad_rows(cs)
            layers.append(entry)
        return {"pe_w": pe_w, "pe_b": vm.embeddings.patch_embedding.bias, "kp": kp, "ip": ip,
                "pos": vm.embeddings.position_embedding.weight, "layers": layers,
                "post": None if vm.post_layernorm is None else (vm.post_layernorm.weight, vm.post_layernorm.bias)}

    def _ensure_packed(self) -> dict:
        if self._packed is None:
            if self.dtype != torch.bfloat16 or self.device.type != "cuda":
                raise RuntimeError(
                    "the gfx950 kernels need the model in bfloat16 on a GPU "
                    f"(got {self.dtype} on {self.device}); there is no CPU path"
                )
            self._packed = self._pack()
        return self._packed

    def vision_tower_forward(self, pixel_values: torch.Tensor) -> torch.Tensor:
        """pixel_values: bf16 [B,3,S,S] on the device -> [B, tokens, H] (after the post-layernorm if the tower has one)."""
        pk = self._ensure_packed()
        vc = self.config.vision_config
        H, nh = vc.hidden_size, vc.num_attention_heads
        d = H // nh
        B = pixel_values.shape[0]
        tokens = (vc.image_size // vc.patch_size) ** 2
        if self.fold_norm:   # 32-bit operand offsets in the folded-norm GEMMs: a batch beyond them runs as several
            most = max(1, ((2**32 - 1) // (2 * max(3 * H, pk["ip"]))) // tokens)
            if B > most:
                return torch.cat([self.vision_tower_forward(pixel_values[i : i + most]) for i in range(0, B, most)])
        M = B * tokens
        # Conv2d(kernel = stride = patch) + position rows as ONE strided-gather GEMM: the patches are fetched from the
        # NCHW image inside the kernel (siglip.py:30-36,94-101); no [tokens, C*patch*patch] buffer exists
        x = ops.gemm(pixel_values.contiguous(), pk["pe_w"], pk["pe_b"], pos=pk["pos"], conv_patch=vc.patch_size)
        plan = ops.attn_plan(np.arange(0, M + 1, tokens, dtype=np.int32), x.device)
        n = torch.empty_like(x)
        qkv = torch.empty((M, 3 * H), dtype=torch.bfloat16, device=x.device)
        att = torch.empty((M, H), dtype=torch.bfloat16, device=x.device)
        hmid = torch.empty((M, pk["ip"]), dtype=torch.bfloat16, device=x.device)
        eps = vc.layer_norm_eps
        act = getattr(vc, "hidden_act", "gelu_pytorch_tanh")
        if act == "gelu_pytorch_tanh":
            epi = ops.EPI_GELU_TANH
        elif act == "gelu":
            epi = ops.EPI_GELU_ERF
        else:
            raise NotImplementedError(f"Activation function {act!r} is not implemented.")
        fold = self.fold_norm
        stats_out = {}
        if self.split_residual:   # the byte plane of the residual stream (see Qwen2_5_VisionTransformer); zero = "x is exact"
            lo = torch.zeros(x.shape, dtype=torch.uint8, device=x.device)
            stats_out = {"residual_lo": lo, "out_lo": lo}
        if fold:
            ss = torch.zeros((M, ops.SUMSQ_PARTS), dtype=torch.float32, device=x.device)
            sm = torch.zeros_like(ss)
            ops.row_stats(x, ss, sm)
            stats_out.update(c_row_sumsq=ss, c_row_sum=sm)
        for lyr in pk["layers"]:
            if fold:
                ops.gemm(x, lyr["qkv_w"], lyr["qkv_b"], out=qkv, a_row_sumsq=ss, a_row_sum=sm,
                         w_col_sum=lyr["qkv_colsum"], norm_eps=eps)
            else:
                ops.layernorm(x, *lyr["ln1"], eps, out=n)
                ops.gemm(n, lyr["qkv_w"], lyr["qkv_b"], out=qkv)
            ops.attn_varlen(qkv[:, :H], qkv[:, H : 2 * H], qkv[:, 2 * H :], plan, nh, d, d**-0.5, out=att)
            ops.gemm(att, *lyr["out"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, **stats_out)
            if fold:
                ops.gemm(x, *lyr["fc1"], epilogue=epi, out=hmid, a_row_sumsq=ss, a_row_sum=sm,
                         w_col_sum=lyr["fc1_colsum"], norm_eps=eps)
            else:
                ops.layernorm(x, *lyr["ln2"], eps, out=n)
                ops.gemm(n, *lyr["fc1"], epilogue=epi, out=hmid)
            ops.gemm(hmid, *lyr["fc2"], epilogue=ops.EPI_RESIDUAL, residual=x, out=x, **stats_out)
        if pk["post"] is None:
            return x.view(B, tokens, H)
        ops.layernorm(x, *pk["post"], eps, out=n)
        return n.view(B, tokens, H)


class Gemma3VisionEncoder(SiglipEncoderBase):
    def __init__(self, config: Any, fold_norm: bool = False) -> None:
        """`fold_norm`: layer_norm1 / layer_norm2 of every SigLIP layer are applied inside the GEMM that follows them
        (the norm's weight and bias are folded into that GEMM's weight and bias at pack time, mean and variance come
        from row sums that the residual GEMMs emit): the normalised activations are not rounded to bf16 on their
        own, unlike the reference (siglip.py:333-345), so results stay inside the parity tolerance but are not
        bit-identical to fold_norm=False.  Off by default: the folded LayerNorm GEMM exists for the 256x160 tile only,
        which costs the wide QKV and fc1 projections more than the norm kernels take (measured on 4 x 896x896 images:
        25.6 against 24.8 ms)."""
        super().__init__()
        self.config = config
        self.vision_tower = SiglipVisionModel(config.vision_config)
        self.multi_modal_projector = Gemma3MultiModalProjectorAdapter()
        self._init_tower(fold_norm)

    @property
    def chunk_shape(self) -> tuple[int, ...]:
        # Same fixed chunking as the reference (gemma3.py:76-88): 256 divides 2560, 3840 and 5376.
        return (1, self.config.mm_tokens_per_image, 256)

    def _apply(self, fn, recurse=True):
        out = super()._apply(fn, recurse)
        for adapter in self.multi_modal_projector.adapters.values():  # adapters sit outside _modules
            adapter._apply(fn)
        return out

    @torch.inference_mode()
    def forward(self, modality: Modality, adapter_name: str, batch: dict[str, list[torch.Tensor]]) -> list[torch.Tensor]:
        """`pixel_values`: each [num_patches, 3, S, S]; `num_crops`: each [1] (reference: gemma3.py:90-136)."""
        if modality != Modality.IMAGE:
            raise ValueError(f"Unsupported modality: {modality}")
        if adapter_name is None:
            raise ValueError("Adapter name must be provided for Gemma 3 vision encoder.")
        size = self.config.vision_config.image_size
        assert len(batch["pixel_values"]) == len(batch["num_crops"])
        for pixels in batch["pixel_values"]:
            assert pixels.ndim == 4
            assert pixels.shape[1] == 3
            assert pixels.shape[2] == pixels.shape[3] == size
        pixel_values = ops.cat_to_device(batch["pixel_values"], self.device, self.dtype)
        num_patches = torch.cat([c.reshape(-1) for c in batch["num_crops"]]).cpu() + 1
        feats = self.vision_tower_forward(pixel_values)
        embeds = self.multi_modal_projector(adapter_name, feats)
        return [e.flatten(0, 1) for e in embeds.split(num_patches.tolist())]


class ModalityProcessor(BaseModalityProcessor):
    """Gemma 3 modality processor (reference: gemma3.py:139-156); needs the model files locally."""

    def __init__(self, model_id: str) -> None:
        super().__init__(model_id=model_id)
        from transformers import AutoProcessor  # deferred

        self.image_processor = AutoProcessor.from_pretrained(model_id).image_processor

    def get_image_processor(self) -> Callable | None:
        def processor(image) -> dict[str, torch.Tensor]:
            return self.image_processor(images=[image], return_tensors="pt").data

        return processor
