"""Base classes of the Eric model layer (reference: eric/models/base.py:17-148)."""

from __future__ import annotations

from abc import ABC, abstractmethod
from collections.abc import Callable
from typing import Any, Generic, TypeVar

import torch
import torch.nn as nn

from cornserve_amd.eric.api import Modality


class EricModel(nn.Module, ABC):
    """Base class for all models in Eric (reference: base.py:17-51)."""

    @abstractmethod
    def forward(self, modality: Modality, adapter_name: str, batch: dict[str, list[torch.Tensor]]) -> list[torch.Tensor]:
        """Embed one batch; returns one tensor per item, in item order."""

    @property
    @abstractmethod
    def dtype(self) -> torch.dtype:
        """Data type of the model's embeddings."""

    @property
    @abstractmethod
    def device(self) -> torch.device:
        """Device the inputs are moved to."""

    @property
    @abstractmethod
    def chunk_shape(self) -> tuple[int, ...]:
        """Shape of the chunks sent to the sidecar."""


ConfigT = TypeVar("ConfigT")


class BaseAdapterModule(nn.Module, Generic[ConfigT], ABC):
    """Container of named adapters (reference: base.py:57-90).

    Adapters live in a plain dict, not in `_modules`: the reference does the same, so an adapter's
    parameters are loaded and moved through the adapter object itself.
    """

    def __init__(self, adapter_cls: Callable[[ConfigT], nn.Module]) -> None:
        super().__init__()
        self.default_adapter_name: str | None = None
        self.adapter_cls = adapter_cls
        self.adapters: dict[str, nn.Module] = {}

    def make_adapter(self, name: str, config: ConfigT) -> nn.Module:
        if self.default_adapter_name is None:
            self.default_adapter_name = name
        adapter = self.adapter_cls(config).eval()
        self.adapters[name] = adapter
        return adapter

    def forward(self, name: str, *args: Any, **kwargs: Any):
        if name not in self.adapters:
            raise ValueError(f"Adapter '{name}' not found.")
        return self.adapters[name](*args, **kwargs)

    def named_modules(self, memo: set[nn.Module] | None = None, prefix: str = "", remove_duplicate: bool = True):
        if self.default_adapter_name is None:
            raise ValueError("No default adapter name set.")
        return self.adapters[self.default_adapter_name].named_modules(memo, prefix, remove_duplicate)


class BaseModalityProcessor:
    """Per-model preprocessing hooks (reference: base.py:93-148). Preprocessing itself is out of scope here."""

    def __init__(self, model_id: str) -> None:
        self.model_id = model_id

    def get_image_processor(self) -> Callable | None:
        return None

    def get_audio_processor(self) -> Callable | None:
        return None

    def get_video_processor(self) -> Callable | None:
        return None

    def process(self, modality: Modality, data) -> dict[str, torch.Tensor]:
        getter = {
            Modality.IMAGE: (self.get_image_processor, "Image"),
            Modality.AUDIO: (self.get_audio_processor, "Audio"),
            Modality.VIDEO: (self.get_video_processor, "Video"),
        }.get(modality)
        if getter is None:
            raise ValueError(f"Unsupported modality: {modality}")
        processor = getter[0]()
        if processor is None:
            raise ValueError(f"{getter[1]} processor not available.")
        return processor(data)


@torch.no_grad()
def fold_layernorm(w: torch.Tensor, b: torch.Tensor | None, ln_w: torch.Tensor, ln_b: torch.Tensor):
    """A LayerNorm's affine part folded into the linear layer behind it, for the GEMM that applies the
    normalisation itself (CsGemmArgs.a_row_sum):  LN(x) . W^T + b  ==  rstd * (x . W'^T - mean * colsum) + b'.
    Returns (W' = W * ln_w along the columns, b' = b + W . ln_b, colsum = row sums of the rounded W' in fp32)."""
    wf = (w.float() * ln_w.float()[None, :]).to(w.dtype)
    bf = (w.float() * ln_b.float()[None, :]).sum(dim=1)   # W . ln_b as an elementwise product and a row sum
    if b is not None:
        bf = bf + b.float()
    return wf.contiguous(), bf.to(w.dtype).contiguous(), wf.float().sum(dim=1).contiguous()
