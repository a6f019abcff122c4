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
    """Named adapters behind one module (the interface of reference base.py:57-90: `make_adapter`, call by name,
    `named_modules` of the default adapter, which is the first one made).

    The adapters are kept in an insertion-ordered dict outside `_modules`, so `state_dict()` / `.to()` of the
    enclosing model do not see them: weights are loaded into, and moved with, each adapter object on its own, as the
    reference's loader expects."""

    def __init__(self, adapter_cls: Callable[[ConfigT], nn.Module]) -> None:
        super().__init__()
        self.adapter_cls = adapter_cls
        self.adapters: dict[str, nn.Module] = {}

    @property
    def default_adapter_name(self) -> str | None:
        return next(iter(self.adapters), None)

    def _adapter(self, name: str | None) -> nn.Module:
        try:
            return self.adapters[name]   # type: ignore[index]
        except KeyError:
            known = ", ".join(self.adapters) or "none made yet"
            raise ValueError(f"adapter {name!r} not found (adapters: {known})") from None

    def make_adapter(self, name: str, config: ConfigT) -> nn.Module:
        self.adapters[name] = self.adapter_cls(config).eval()
        return self.adapters[name]

    def forward(self, name: str, *args: Any, **kwargs: Any):
        return self._adapter(name)(*args, **kwargs)

    def named_modules(self, memo: set[nn.Module] | None = None, prefix: str = "", remove_duplicate: bool = True):
        return self._adapter(self.default_adapter_name).named_modules(memo, prefix, remove_duplicate)


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
