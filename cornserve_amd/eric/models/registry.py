"""Registry entries for the MI355X-native encoders (reference: eric/models/registry.py:11-233).

Same record types and the same entries the reference keeps for these model types, so that
`loader.load_model` (eric/executor/loader.py:62-96) can resolve them by `hf_config.model_type`.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, field

from cornserve_amd.eric.api import Modality


@dataclass
class WeightInfo:
    required_prefixes: list[str]
    ignored_prefixes: list[str] = field(default_factory=list)
    adapter_prefixes: list[str] = field(default_factory=list)
    strip_prefixes: bool = True


class ViTResolutionType(enum.Enum):
    FIXED = "fixed"
    DYNAMIC = "dynamic"


@dataclass
class ModalityEntry:
    """Modality entry for a model class."""


@dataclass
class RegistryEntry:
    module: str
    class_name: str
    adapter_attr: str | None
    vit_resolution_type: ViTResolutionType
    weight: WeightInfo
    modality: dict[Modality, ModalityEntry]

    def __post_init__(self) -> None:
        if self.adapter_attr is not None and not self.weight.adapter_prefixes:
            raise ValueError(f"Registry entry for {self.class_name} must have `adapter_prefixes` set if `adapter_attr` is specified.")
        if self.adapter_attr is None and self.weight.adapter_prefixes:
            raise ValueError(f"Registry entry for {self.class_name} must have `adapter_attr` set if `adapter_prefixes` is specified.")


def _entry(module: str, class_name: str, resolution: ViTResolutionType, required: list[str],
           modalities: tuple[Modality, ...], *, strip: bool = True, ignored: tuple[str, ...] = (),
           adapter_attr: str | None = None, adapter_prefixes: tuple[str, ...] = ()) -> RegistryEntry:
    weight = WeightInfo(required_prefixes=list(required), ignored_prefixes=list(ignored),
                        adapter_prefixes=list(adapter_prefixes), strip_prefixes=strip)
    return RegistryEntry(module=module, class_name=class_name, adapter_attr=adapter_attr, vit_resolution_type=resolution,
                         weight=weight, modality={m: ModalityEntry() for m in modalities})


_IMAGE_VIDEO = (Modality.IMAGE, Modality.VIDEO)
_SIGLIP_POST_NORM = ("vision_tower.vision_model.post_layernorm",)

# model_type of the checkpoint's config.json -> how to build and fill the encoder (the reference's entries for the
# encoders built here, registry.py:59-233: same modules, class names, prefixes and modalities).
MODEL_REGISTRY: dict[str, RegistryEntry] = {
    "qwen2_vl": _entry("qwen2_vl", "Qwen2VisionTransformer", ViTResolutionType.DYNAMIC, ["visual."], _IMAGE_VIDEO),
    "qwen2_5_vl": _entry("qwen2_5_vl", "Qwen2_5_VisionTransformer", ViTResolutionType.DYNAMIC, ["visual."], _IMAGE_VIDEO),
    "qwen3_vl": _entry("qwen3_vl", "Qwen3_VisionTransformer", ViTResolutionType.DYNAMIC, ["model.visual."], _IMAGE_VIDEO),
    "qwen3_vl_moe": _entry("qwen3_vl", "Qwen3_VisionTransformer", ViTResolutionType.DYNAMIC, ["model.visual."], _IMAGE_VIDEO),
    "llava_onevision": _entry("llava_onevision", "LlavaOneVisionEncoder", ViTResolutionType.FIXED,
                              ["vision_tower.", "multi_modal_projector.", "image_newline"], _IMAGE_VIDEO,
                              strip=False, ignored=_SIGLIP_POST_NORM),
    "gemma3": _entry("gemma3", "Gemma3VisionEncoder", ViTResolutionType.FIXED, ["vision_tower.", "multi_modal_projector."],
                     (Modality.IMAGE,), strip=False, ignored=_SIGLIP_POST_NORM, adapter_attr="multi_modal_projector",
                     adapter_prefixes=("multi_modal_projector.",)),
}
