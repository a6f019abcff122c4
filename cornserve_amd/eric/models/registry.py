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


MODEL_REGISTRY: dict[str, RegistryEntry] = {
    "qwen2_vl": RegistryEntry(
        module="qwen2_vl",
        class_name="Qwen2VisionTransformer",
        adapter_attr=None,
        vit_resolution_type=ViTResolutionType.DYNAMIC,
        weight=WeightInfo(required_prefixes=["visual."], strip_prefixes=True),
        modality={Modality.IMAGE: ModalityEntry(), Modality.VIDEO: ModalityEntry()},
    ),
    "qwen2_5_vl": RegistryEntry(
        module="qwen2_5_vl",
        class_name="Qwen2_5_VisionTransformer",
        adapter_attr=None,
        vit_resolution_type=ViTResolutionType.DYNAMIC,
        weight=WeightInfo(required_prefixes=["visual."], strip_prefixes=True),
        modality={Modality.IMAGE: ModalityEntry(), Modality.VIDEO: ModalityEntry()},
    ),
    "qwen3_vl": RegistryEntry(
        module="qwen3_vl",
        class_name="Qwen3_VisionTransformer",
        adapter_attr=None,
        vit_resolution_type=ViTResolutionType.DYNAMIC,
        weight=WeightInfo(required_prefixes=["model.visual."], strip_prefixes=True),
        modality={Modality.IMAGE: ModalityEntry(), Modality.VIDEO: ModalityEntry()},
    ),
    "qwen3_vl_moe": RegistryEntry(
        module="qwen3_vl",
        class_name="Qwen3_VisionTransformer",
        adapter_attr=None,
        vit_resolution_type=ViTResolutionType.DYNAMIC,
        weight=WeightInfo(required_prefixes=["model.visual."], strip_prefixes=True),
        modality={Modality.IMAGE: ModalityEntry(), Modality.VIDEO: ModalityEntry()},
    ),
    "llava_onevision": RegistryEntry(
        module="llava_onevision",
        class_name="LlavaOneVisionEncoder",
        adapter_attr=None,
        vit_resolution_type=ViTResolutionType.FIXED,
        weight=WeightInfo(
            required_prefixes=["vision_tower.", "multi_modal_projector.", "image_newline"],
            ignored_prefixes=["vision_tower.vision_model.post_layernorm"],
            strip_prefixes=False,
        ),
        modality={Modality.IMAGE: ModalityEntry(), Modality.VIDEO: ModalityEntry()},
    ),
    "gemma3": RegistryEntry(
        module="gemma3",
        class_name="Gemma3VisionEncoder",
        adapter_attr="multi_modal_projector",
        vit_resolution_type=ViTResolutionType.FIXED,
        weight=WeightInfo(
            required_prefixes=["vision_tower.", "multi_modal_projector."],
            ignored_prefixes=["vision_tower.vision_model.post_layernorm"],
            adapter_prefixes=["multi_modal_projector."],
            strip_prefixes=False,
        ),
        modality={Modality.IMAGE: ModalityEntry()},
    ),
}
