"""The one piece of Eric's API schema the model layer depends on (reference: eric/api.py:12-17)."""

from __future__ import annotations

import enum


class Modality(str, enum.Enum):
    """Modality of the data to be embedded (a str-valued enum, like the reference's StrEnum)."""

    IMAGE = "image"
    VIDEO = "video"
    AUDIO = "audio"

    def __str__(self) -> str:  # StrEnum semantics on Python 3.10
        return self.value
