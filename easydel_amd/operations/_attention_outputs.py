"""Result container of attention operations (reference ``easydel/operations/_attention_outputs.py:56-111``)."""

from __future__ import annotations

import typing as tp
from dataclasses import dataclass


@dataclass
class AttentionOutput:
    attention_weights: tp.Any | None = None
    attention_outputs: tp.Any | None = None
    cache_view: tp.Any | None = None
