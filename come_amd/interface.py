"""Packed ("jagged") token container and the token-merger interface.

Mirrors ``src/interface/token_merger.py:10-21, 102-116`` of the reference:
``JaggedTokens{tokens [1, P, C], weight [P], offset [n_seg + 1]}`` and the four
methods of ``ITokenMerger``.
"""

from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Any, Callable

import torch


@dataclass
class JaggedTokens:
    tokens: torch.Tensor      # [1, P, C]
    weight: torch.Tensor      # [P]   source tokens per packed row (1 or the window size)
    offset: torch.Tensor      # [n_seg + 1] int64 segment boundaries

    def apply(self, func: Callable[[torch.Tensor], torch.Tensor]) -> "JaggedTokens":
        return JaggedTokens(tokens=func(self.tokens), weight=self.weight, offset=self.offset)


class ITokenMerger(ABC):
    JaggedTokens = JaggedTokens

    @abstractmethod
    def build_ctx(self, feature: torch.Tensor, confidence: torch.Tensor | None = None) -> Any: ...

    @abstractmethod
    def merge(self, ctx: Any, tokens: torch.Tensor, stub: Any | None = None, *,
              start_index: int | None = None) -> tuple[JaggedTokens, Any]: ...

    @abstractmethod
    def split(self, ctx: Any, stub: Any, tokens: JaggedTokens) -> torch.Tensor: ...

    @abstractmethod
    def build_infer_mask(self, ctx: Any) -> torch.Tensor: ...
