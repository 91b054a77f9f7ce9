"""Packed ("jagged") token container and the token-merger interface.

Mirrors ``src/interface/token_merger.py:10-21, 102-116`` of the reference:
``JaggedTokens{tokens [1, P, C], weight [P], offset [n_seg + 1]}`` with its suffix operators
(``:23-100``, here one HIP kernel each) and the four methods of ``ITokenMerger``.
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

    def add_suffix(self, suffix: torch.Tensor) -> "JaggedTokens":
        """Appends ``suffix[m]`` (``suffix [M, T, C]``, weight 1) to each of the ``M`` segments
        (reference ``src/interface/token_merger.py:23-58``); one HIP kernel."""
        from . import _lib

        M = self.offset.shape[0] - 1
        if suffix.shape[0] != M:
            raise ValueError(f"suffix batch dim ({suffix.shape[0]}) must match segment count ({M})")
        _lib.require_gpu_tensor(self.tokens, "tokens")
        T, C = int(suffix.shape[1]), int(suffix.shape[2])
        tokens = self.tokens[0].contiguous()
        P = tokens.shape[0]
        if tokens.shape[1] != C:
            raise ValueError(f"suffix channels ({C}) must match the tokens' ({tokens.shape[1]})")
        dev = tokens.device
        weight = self.weight.to(device=dev, dtype=torch.float32).contiguous()
        offset = self.offset.to(device=dev, dtype=torch.int64).contiguous()
        suffix_c = suffix.to(device=dev, dtype=tokens.dtype).contiguous()
        with torch.cuda.device(dev):
            out = torch.empty(P + M * T, C, dtype=tokens.dtype, device=dev)
            out_w = torch.empty(P + M * T, dtype=torch.float32, device=dev)
            out_o = torch.empty(M + 1, dtype=torch.int64, device=dev)
            _lib.check(_lib.load().come_jagged_add_suffix(
                tokens.data_ptr(), weight.data_ptr(), _lib.dtype_code(tokens.dtype), P, C, offset.data_ptr(), M,
                suffix_c.data_ptr(), T, out.data_ptr(), out_w.data_ptr(), out_o.data_ptr(), _lib.current_stream(dev)))
        return JaggedTokens(tokens=out.unsqueeze(0), weight=out_w.to(self.weight.dtype), offset=out_o.to(self.offset.dtype))

    def split_suffix(self, count: int) -> "tuple[JaggedTokens, torch.Tensor]":
        """Strips the last ``count`` rows of every segment (inverse of ``add_suffix``; reference
        ``src/interface/token_merger.py:60-100``).  Returns ``(stripped, suffix [M, count, C])``."""
        from . import _lib

        M = self.offset.shape[0] - 1
        T, C = int(count), int(self.tokens.shape[2])
        P = int(self.tokens.shape[1])
        if P - M * T < 0:
            raise ValueError(f"Cannot strip {T} tokens from each of {M} segments (total tokens = {P})")
        seg_lens = self.offset[1:] - self.offset[:-1]
        if bool((seg_lens < T).any()):                   # the same device-to-host read the reference makes
            raise ValueError(f"count={T} exceeds the length of at least one segment")
        _lib.require_gpu_tensor(self.tokens, "tokens")
        tokens = self.tokens[0].contiguous()
        dev = tokens.device
        weight = self.weight.to(device=dev, dtype=torch.float32).contiguous()
        offset = self.offset.to(device=dev, dtype=torch.int64).contiguous()
        with torch.cuda.device(dev):
            out = torch.empty(P - M * T, C, dtype=tokens.dtype, device=dev)
            out_w = torch.empty(P - M * T, dtype=torch.float32, device=dev)
            out_o = torch.empty(M + 1, dtype=torch.int64, device=dev)
            suffix = torch.empty(M, T, C, dtype=tokens.dtype, device=dev)
            _lib.check(_lib.load().come_jagged_split_suffix(
                tokens.data_ptr(), weight.data_ptr(), _lib.dtype_code(tokens.dtype), P, C, offset.data_ptr(), M, T,
                out.data_ptr(), out_w.data_ptr(), out_o.data_ptr(), suffix.data_ptr(), _lib.current_stream(dev)))
        stripped = JaggedTokens(tokens=out.unsqueeze(0), weight=out_w.to(self.weight.dtype),
                                offset=out_o.to(self.offset.dtype))
        return stripped, suffix


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
