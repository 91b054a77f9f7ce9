"""Packed ("jagged") token container of the oracle.  Test infrastructure only.

Same three fields as the reference's ``ITokenMerger.JaggedTokens``
(``src/interface/token_merger.py:12-21``): ``tokens [1, P, C]``,
``weight [P]`` (how many source tokens each packed row stands for) and
``offset [n_seg + 1]`` (segment boundaries, int64).
"""

from dataclasses import dataclass

import torch


@dataclass
class JaggedTokens:
    tokens: torch.Tensor
    weight: torch.Tensor
    offset: torch.Tensor
