"""Token mergers on the HIP kernels (mirror of ``src/accelerate/token_merger`` of the reference)."""

from .co_me import func_token_merge, func_token_split, func_token_split_pair, CoMe_TokenMerger  # noqa: F401
from .co_me_2d import (  # noqa: F401
    func_token_merge_2d,
    naive_func_token_merge_2d,
    CoMe_2D_TokenMerger,
    Naive_CoMe_2D_TokenMerger,
)
