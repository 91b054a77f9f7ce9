"""come_amd — MI355X (gfx950) implementation of the Co-Me accelerated-inference hot path.

Three operators, all backed by hand-written HIP kernels in ``libcome_hip.so``
(C ABI in ``include/come_hip.h``):

* confidence-guided token merge (window confidence reduction, lowest-confidence
  window selection, gather-mean into packed tokens + index map + counts + offsets),
* unmerge (gather back to the dense token grid),
* forward attention over packed variable-length sequences with an additive
  per-key bias (head_dim 64).

``come_amd.cuda_extension`` mirrors the module layout and names of the
reference's ``src/cuda_extension`` package so callers switch by changing one
import; ``come_amd.token_merger`` mirrors ``src/accelerate/token_merger``.
"""

from .interface import ITokenMerger, JaggedTokens  # noqa: F401

__version__ = "0.1.0"
