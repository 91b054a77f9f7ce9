"""come_amd — MI355X (gfx950) implementation of the Co-Me accelerated-inference hot path.

Three operators, all backed by hand-written HIP kernels in ``libcome_hip.so``
(C ABI in ``include/come_hip.h``):

* confidence-guided token merge (window confidence reduction, lowest-confidence
  window selection, gather-mean into packed tokens + index map + counts + offsets),
* unmerge (gather back to the dense token grid),
* forward attention over packed variable-length sequences with an additive
  per-key bias (head_dim 64, the width of the shipped models; 32 and 128 as well).

``come_amd.cuda_extension`` mirrors the module layout and names of the
reference's ``src/cuda_extension`` package so callers switch by changing one
import; ``come_amd.token_merger`` mirrors ``src/accelerate/token_merger``,
``come_amd.common`` the q / k preparation of ``src/accelerate/common/qkv.py`` (LayerNorm +
2-D RoPE in one in-place kernel), ``come_amd.interface`` the packed-token container with its
suffix operators.  ``come_amd.harness`` is a random-init aggregator with the data flow of the
reference's fused VGGT path, used by the end-to-end tests and the benchmark.
"""

from .interface import ITokenMerger, JaggedTokens  # noqa: F401

__version__ = "0.1.0"
