"""CPU oracle for the Co-Me hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, on the CPU and with stock torch / numpy operators, the
algorithms the reference implements in

  * ``src/accelerate/token_merger/co_me.py``     (1-D token merge / split),
  * ``src/accelerate/token_merger/co_me_2d.py``  (2-D window merge, window
    confidence reduction, lowest-confidence selection),
  * ``src/cuda_extension/flash_attn``            (varlen attention forward with
    an additive per-key bias; semantics pinned by
    ``test/auto_test/test_flex_attention_bias.py:26-36``).

Nothing in the shipped package may import it: only ``tests/``, the smoke entry
and the ``cpu_baseline`` leg of the benchmark use it, and only as the checker.

Pinning status of each function (what fixes its answers besides this text):

  token_merge_1d / token_split        the 9 known-answer cases of the
                                      reference (tests/golden/merge_1d.json),
                                      a triple-loop brute force, invariants.
  token_merge_2d                      the 3 known-answer cases of the reference
                                      (tests/golden/merge_2d.json), brute force,
                                      "permute o 1-D o unpermute" identity.
  token_merge_2d(allow_remainder)     no reference counterpart (the reference
                                      rejects ragged grids); brute force and
                                      reduction to the divisible case.
  window_confidence_means,            PARITY UNPINNED by the reference's own
  select_lowest_confidence            tests (nothing there calls build_ctx).
                                      Pinned here by library composition
                                      (torch.quantile), numpy.quantile, a sort
                                      based closed form and count identities;
                                      the normalised-score branch by a
                                      hand-computed case and an fp64 loop
                                      brute force.
  select_groups_1d                    same status (the 1-D merger's build_ctx);
                                      same pins plus its per-frame ranking /
                                      per-batch-element normalisation scope.
  biased_varlen_attention             closed form softmax(q k^T s + b) v used by
                                      the reference's tests; reductions to
                                      torch SDPA, key-duplication identity,
                                      logsumexp identity.
  add_suffix / split_suffix           the reference's 3 known-answer cases
                                      (tests/golden/suffix.json), round trip.
  qk_norm_rope / rope_2d              layer_norm is the library routine; the
                                      rotation is PARITY UNPINNED by the
                                      reference's tests and pinned here by
                                      closed forms (identity at 0, pair norms,
                                      single-pair angle, relative-position
                                      property of q.k).
"""

from .jagged import JaggedTokens, add_suffix, split_suffix  # noqa: F401
from .token_merge import (  # noqa: F401
    token_merge_1d,
    token_merge_2d,
    token_split,
    window_major_permutation,
)
from .selection import (  # noqa: F401
    window_confidence_means,
    select_lowest_confidence,
    select_groups_1d,
    quantile_threshold,
)
from .attention import (  # noqa: F401
    biased_varlen_attention,
    biased_varlen_attention_sdpa_bf16,
    sdpa_bf16_chunk,
)
from .qk_prologue import qk_norm_rope, rope_2d, rope_tables  # noqa: F401
