"""Oracle: q/k LayerNorm + 2-D rotary position embedding on packed rows.  Test infrastructure only.

Restates the inference branch of ``prepare_packed_self_attention_qkv``
(``src/accelerate/common/qkv.py:31-39``) with the reference's rotary embedding
(``src/thirdparty/vggt/layers/rope.py:100-187``): frequency tables with angles rounded to the
tensor dtype (``:100-115``), ``rotate(x) = cat(-x2, x1)`` (``:119-131``), per-direction
``x * cos + rotate(x) * sin`` evaluated with tensor operations in the tensor dtype (``:133-153``), the
first half of a head using the y coordinate and the second the x coordinate (``:176-187``).

Pinning: ``layer_norm`` is the library routine the reference calls; the rotation is not covered by a
known-answer test of the reference (PARITY UNPINNED there) and is pinned here by what the mathematics
fixes: identity at position 0, norm preservation per rotated pair, the closed-form angle of a single
pair, and the relative-position property of the q.k product (tests/test_oracle_qk_prologue.py).
"""

from __future__ import annotations

import torch


def rope_tables(head_dim: int, n_pos: int, base: float, dtype: torch.dtype):
    """cos / sin ``[n_pos, head_dim // 2]`` (``rope.py:100-115``)."""
    dim = head_dim // 2
    exponents = torch.arange(0, dim, 2).float() / dim
    inv_freq = 1.0 / (base ** exponents)
    angles = torch.einsum("i,j->ij", torch.arange(n_pos, dtype=inv_freq.dtype), inv_freq)
    angles = angles.to(dtype)
    angles = torch.cat((angles, angles), dim=-1)
    return angles.cos().to(dtype), angles.sin().to(dtype)


def _rotate(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1]
    return torch.cat((-x[..., d // 2:], x[..., : d // 2]), dim=-1)


def rope_2d(t: torch.Tensor, pos: torch.Tensor, base: float = 100.0) -> torch.Tensor:
    """``t [P, H, D]``, ``pos [P, 2]`` integer (y, x) -> rotated ``[P, H, D]`` in ``t.dtype``."""
    D = t.shape[-1]
    cos_t, sin_t = rope_tables(D, int(pos.max()) + 1 if pos.numel() else 1, base, t.dtype)
    vert, horiz = t.chunk(2, dim=-1)

    def one(x, p):
        cos = torch.nn.functional.embedding(p, cos_t)[:, None, :]
        sin = torch.nn.functional.embedding(p, sin_t)[:, None, :]
        return (x * cos) + (_rotate(x) * sin)

    return torch.cat((one(vert, pos[:, 0]), one(horiz, pos[:, 1])), dim=-1)


def qk_norm_rope(qkv: torch.Tensor, q_weight, q_bias, k_weight, k_bias, eps: float, pos, base: float = 100.0,
                 apply_norm: bool = True) -> torch.Tensor:
    """Out-of-place restatement: returns a new ``[P, 3, H, D]`` with q and k normalised over ``D``
    (``torch.nn.functional.layer_norm``) and rotated; v is copied."""
    out = qkv.clone()
    D = qkv.shape[-1]
    for idx, (w, b) in enumerate(((q_weight, q_bias), (k_weight, k_bias))):
        x = qkv[:, idx]
        if apply_norm:
            x = torch.nn.functional.layer_norm(x, (D,), w, b, eps)
        if pos is not None:
            x = rope_2d(x, pos, base).to(qkv.dtype)
        out[:, idx] = x
    return out
