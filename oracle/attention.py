"""Oracle: attention over packed variable-length sequences with an additive
per-key bias.  Test infrastructure only.

The reference computes ``softmax(Q K^T * scale + bias[key]) V`` independently
for every packed segment and head
(``src/cuda_extension/flash_attn/__init__.py:439-456``; the closed form its own
tests check against is ``test/auto_test/test_flex_attention_bias.py:26-36``,
evaluated in fp32 on ``.float()`` copies of the bf16 inputs, ``:231-241``).
``lse`` follows ``src/cuda_extension/flash_attn/src/softmax.h:178-183``:
``lse = logsumexp_k(scale * q.k + bias[k])``, laid out ``[H, total]``.
"""

from __future__ import annotations

import torch


def biased_varlen_attention(
    qkv: torch.Tensor,
    cu_seqlens: torch.Tensor,
    perkey_bias: torch.Tensor | None,
    softmax_scale: float | None = None,
    q_chunk: int = 2048,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``qkv [P, 3, H, D]`` (any float dtype) -> ``(out [P, H, D] fp32, lse [H, P] fp32)``.

    fp32 closed form; ``perkey_bias [P]`` may be ``None`` (plain attention).
    Queries are processed ``q_chunk`` rows at a time so the score matrix stays small.
    """
    P, three, H, D = qkv.shape
    assert three == 3
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    q, k, v = (t.float() for t in qkv.unbind(dim=1))                 # [P, H, D]
    bias = torch.zeros(P) if perkey_bias is None else perkey_bias.float()
    out = torch.zeros(P, H, D, dtype=torch.float32)
    lse = torch.full((H, P), float("inf"), dtype=torch.float32)
    bounds = [int(x) for x in cu_seqlens.tolist()]
    for s, e in zip(bounds[:-1], bounds[1:]):
        if e <= s:
            continue
        kh = k[s:e].permute(1, 2, 0)                                  # [H, D, L]
        vh = v[s:e].permute(1, 0, 2)                                  # [H, L, D]
        for c0 in range(s, e, q_chunk):
            c1 = min(e, c0 + q_chunk)
            qh = q[c0:c1].permute(1, 0, 2)                            # [H, Lq, D]
            scores = torch.matmul(qh, kh) * scale + bias[s:e][None, None, :]
            lse[:, c0:c1] = torch.logsumexp(scores, dim=-1)
            out[c0:c1] = torch.matmul(torch.softmax(scores, dim=-1), vh).permute(1, 0, 2)
    return out, lse


def biased_varlen_attention_sdpa_bf16(
    qkv: torch.Tensor,
    cu_seqlens: torch.Tensor,
    perkey_bias: torch.Tensor | None,
    softmax_scale: float | None = None,
    q_chunk: int = 4096,
) -> torch.Tensor:
    """The reference's PyTorch path for this operator on the CPU: per segment,
    ``F.scaled_dot_product_attention`` in the input dtype with the per-key bias
    passed as ``attn_mask``.  Used only as the timed CPU baseline.
    """
    P, _, H, D = qkv.shape
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    q, k, v = qkv.unbind(dim=1)
    out = torch.empty(P, H, D, dtype=qkv.dtype)
    bounds = [int(x) for x in cu_seqlens.tolist()]
    for s, e in zip(bounds[:-1], bounds[1:]):
        if e <= s:
            continue
        kh = k[s:e].transpose(0, 1).unsqueeze(0)                      # [1, H, L, D]
        vh = v[s:e].transpose(0, 1).unsqueeze(0)
        mask = None
        if perkey_bias is not None:
            mask = perkey_bias[s:e].to(qkv.dtype)[None, None, None, :]
        for c0 in range(s, e, q_chunk):
            c1 = min(e, c0 + q_chunk)
            qh = q[c0:c1].transpose(0, 1).unsqueeze(0)
            o = torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask, scale=scale)
            out[c0:c1] = o[0].transpose(0, 1)
    return out


def sdpa_bf16_chunk(qkv, perkey_bias, seg_start: int, seg_end: int, q_start: int, q_end: int, scale: float):
    """One query chunk ``[q_start, q_end)`` of the CPU baseline above against all keys of its segment
    ``[seg_start, seg_end)``; lets a caller bound the time it spends."""
    q, k, v = qkv.unbind(dim=1)
    kh = k[seg_start:seg_end].transpose(0, 1).unsqueeze(0)
    vh = v[seg_start:seg_end].transpose(0, 1).unsqueeze(0)
    mask = None if perkey_bias is None else perkey_bias[seg_start:seg_end].to(qkv.dtype)[None, None, None, :]
    qh = q[q_start:q_end].transpose(0, 1).unsqueeze(0)
    return torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask, scale=scale)[0].transpose(0, 1)
