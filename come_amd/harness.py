"""End-to-end harness: a random-init VGGT-style alternating-attention aggregator that runs on
packed ("jagged") tokens through the merge / unmerge / biased-attention operators.

It reproduces the data flow of the reference's fused VGGT path
(``src/accelerate/vggt/fused.py:96-173``): tokens and patch positions are merged once, frame and
global attention alternate by swapping the segment offsets only (``offset`` vs every S-th entry,
``:136, 142``), each block is the pre-norm block of ``src/accelerate/vggt/module/block.py:51-81``
around the attention of ``src/accelerate/vggt/module/bias_attention.py:100-137`` (qkv Linear ->
q/k LayerNorm -> 2-D RoPE in place -> varlen attention with ``log(weight)`` per-key bias -> proj),
and the dense grid is restored only at the tap layers (``fused.py:157-165``).  Architecture
constants follow ``src/thirdparty/vggt/models/aggregator.py:51-70, 128-135`` (two variants of the
camera / register tokens: first frame and other frames, LayerScale 0.01, RoPE base 100, qk-norm).

The backbone the reference wraps (DINOv2 encoder, DPT heads, trained weights) is replaced by a
14x14 patch-embedding convolution and a light dense head; weights are random.  All operators are
injected: ``merger`` implements ``ITokenMerger``, ``attention`` has the signature of
``flash_attn_varlen_qkvpacked_func_w_perkey_bias`` and ``prologue`` that of
``prepare_packed_self_attention_qkv`` (``src/accelerate/common/qkv.py:7-39``), so the same model runs on
the HIP kernels (the default) or on any other implementation of the three interfaces.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Sequence

import torch
from torch import nn

from .interface import ITokenMerger, JaggedTokens


@dataclass
class AggregatorConfig:
    dim: int = 1024
    heads: int = 16
    mlp_dim: int = 4096
    depth: int = 24                       # frame blocks = global blocks = depth
    patch: int = 14
    registers: int = 4                    # + 1 camera token = 5 special tokens per frame
    merge_block: int = 4                  # blocks [0, merge_block) run dense, the rest packed
    taps: Sequence[int] = (4, 11, 17, 23)
    rope_base: float = 100.0
    layer_scale: float = 0.01
    head_hidden: int = 256
    conf_hidden: int = 256
    window: tuple[int, int] = (3, 3)

    @property
    def specials(self) -> int:
        return 1 + self.registers


def _default_attention(qkv, cu_seqlens, max_seqlen, perkey_bias, softmax_scale):
    from .cuda_extension import (flash_attn_varlen_qkvpacked_func,
                                 flash_attn_varlen_qkvpacked_func_w_perkey_bias)

    if perkey_bias is None:
        return flash_attn_varlen_qkvpacked_func(qkv, cu_seqlens, max_seqlen, softmax_scale=softmax_scale)
    return flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu_seqlens, max_seqlen, perkey_bias=perkey_bias,
                                                          softmax_scale=softmax_scale)


def _default_prologue(qkv, q_norm, k_norm, rope_base, pos, max_position):
    from .common import RotaryPositionEmbedding2D, prepare_packed_self_attention_qkv

    rope = _ROPES.setdefault(rope_base, RotaryPositionEmbedding2D(rope_base))
    return prepare_packed_self_attention_qkv(qkv, q_norm, k_norm, rope, pos, qkv.dtype, max_position=max_position)


def deferred_q_prologue(qkv, q_norm, k_norm, rope_base, pos, max_position):
    """The same prologue with its q half left to the attention kernel (``defer_q=True``): k is rewritten in place, q
    stays the raw projection and is normalised and rotated as the attention kernel loads it - the same bits, one read
    and one write of q less per block."""
    from .common import RotaryPositionEmbedding2D, prepare_packed_self_attention_qkv

    rope = _ROPES.setdefault(rope_base, RotaryPositionEmbedding2D(rope_base))
    return prepare_packed_self_attention_qkv(qkv, q_norm, k_norm, rope, pos, qkv.dtype, max_position=max_position,
                                             defer_q=True)


_ROPES: dict = {}


class JaggedBlock(nn.Module):
    """Pre-norm transformer block on packed tokens ``[P, C]``."""

    def __init__(self, cfg: AggregatorConfig):
        super().__init__()
        C, D = cfg.dim, cfg.dim // cfg.heads
        self.heads, self.head_dim, self.rope_base = cfg.heads, D, cfg.rope_base
        self.norm1 = nn.LayerNorm(C)
        self.qkv = nn.Linear(C, 3 * C)
        self.q_norm, self.k_norm = nn.LayerNorm(D), nn.LayerNorm(D)
        self.proj = nn.Linear(C, C)
        self.ls1 = nn.Parameter(torch.full((C,), cfg.layer_scale))
        self.norm2 = nn.LayerNorm(C)
        self.fc1, self.fc2 = nn.Linear(C, cfg.mlp_dim), nn.Linear(cfg.mlp_dim, C)
        self.ls2 = nn.Parameter(torch.full((C,), cfg.layer_scale))

    def forward(self, x, pos, max_position, cu_seqlens, max_seqlen, perkey_bias, attention, prologue) -> torch.Tensor:
        P, C = x.shape
        qkv = self.qkv(self.norm1(x)).view(P, 3, self.heads, self.head_dim)
        qkv = prologue(qkv, self.q_norm, self.k_norm, self.rope_base, pos, max_position)
        o = attention(qkv, cu_seqlens, max_seqlen, perkey_bias, self.head_dim ** -0.5)
        x = x + self.ls1 * self.proj(o.reshape(P, C).to(x.dtype))
        return x + self.ls2 * self.fc2(nn.functional.gelu(self.fc1(self.norm2(x))))


class AlternatingAggregator(nn.Module):
    """Patch embedding -> ``depth`` x (frame block, global block) -> dense head on the tap layers."""

    def __init__(self, cfg: AggregatorConfig):
        super().__init__()
        self.cfg = cfg
        C = cfg.dim
        self.patch_embed = nn.Conv2d(3, C, cfg.patch, cfg.patch)
        self.camera_token = nn.Parameter(torch.randn(1, 2, 1, C) * 1e-2)
        self.register_token = nn.Parameter(torch.randn(1, 2, cfg.registers, C) * 1e-2)
        self.frame_blocks = nn.ModuleList(JaggedBlock(cfg) for _ in range(cfg.depth))
        self.global_blocks = nn.ModuleList(JaggedBlock(cfg) for _ in range(cfg.depth))
        self.conf_fc1 = nn.Linear(C, cfg.conf_hidden)
        self.conf_fc2 = nn.Linear(cfg.conf_hidden, 1)
        self.tap_norm = nn.ModuleList(nn.LayerNorm(2 * C) for _ in cfg.taps)
        self.tap_proj = nn.ModuleList(nn.Linear(2 * C, cfg.head_hidden) for _ in cfg.taps)
        self.head_out = nn.Linear(cfg.head_hidden, cfg.patch * cfg.patch * 4)

    # ---- pieces ---------------------------------------------------------------------------
    def embed(self, images: torch.Tensor):
        """``images [B, S, 3, H, W]`` -> tokens ``[B, S, N, C]``, positions ``[B, S, N, 2]`` (y, x; specials 0,
        patches 1-based), grid ``(gh, gw)``."""
        B, S, _, H, W = images.shape
        p = self.cfg.patch
        gh, gw = H // p, W // p
        # the stride-p convolution as one GEMM over unfolded patches (same weights, same arithmetic)
        x = images.flatten(0, 1)[:, :, : gh * p, : gw * p].to(self.patch_embed.weight.dtype)
        x = x.reshape(B * S, 3, gh, p, gw, p).permute(0, 2, 4, 1, 3, 5).reshape(B * S, gh * gw, 3 * p * p)
        patches = nn.functional.linear(x, self.patch_embed.weight.flatten(1), self.patch_embed.bias)

        def first_and_others(tok):
            return torch.cat((tok[:, :1].expand(B, 1, -1, -1), tok[:, 1:].expand(B, S - 1, -1, -1)), dim=1).flatten(0, 1)

        tokens = torch.cat((first_and_others(self.camera_token), first_and_others(self.register_token), patches), dim=1)
        ys, xs = torch.meshgrid(torch.arange(gh, device=x.device), torch.arange(gw, device=x.device), indexing="ij")
        pos = torch.stack((ys, xs), dim=-1).reshape(1, gh * gw, 2) + 1
        pos = torch.cat((pos.new_zeros(1, self.cfg.specials, 2), pos), dim=1).expand(B * S, -1, -1)
        N = tokens.shape[1]
        return tokens.view(B, S, N, -1), pos.reshape(B, S, N, 2), (gh, gw)

    def confidence(self, tokens: torch.Tensor, gh: int, gw: int) -> torch.Tensor:
        """Two-layer MLP on the patch tokens -> one positive scalar per patch, ``[B*S, gh, gw]`` fp32."""
        B, S, N, C = tokens.shape
        h = nn.functional.gelu(self.conf_fc1(tokens[:, :, self.cfg.specials:]))
        logit = nn.functional.linear(h.float(), self.conf_fc2.weight.float(), self.conf_fc2.bias.float())
        return (logit.exp() + 1.0).reshape(B * S, gh, gw)

    def dense_head(self, taps: list[torch.Tensor], B: int, S: int, gh: int, gw: int) -> torch.Tensor:
        """``taps``: per tap layer ``[B*S*N, 2C]`` (frame | global features) -> maps ``[B, S, 4, gh*p, gw*p]``
        (channel 0 depth-like = exp, channels 1-3 point-like)."""
        p, s0 = self.cfg.patch, self.cfg.specials
        acc = None
        for feat, norm, proj in zip(taps, self.tap_norm, self.tap_proj):
            f = proj(norm(feat.view(B * S, -1, feat.shape[-1])[:, s0:]))
            acc = f if acc is None else acc + f
        maps = self.head_out(nn.functional.gelu(acc)).float()                            # [B*S, gh*gw, p*p*4]
        maps = maps.view(B, S, gh, gw, 4, p, p).permute(0, 1, 4, 2, 5, 3, 6).reshape(B, S, 4, gh * p, gw * p)
        return torch.cat((maps[:, :, :1].exp(), maps[:, :, 1:]), dim=2)

    # ---- forward --------------------------------------------------------------------------
    @torch.no_grad()
    def forward(self, images: torch.Tensor, merger: ITokenMerger | None = None,
                attention: Callable | None = None, prologue: Callable | None = None) -> dict:
        """Runs the aggregator.  ``merger = None``: every block on the dense token set (the unmerged baseline, same
        kernels with every count equal to 1 and no bias).  Otherwise blocks ``>= merge_block`` run on the packed
        tokens ``merger`` produces from the confidence predicted at ``merge_block``."""
        cfg = self.cfg
        attention = _default_attention if attention is None else attention
        prologue = _default_prologue if prologue is None else prologue
        tokens, pos, (gh, gw) = self.embed(images)
        B, S, N, C = tokens.shape
        dev, dtype = tokens.device, tokens.dtype
        dense_offset = torch.arange(0, B * S + 1, device=dev, dtype=torch.int64) * N

        max_position = max(gh, gw)                              # patch coordinates are 1-based, specials sit at 0
        state = dict(x=tokens.reshape(B * S * N, C), offset=dense_offset, weight=None, bias=None, ctx=None, stub=None,
                     pos=pos.reshape(-1, 2).contiguous())

        def segments():
            # the attention operator takes any upper bound of the segment lengths: the dense frame / sequence lengths
            # are known without reading the merged offsets back (the reference reads the maximum in every layer,
            # flash_attn/__init__.py:21-33)
            frame = state["offset"].to(torch.int32)
            glob = state["offset"][::S].to(torch.int32)
            return (frame, N), (glob, S * N)

        (cu_f, max_f), (cu_g, max_g) = segments()
        taps: list[torch.Tensor] = []
        info = dict(tokens_dense=B * S * N, tokens_packed=B * S * N)

        for i in range(cfg.depth):
            if merger is not None and i == cfg.merge_block:
                conf = self.confidence(state["x"].view(B, S, N, C), gh, gw)
                ctx = merger.build_ctx(torch.empty(B, S, 0, gh, gw, device=dev), confidence=conf)
                merged, stub = merger.merge(ctx, state["x"].view(B, S, N, C))
                merged_pos = merger.merge(ctx, pos.to(torch.bfloat16), stub=stub)[0].tokens.squeeze(0).long()
                state.update(x=merged.tokens.squeeze(0), offset=merged.offset, weight=merged.weight, ctx=ctx, stub=stub,
                             bias=merged.weight.float().log().to(dtype), pos=merged_pos)
                (cu_f, max_f), (cu_g, max_g) = segments()
                info.update(tokens_packed=int(merged.tokens.shape[1]), merge_mask=ctx[0] if isinstance(ctx, tuple) else None)
            x_frame = self.frame_blocks[i](state["x"], state["pos"], max_position, cu_f, max_f, state["bias"],
                                           attention, prologue)
            x_glob = self.global_blocks[i](x_frame, state["pos"], max_position, cu_g, max_g, state["bias"],
                                           attention, prologue)
            state["x"] = x_glob
            if i in cfg.taps:
                if state["ctx"] is not None:
                    def jagged(t):
                        return JaggedTokens(tokens=t.unsqueeze(0), weight=state["weight"], offset=state["offset"])
                    if hasattr(merger, "split_pair"):      # both splits and the concatenation in one launch
                        tap = merger.split_pair(state["ctx"], state["stub"], jagged(x_frame), jagged(x_glob))
                        taps.append(tap.reshape(B * S * N, 2 * C))
                    else:
                        taps.append(torch.cat([merger.split(state["ctx"], state["stub"], jagged(t))
                                               .reshape(B * S * N, C) for t in (x_frame, x_glob)], dim=-1))
                else:
                    taps.append(torch.cat((x_frame, x_glob), dim=-1))
        info["maps"] = self.dense_head(taps, B, S, gh, gw)
        info["grid"] = (gh, gw)
        return info


def relative_l1(a: torch.Tensor, b: torch.Tensor, mask: torch.Tensor | None = None) -> float:
    """``sum |a - b| / sum |b|`` over the selected elements (``mask`` broadcastable to ``a``)."""
    a, b = a.float(), b.float()
    if mask is not None:
        mask = mask.expand_as(a)
        a, b = a[mask], b[mask]
    return float((a - b).abs().sum() / b.abs().sum().clamp_min(1e-30))
