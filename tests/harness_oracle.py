"""Oracle-backed operators for the end-to-end harness: the same two interfaces the HIP path
implements (``ITokenMerger``, the varlen attention callable and the q/k prologue), built on ``oracle/`` only."""

from __future__ import annotations

import torch

import oracle
from come_amd.interface import ITokenMerger, JaggedTokens


class OracleMerger(ITokenMerger):
    def __init__(self, start_idx: int, group_h: int, group_w: int, threshold: float):
        self.start_idx, self.group_h, self.group_w, self.threshold = start_idx, group_h, group_w, threshold

    def build_ctx(self, feature, confidence=None):
        B, S, C, H, W = feature.shape
        mask = oracle.select_lowest_confidence(confidence.reshape(B * S, H, W).cpu(), B, self.group_h, self.group_w,
                                               self.threshold)
        return mask, (B, S, C, H, W)

    def merge(self, ctx, tokens, stub=None, *, start_index=None):
        mask, (B, S, C, H, W) = ctx
        jag, rev = oracle.token_merge_2d(tokens.flatten(0, 1).cpu(), self.start_idx, self.group_h, self.group_w, H, W,
                                         mask, allow_remainder=True)
        dev = tokens.device
        out = JaggedTokens(tokens=jag.tokens.to(dev), weight=jag.weight.to(dev), offset=jag.offset.to(dev))
        return out, (rev, tokens.shape)

    def split(self, ctx, stub, tokens):
        rev, shape = stub
        jag = oracle.JaggedTokens(tokens=tokens.tokens.cpu(), weight=tokens.weight.cpu(), offset=tokens.offset.cpu())
        return oracle.token_split(jag, rev, tuple(shape)).to(tokens.tokens.device)

    def build_infer_mask(self, ctx):
        raise NotImplementedError


def oracle_attention(qkv, cu_seqlens, max_seqlen, perkey_bias, softmax_scale):
    out, _ = oracle.biased_varlen_attention(qkv.cpu(), cu_seqlens.cpu(), None if perkey_bias is None else perkey_bias.cpu(),
                                            softmax_scale)
    return out.to(device=qkv.device, dtype=qkv.dtype)


def oracle_prologue(qkv, q_norm, k_norm, rope_base, pos, max_position):
    out = oracle.qk_norm_rope(qkv.cpu(), q_norm.weight.cpu(), q_norm.bias.cpu(), k_norm.weight.cpu(), k_norm.bias.cpu(),
                              q_norm.eps, pos.cpu(), rope_base)
    return out.to(qkv.device)
