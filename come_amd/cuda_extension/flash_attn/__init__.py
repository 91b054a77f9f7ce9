"""Python surface of the forward-only varlen attention, mirroring
``src/cuda_extension/flash_attn/__init__.py:21-33, 235-295, 439-477`` of the reference:
``flash_attn_varlen_qkvpacked_func``, ``flash_attn_varlen_qkvpacked_func_w_perkey_bias`` and
``infer_flash_attn_varlen_max_seqlen`` with the same arguments, defaults and return values.
Calling backward raises ``RuntimeError`` (forward-only build, as in the reference).
"""

from __future__ import annotations

import torch

from . import flash_attn_fwd_cuda as _C

__all__ = [
    "flash_attn_varlen_qkvpacked_func",
    "flash_attn_varlen_qkvpacked_func_w_perkey_bias",
    "infer_flash_attn_varlen_max_seqlen",
    "FOLD_SCALE_MAX_LOGIT",
]

# How ``softmax_scale`` reaches the scores is decided per call.  The kernel's default applies it in fp32 to every
# score, as the reference's kernel does (``src/softmax.h:76-88``).  Folding it into a 16-bit q saves about 10 % of the
# run time and moves a logit by up to 2^-9 of its size, which stays inside the tolerance of the operator only while
# logits are small; it is chosen only when a bound on ``|q . k|`` is known for the call and
# ``bound * softmax_scale <= FOLD_SCALE_MAX_LOGIT`` (nats).  ``prepare_packed_self_attention_qkv`` attaches such a
# bound to the tensor it returns (attribute ``come_qk_bound``) when q and k went through LayerNorm: it follows from
# the gains and biases of the two layers alone.  Tensors without the attribute get the reference's arithmetic.
FOLD_SCALE_MAX_LOGIT = 10.0


def _fold_scale(qkv: torch.Tensor, softmax_scale: float, scale_mode: str) -> bool:
    if scale_mode == "exact":
        return False
    if scale_mode == "folded":
        return True
    if scale_mode != "auto":
        raise ValueError(f"scale_mode must be 'auto', 'exact' or 'folded', got {scale_mode!r}")
    bound = getattr(qkv, "come_qk_bound", None)
    return bound is not None and float(bound) * float(softmax_scale) <= FOLD_SCALE_MAX_LOGIT


def infer_flash_attn_varlen_max_seqlen(cu_seqlens: torch.Tensor) -> int:
    """Longest segment of ``cu_seqlens`` as a Python int (one host sync); 0 during ONNX export."""
    if torch.onnx.is_in_onnx_export():
        return 0
    return int((cu_seqlens[1:] - cu_seqlens[:-1]).max().item())


def _pad_head(t: torch.Tensor, head_size: int) -> torch.Tensor:
    if head_size % 8 != 0:
        return torch.nn.functional.pad(t, [0, 8 - head_size % 8])
    return t


def _forward(qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p, softmax_scale, causal, window_size, softcap,
             alibi_slopes, return_softmax, scale_mode="auto", work_queue=False):
    """Shared forward of the plain and the biased operator (``perkey_bias`` may be None)."""
    if softmax_scale is None:
        softmax_scale = qkv.shape[-1] ** (-0.5)
    fold = _fold_scale(qkv, softmax_scale, scale_mode)
    if len(window_size) != 2:
        raise ValueError(f"window_size must contain 2 values, got {window_size}")
    q, k, v = qkv[:, 0].detach(), qkv[:, 1].detach(), qkv[:, 2].detach()
    head_size_og = q.size(2)
    if head_size_og % 8 != 0:
        q, k, v = (_pad_head(t, head_size_og) for t in (q, k, v))
    args = (q, k, v, None, cu_seqlens, cu_seqlens, None, None, None, alibi_slopes)
    tail = (max_seqlen, max_seqlen, dropout_p, softmax_scale, False, causal, int(window_size[0]),
            int(window_size[1]), softcap, return_softmax and dropout_p > 0, None)
    # the q half of the prologue, when prepare_packed_self_attention_qkv(..., defer_q=True) left it to the kernel
    extra = dict(fold_scale=fold, work_queue=work_queue, q_prologue=getattr(qkv, "come_q_prologue", None))
    if perkey_bias is None:
        out_padded, softmax_lse, s_dmask, rng_state = _C.varlen_fwd(*args, *tail, **extra)
    else:
        out_padded, softmax_lse, s_dmask, rng_state = _C.varlen_fwd_w_perkey_bias(*args, perkey_bias, *tail, **extra)
    out = out_padded if out_padded.shape[-1] == head_size_og else out_padded[..., :head_size_og]
    return out, softmax_lse, s_dmask, rng_state


class _VarlenQKVPacked(torch.autograd.Function):
    """Records the operator in the autograd graph so that a backward pass raises, as in the reference
    (``flash_attn/__init__.py:194-200, 398-403``).  Only used when an input requires a gradient."""

    @staticmethod
    def forward(ctx, qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p, softmax_scale, causal, window_size,
                softcap, alibi_slopes, deterministic, return_softmax, is_grad_enabled, op_name, scale_mode,
                work_queue):
        ctx.op_name = op_name
        out, softmax_lse, s_dmask, rng_state = _forward(qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p,
                                                        softmax_scale, causal, window_size, softcap, alibi_slopes,
                                                        return_softmax, scale_mode, work_queue)
        ctx.mark_non_differentiable(softmax_lse, s_dmask, rng_state)
        return out if not return_softmax else (out, softmax_lse, s_dmask)

    @staticmethod
    def backward(ctx, *args):
        raise RuntimeError(f"{ctx.op_name} backward is not supported in this forward-only build.")


def _call(op_name, qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p, softmax_scale, causal, window_size, softcap,
          alibi_slopes, deterministic, return_attn_probs, scale_mode, work_queue=False):
    needs_graph = torch.is_grad_enabled() and (qkv.requires_grad
                                               or (perkey_bias is not None and perkey_bias.requires_grad))
    if needs_graph:
        return _VarlenQKVPacked.apply(qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p, softmax_scale, causal,
                                      window_size, softcap, alibi_slopes, deterministic, return_attn_probs, True,
                                      op_name, scale_mode, work_queue)
    # inference: nothing to record, skip the autograd.Function machinery (about 10 us of host time per call)
    out, softmax_lse, s_dmask, _ = _forward(qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p, softmax_scale,
                                            causal, window_size, softcap, alibi_slopes, return_attn_probs, scale_mode,
                                            work_queue)
    return out if not return_attn_probs else (out, softmax_lse, s_dmask)


def flash_attn_varlen_qkvpacked_func(qkv, cu_seqlens, max_seqlen, dropout_p=0.0, softmax_scale=None, causal=False,
                                     window_size=(-1, -1), softcap=0.0, alibi_slopes=None, deterministic=False,
                                     return_attn_probs=False, *, scale_mode="auto", work_queue=False):
    """``qkv [total, 3, nheads, headdim]``, ``cu_seqlens [batch + 1] int32`` -> ``out [total, nheads, headdim]``
    (plus ``softmax_lse [nheads, total]`` and an empty tensor when ``return_attn_probs``).

    ``scale_mode`` (keyword only, not in the reference): ``"exact"`` applies ``softmax_scale`` in fp32 to every score,
    ``"folded"`` folds it into a 16-bit q, ``"auto"`` (default) folds only for a ``qkv`` that carries a small enough
    ``come_qk_bound`` (see ``FOLD_SCALE_MAX_LOGIT``).  ``work_queue`` (keyword only): segments of at most 2048 keys are
    computed by resident workgroups that take their query blocks from a work list built on the device; same bits,
    measured slower than the default grid on every shape tried (kept for segment mixes that defeat a static grid)."""
    return _call("flash_attn_varlen_qkvpacked_func", qkv, cu_seqlens, max_seqlen, None, dropout_p, softmax_scale,
                 causal, window_size, softcap, alibi_slopes, deterministic, return_attn_probs, scale_mode, work_queue)


def flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p=0.0,
                                                   softmax_scale=None, causal=False, window_size=(-1, -1),
                                                   softcap=0.0, alibi_slopes=None, deterministic=False,
                                                   return_attn_probs=False, *, scale_mode="auto", work_queue=False):
    """Same as :func:`flash_attn_varlen_qkvpacked_func` with ``softmax(Q K^T * scale + perkey_bias[key]) V``;
    ``perkey_bias [total]`` has the dtype of ``qkv`` and is indexed like the packed keys."""
    return _call("flash_attn_varlen_qkvpacked_func_w_perkey_bias", qkv, cu_seqlens, max_seqlen, perkey_bias, dropout_p,
                 softmax_scale, causal, window_size, softcap, alibi_slopes, deterministic, return_attn_probs,
                 scale_mode, work_queue)
