"""``varlen_fwd`` / ``varlen_fwd_w_perkey_bias`` on the HIP attention kernel.

Positional signatures and return lists follow the reference's pybind module
``flash_attn_fwd_cuda`` (``src/cuda_extension/flash_attn/flash_api.cpp:538-607``,
checks ``:291-408``, bias checks ``:274-288``).  Only what the Co-Me call sites
reach is implemented: fp16 / bf16, head_dim 32 / 64 / 128 (other multiples of 8 up to 128 are zero-padded to the next
of them), self-attention over one set of
``cu_seqlens``, no causal mask, no dropout, no alibi / softcap / sliding window /
paged KV / left padding.  Anything else raises ``RuntimeError`` instead of
computing something different.
"""

from __future__ import annotations

import math

import torch

from ... import _lib


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _unsupported(cond: bool, what: str) -> None:
    if cond:
        raise RuntimeError(f"come_amd flash-attention: {what} is not supported by this forward-only HIP build")


class _on_device:
    """``torch.cuda.device(dev)`` that costs nothing when ``dev`` already is the current device."""

    def __init__(self, dev: torch.device):
        self.guard = None if dev.index is None or dev.index == torch.cuda.current_device() else torch.cuda.device(dev)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            return self.guard.__exit__(*exc)
        return False


def _placeholders(dev: torch.device, dtype: torch.dtype):
    """The two results the forward never fills (attention probabilities, dropout RNG state): a fresh empty tensor
    and a fresh two-element int64 tensor per call, as the reference returns (``flash_api.cpp:470-476, 489-493``), so
    that no two callers ever hold the same object.  Neither costs a kernel launch."""
    return torch.empty((0,), dtype=dtype, device=dev), torch.empty((2,), dtype=torch.int64, device=dev)


def _varlen_fwd_impl(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table, alibi_slopes,
                     perkey_bias, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal,
                     window_size_left, window_size_right, softcap, return_softmax, gen, fold_scale=False,
                     work_queue=False, q_prologue=None):
    _check(q.dtype in (torch.float16, torch.bfloat16), "FlashAttention only support fp16 and bf16 data type")
    _check(k.dtype == q.dtype, "query and key must have the same dtype")
    _check(v.dtype == q.dtype, "query and value must have the same dtype")
    _check(cu_seqlens_q.dtype == torch.int32, "cu_seqlens_q must have dtype int32")
    _check(cu_seqlens_k.dtype == torch.int32, "cu_seqlens_k must have dtype int32")
    for name, t in (("q", q), ("k", k), ("v", v), ("cu_seqlens_q", cu_seqlens_q), ("cu_seqlens_k", cu_seqlens_k)):
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be on CUDA")
    _check(q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1,
           "Input tensor must have contiguous last dimension")
    _check(cu_seqlens_q.is_contiguous() and cu_seqlens_k.is_contiguous(), "cu_seqlens must be contiguous")
    _check(q.dim() == 3 and k.dim() == 3 and v.dim() == 3, "q, k, v must be [total, nheads, headdim]")

    _unsupported(block_table is not None, "paged KV (block_table)")
    _unsupported(seqused_k is not None, "seqused_k")
    _unsupported(leftpad_k is not None, "leftpad_k")
    _unsupported(alibi_slopes is not None, "alibi_slopes")
    _unsupported(p_dropout != 0.0, "dropout")
    _unsupported(softcap != 0.0, "softcap")
    _unsupported(return_softmax, "return_softmax")
    max_seqlen_q, max_seqlen_k = int(max_seqlen_q), int(max_seqlen_k)
    if max_seqlen_q == 1:
        is_causal = False
    _unsupported(bool(is_causal), "causal masking")
    if window_size_left >= max_seqlen_k:
        window_size_left = -1
    if window_size_right >= max_seqlen_k:
        window_size_right = -1
    _unsupported(window_size_left >= 0 or window_size_right >= 0, "sliding-window attention")

    batch_size = cu_seqlens_q.numel() - 1
    total_q, num_heads, head_size = q.shape
    total_k, num_heads_k, _ = k.shape
    _check(batch_size > 0, "batch size must be positive")
    _check(head_size <= 256, "FlashAttention forward only supports head dimension at most 256")
    _check(head_size % 8 == 0, "query, key, value, and out_ must have a head_size that is a multiple of 8")
    _check(num_heads % num_heads_k == 0, "Number of heads in key/value must divide number of heads in query")
    _check(tuple(k.shape) == (total_k, num_heads_k, head_size), "k must have shape (total_k, num_heads_k, head_size)")
    _check(tuple(v.shape) == (total_k, num_heads_k, head_size), "v must have shape (total_k, num_heads_k, head_size)")
    _check(tuple(cu_seqlens_k.shape) == (batch_size + 1,), "cu_seqlens_k must have shape (batch_size + 1)")
    _unsupported(num_heads != num_heads_k, "grouped-query attention (num_heads != num_heads_k)")
    if head_size > 128:
        _unsupported(True, f"head_dim {head_size} (32, 64, 128 and, zero-padded, other multiples of 8 up to 128 "
                           "are implemented)")
    _unsupported(total_q != total_k or max_seqlen_q != max_seqlen_k
                 or (cu_seqlens_q.data_ptr() != cu_seqlens_k.data_ptr() and not torch.equal(cu_seqlens_q, cu_seqlens_k)),
                 "cross attention (different query and key packing)")

    dev = q.device
    if perkey_bias is not None:
        if perkey_bias.dtype != q.dtype:
            raise RuntimeError(f"perkey_bias dtype must match QKV dtype ({q.dtype}), got {perkey_bias.dtype}")
        _check(perkey_bias.is_cuda, "perkey_bias must be on CUDA")
        _check(perkey_bias.is_contiguous(), "perkey_bias must be contiguous")
        if perkey_bias.dim() != 1 or perkey_bias.shape[0] != total_k:
            raise RuntimeError(f"perkey_bias must have shape (total_k,), got {tuple(perkey_bias.shape)}")

    def _aligned(t):          # the kernel issues 16-byte loads
        return t.data_ptr() % 16 == 0 and t.stride(0) % 8 == 0 and t.stride(1) % 8 == 0

    kernel_width = 32 if head_size <= 32 else 64 if head_size <= 64 else 128
    if q_prologue is not None:
        _check(head_size == 64, "a deferred q prologue needs head_dim 64")
    if head_size != kernel_width:
        # in-between widths run zero-padded on the next kernel width: zero columns change neither q . k nor the
        # other columns of the output (softmax_scale was fixed by the caller from the real width); costs a padded
        # copy of q, k, v
        padded = _varlen_fwd_impl(*(torch.nn.functional.pad(t, [0, kernel_width - head_size]) for t in (q, k, v)),
                                  None, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table, alibi_slopes,
                                  perkey_bias, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, False, is_causal,
                                  window_size_left, window_size_right, softcap, return_softmax, gen, fold_scale, work_queue, q_prologue)
        narrow = padded[0][..., :head_size]
        if out_ is not None:
            _check(out_.dtype == q.dtype and tuple(out_.shape) == (total_q, num_heads, head_size),
                   "out has the wrong shape or dtype")
            out_.copy_(narrow)
            narrow = out_
        else:
            narrow = narrow.contiguous()
        return [narrow, padded[1], padded[2], padded[3]]

    q, k, v = (t if _aligned(t) else t.contiguous() for t in (q, k, v))

    with _on_device(dev):
        if out_ is not None:
            out = out_
            _check(out.dtype == q.dtype, "Output must have the same dtype as inputs")
            _check(out.is_cuda, "out must be on CUDA")
            _check(out.stride(-1) == 1, "Output tensor must have contiguous last dimension")
            _check(tuple(out.shape) == (total_q, num_heads, head_size), "out has the wrong shape")
        else:
            out = torch.empty((total_q, num_heads, head_size), dtype=q.dtype, device=dev)
        softmax_lse = torch.empty((num_heads, total_q), dtype=torch.float32, device=dev)
        p, rng_state = _placeholders(dev, q.dtype)
        if zero_tensors:
            out.zero_()
            softmax_lse.fill_(-math.inf)
        if max_seqlen_k > 0:
            lib = _lib.load()
            # work buffer for the key-split tail of long launches (0 bytes: the launch does not use one)
            work_bytes = (lib.come_attn_work_bytes(batch_size, total_q, num_heads, max_seqlen_k)
                          if head_size == 64 else 0)
            flags = _lib.COME_ATTN_FOLD_SCALE if fold_scale else 0
            if work_queue and head_size == 64:
                work_bytes = max(work_bytes, lib.come_attn_queue_bytes(batch_size, num_heads, max_seqlen_k))
                flags |= _lib.COME_ATTN_WORK_QUEUE
            work = torch.empty(work_bytes, dtype=torch.uint8, device=dev) if work_bytes > 0 else None
            common = (q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.dtype_code(q.dtype),
                      q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
                      cu_seqlens_q.data_ptr(), batch_size, total_q, num_heads, head_size,
                      _lib.ptr(perkey_bias), max_seqlen_k, float(softmax_scale),
                      out.data_ptr(), out.stride(0), out.stride(1), softmax_lse.data_ptr(),
                      _lib.ptr(work), work_bytes)
            if q_prologue is None:
                _lib.check(lib.come_attn_varlen_fwd_ws(*common, flags, _lib.current_stream(dev)))
            else:
                qp = q_prologue
                for t in (qp.weight, qp.bias, qp.positions, qp.cos_table, qp.sin_table):
                    _check(t is None or (t.device == dev and t.is_contiguous()),
                           "the tensors of a deferred q prologue must be contiguous and on the device of q")
                _check(qp.positions is None or (qp.positions.dtype == torch.int64 and qp.positions.numel() == 2 * total_q),
                       "the positions of a deferred q prologue must be int64 [total, 2]")
                for t in (qp.weight, qp.bias, qp.cos_table, qp.sin_table):
                    _check(t is None or t.dtype == q.dtype, "the tensors of a deferred q prologue must have the dtype of q")
                desc = _lib.QPrologue(1 if qp.apply_norm else 0, float(qp.eps), _lib.ptr(qp.weight), _lib.ptr(qp.bias),
                                      _lib.ptr(qp.positions), _lib.ptr(qp.cos_table), _lib.ptr(qp.sin_table),
                                      int(qp.n_pos))
                _lib.check(lib.come_attn_varlen_fwd_qp(*common, desc, flags, _lib.current_stream(dev)))
        else:
            out.zero_()
            softmax_lse.fill_(math.inf)
    return [out, softmax_lse, p, rng_state]


def varlen_fwd(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table, alibi_slopes,
               max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal,
               window_size_left, window_size_right, softcap, return_softmax, gen=None, *, fold_scale=False,
               work_queue=False, q_prologue=None):
    """Forward pass (variable length).  Returns ``[out, softmax_lse, p, rng_state]``.

    Keyword only, not in the reference: ``fold_scale`` folds ``softmax_scale`` into a 16-bit q instead of applying
    it in fp32 to every score (``COME_ATTN_FOLD_SCALE`` of the C ABI), for callers that know their logits stay within
    about +-10 nats; ``work_queue`` runs short segments as resident workgroups fed from a device-side work list
    (``COME_ATTN_WORK_QUEUE``: same bits, slower on every shape measured, see the header); ``q_prologue`` (a
    ``come_amd.common.qkv.DeferredQPrologue``) makes the kernel normalise and rotate the query rows as it loads them
    (``come_attn_varlen_fwd_qp``: q is then the raw projection, head_dim 64 only)."""
    return _varlen_fwd_impl(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table,
                            alibi_slopes, None, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
                            zero_tensors, is_causal, window_size_left, window_size_right, softcap,
                            return_softmax, gen, fold_scale, work_queue, q_prologue)


def varlen_fwd_w_perkey_bias(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table,
                             alibi_slopes, perkey_bias, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
                             zero_tensors, is_causal, window_size_left, window_size_right, softcap,
                             return_softmax, gen=None, *, fold_scale=False, work_queue=False, q_prologue=None):
    """Forward pass (variable length) with a per-key additive bias (keywords: see :func:`varlen_fwd`)."""
    return _varlen_fwd_impl(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table,
                            alibi_slopes, perkey_bias, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
                            zero_tensors, is_causal, window_size_left, window_size_right, softcap,
                            return_softmax, gen, fold_scale, work_queue, q_prologue)
