"""Packed q/k preparation for the varlen attention: q/k LayerNorm + 2-D RoPE in one HIP kernel.

Mirrors ``prepare_packed_self_attention_qkv`` of the reference
(``src/accelerate/common/qkv.py:7-39``, inference branch ``:31-39``) and the parts of
``RotaryPositionEmbedding2D`` it relies on (``src/thirdparty/vggt/layers/rope.py:62-117``:
frequency tables with the angles rounded to the run dtype before cos / sin).  The packed tensor is
updated in place, as in the reference; there is no out-of-place (autograd) branch.
"""

from __future__ import annotations

import dataclasses

import torch

from .. import _lib


class RotaryPositionEmbedding2D:
    """Holds the base frequency and caches the cos / sin tables ``[n_pos, head_dim // 4]``."""

    def __init__(self, frequency: float = 100.0):
        self.base_frequency = float(frequency)
        self._cache: dict = {}

    def tables(self, head_dim: int, n_pos: int, device, dtype):
        key = (head_dim, n_pos, str(device), dtype)
        if key not in self._cache:
            half = head_dim // 2
            exponents = torch.arange(0, half, 2, device=device).float() / half
            inv_freq = 1.0 / (self.base_frequency ** exponents)
            positions = torch.arange(n_pos, device=device, dtype=inv_freq.dtype)
            angles = torch.einsum("i,j->ij", positions, inv_freq).to(dtype)
            self._cache[key] = (angles.cos().to(dtype).contiguous(), angles.sin().to(dtype).contiguous())
        return self._cache[key]


_TABLES: dict[float, RotaryPositionEmbedding2D] = {}


def _norm_params(norm):
    """LayerNorm -> (apply, weight, bias, eps); Identity / None -> no normalisation."""
    if norm is None or isinstance(norm, torch.nn.Identity):
        return False, None, None, 0.0
    if isinstance(norm, torch.nn.LayerNorm):
        return True, norm.weight, norm.bias, float(norm.eps)
    raise RuntimeError(f"q_norm / k_norm must be LayerNorm or Identity, got {type(norm).__name__}")


@dataclasses.dataclass
class DeferredQPrologue:
    """The q half of the prologue, left to the attention kernel (``come_attn_varlen_fwd_qp``): what
    ``prepare_packed_self_attention_qkv(..., defer_q=True)`` attaches to the tensor it returns as ``come_q_prologue``.
    Holds the tensors the kernel reads, so that they live as long as the packed tensor does."""
    apply_norm: bool
    eps: float
    weight: torch.Tensor | None
    bias: torch.Tensor | None
    positions: torch.Tensor | None
    cos_table: torch.Tensor | None
    sin_table: torch.Tensor | None
    n_pos: int


_BOUND_CACHE: dict = {}


def _norm_bound(weight, bias, head_dim: int, run_dtype) -> float:
    """Upper bound of the Euclidean norm of a LayerNorm'd head: ``sqrt(D) max|gain| + |bias|_2`` (the normalised
    vector has norm ``<= sqrt(D)``), with gain and bias as the kernel uses them (rounded to the run dtype).  One
    device read per parameter version, cached."""
    key = (None if weight is None else (weight.data_ptr(), weight._version),
           None if bias is None else (bias.data_ptr(), bias._version), head_dim, run_dtype)
    if key not in _BOUND_CACHE:
        if len(_BOUND_CACHE) > 4096:
            _BOUND_CACHE.clear()
        gain = 1.0 if weight is None else float(weight.detach().to(run_dtype).float().abs().max())
        shift = 0.0 if bias is None else float(bias.detach().to(run_dtype).float().norm())
        _BOUND_CACHE[key] = head_dim ** 0.5 * gain + shift
    return _BOUND_CACHE[key]


def prepare_packed_self_attention_qkv(qkv: torch.Tensor, q_norm, k_norm, rope, pos: torch.Tensor | None,
                                      run_dtype: torch.dtype, max_position: int | None = None, *,
                                      defer_q: bool = False) -> torch.Tensor:
    """Normalises the packed q and k (``qkv [P, 3, H, D]``) and applies the 2-D RoPE, in place.

    ``rope`` is an object with ``base_frequency`` or ``base`` (or ``None``), ``pos [P, 2]`` / ``[1, P, 2]`` integer
    (y, x).  ``max_position`` (largest coordinate that can occur) avoids the device-to-host read of
    ``pos.max()`` that sizes the frequency tables.

    When q and k are LayerNorm'd, the returned tensor carries ``come_qk_bound``: an upper bound of ``|q . k|`` over
    all pairs, ``(sqrt(D) max|gain_q| + |bias_q|) (sqrt(D) max|gain_k| + |bias_k|)`` (the rotation keeps norms; 2 %
    are added for its rounding).  The attention operators use it to choose how ``softmax_scale`` is applied.

    ``defer_q`` (keyword only, not in the reference; head_dim 64): only k is rewritten here; q stays the raw
    projection and the returned tensor carries ``come_q_prologue``, from which the attention operators of this
    package normalise and rotate the query rows as their kernel loads them - the same bits as the in-place pass,
    without reading and writing q once more.  For callers that hand the tensor straight to the attention operator
    (as ``bias_attention.py:100-137`` of the reference does) and read q nowhere else.
    """
    if torch.is_grad_enabled() and qkv.requires_grad:
        raise RuntimeError("prepare_packed_self_attention_qkv is forward only (in place); run it under torch.no_grad()")
    if not qkv.is_cuda:
        raise RuntimeError("qkv must be on the GPU")
    if qkv.dim() != 4 or qkv.shape[1] != 3:
        raise RuntimeError("qkv must be [P, 3, H, D]")
    if qkv.dtype != run_dtype or run_dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError("qkv must be bf16 / fp16 and match run_dtype")
    if qkv.stride(-1) != 1:
        raise RuntimeError("qkv must have unit stride in the last dimension")
    P, _, H, D = qkv.shape
    apply_q, qw, qb, q_eps = _norm_params(q_norm)
    apply_k, kw, kb, k_eps = _norm_params(k_norm)
    if apply_q != apply_k or (apply_q and q_eps != k_eps):
        raise RuntimeError("q_norm and k_norm must be the same kind of layer with the same eps")
    use_rope = rope is not None and pos is not None
    dev = qkv.device

    def as_dtype(t):
        return None if t is None else t.detach().to(device=dev, dtype=run_dtype).contiguous()

    qw, qb, kw, kb = as_dtype(qw), as_dtype(qb), as_dtype(kw), as_dtype(kb)
    positions = cos_t = sin_t = None
    n_pos = 0
    if use_rope:
        positions = pos.reshape(-1, 2).to(device=dev, dtype=torch.int64).contiguous()
        if positions.shape[0] != P:
            raise RuntimeError(f"pos must hold one (y, x) pair per packed row ({P}), got {positions.shape[0]}")
        n_pos = (int(positions.max().item()) if max_position is None else int(max_position)) + 1 if P > 0 else 1
        if not isinstance(rope, RotaryPositionEmbedding2D):
            # the reference's rope modules: RotaryPositionEmbedding2D of VGGT / DA3 (``base_frequency``,
            # thirdparty/vggt/layers/rope.py:78-83) and RoPE2D of Pi3 (``base``, thirdparty/pi3/models/layers/pos_embed.py:114-118);
            # both build the same tables and apply x cos + rotate_half(x) sin per coordinate half
            base = getattr(rope, "base_frequency", None)
            if base is None:
                base = getattr(rope, "base", None)
            if base is None:
                raise RuntimeError(f"rope must carry its base frequency as base_frequency or base, got {type(rope).__name__}")
            rope = _TABLES.setdefault(float(base), RotaryPositionEmbedding2D(float(base)))
        cos_t, sin_t = rope.tables(D, n_pos, dev, run_dtype)
    q, k = qkv[:, 0], qkv[:, 1]
    if defer_q and D != 64:
        raise RuntimeError(f"defer_q needs head_dim 64 (the attention kernel that applies the q prologue), got {D}")
    lib = _lib.load()
    with torch.cuda.device(dev):
        _lib.check(lib.come_qk_norm_rope(None if defer_q else q.data_ptr(), k.data_ptr(), _lib.dtype_code(run_dtype),
                                         q.stride(0), q.stride(1), k.stride(0), k.stride(1), P, H, D,
                                         1 if apply_q else 0, _lib.ptr(qw), _lib.ptr(qb), _lib.ptr(kw), _lib.ptr(kb),
                                         q_eps, _lib.ptr(positions), _lib.ptr(cos_t), _lib.ptr(sin_t), n_pos,
                                         _lib.current_stream(dev)))
    if apply_q:
        qkv.come_qk_bound = 1.02 * _norm_bound(q_norm.weight, q_norm.bias, D, run_dtype) * \
            _norm_bound(k_norm.weight, k_norm.bias, D, run_dtype)
    elif hasattr(qkv, "come_qk_bound"):
        del qkv.come_qk_bound
    if defer_q and (apply_q or use_rope):
        qkv.come_q_prologue = DeferredQPrologue(apply_q, q_eps, qw, qb, positions, cos_t, sin_t, n_pos)
    elif hasattr(qkv, "come_q_prologue"):
        del qkv.come_q_prologue
    return qkv
