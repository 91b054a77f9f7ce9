"""Token merge / split operators on HIP kernels.

Same names, argument meaning and return values as the reference's pybind module
``co_me_cuext`` (``src/cuda_extension/co_me/src/binding.cpp:33-51``,
``co_me_cuext.pyi:8-58``); argument errors raise ``RuntimeError`` as ``TORCH_CHECK``
does there (``kernel_token_merge.cu:246-261, 360-363``).  Unlike the reference the
kernels run on the current HIP stream of the tensors' device.

Two additional operators have no counterpart in the reference: the 2-D window
merge without a permuted copy (``co_me_token_merge_2d_cuda``) and the fused
confidence selection + merge (``co_me_select_merge_2d``).
"""

from __future__ import annotations

import torch

from ... import _lib

__all__ = [
    "co_me_token_merge_cuda",
    "co_me_token_split_cuda",
    "co_me_token_split_pair_cuda",
    "co_me_token_merge_2d_cuda",
    "co_me_select_windows",
    "co_me_select_merge_2d",
]


def _torch_check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _merge_impl(tokens, start_index, gh, gw, H, W, mask_u8, n_groups, tail, index_dtype, count_dtype, planned=None):
    """plan -> read P -> allocate -> merge.  Returns (out, offsets_i32, index_map, counts).
    ``planned = (offsets, prefix)``: the plan was already made on the device (``come_select_plan``)."""
    lib = _lib.load()
    dev = tokens.device
    B, N, C = tokens.shape
    with torch.cuda.device(dev):
        stream = _lib.current_stream(dev)
        if planned is None:
            offsets = torch.empty(B + 1, dtype=torch.int32, device=dev)
            prefix = torch.empty(B, max(n_groups, 1), dtype=torch.int32, device=dev)
            _lib.check(lib.come_merge_plan(_lib.ptr(mask_u8), B, n_groups, start_index, gh * gw, tail,
                                           offsets.data_ptr(), prefix.data_ptr(), stream))
        else:
            offsets, prefix = planned
        P = int(offsets[-1].item()) if B > 0 else 0          # the one host sync (output shape)
        out = torch.empty(P, C, dtype=tokens.dtype, device=dev)
        index_map = torch.empty(B * N, dtype=index_dtype, device=dev)
        counts = torch.empty(P, dtype=count_dtype, device=dev)
        rev64 = index_map.data_ptr() if index_dtype == torch.int64 else None
        rev32 = index_map.data_ptr() if index_dtype == torch.int32 else None
        w32 = counts.data_ptr() if count_dtype == torch.float32 else None
        c32 = counts.data_ptr() if count_dtype == torch.int32 else None
        _lib.check(lib.come_token_merge(tokens.data_ptr(), _lib.dtype_code(tokens.dtype), B, N, C, start_index,
                                        gh, gw, H, W, _lib.ptr(mask_u8), offsets.data_ptr(), prefix.data_ptr(),
                                        out.data_ptr(), P, rev64, rev32, w32, c32, stream))
    return out, offsets, index_map, counts


def co_me_token_merge_cuda(tokens: torch.Tensor, start_index: int, group_size: int, merge_mask: torch.Tensor):
    """Fused token merge: ``(tokens [B,N,C], start_index, G, merge_mask [B,M] bool)`` ->
    ``(out_flat [P,C], offsets [B+1] int32, rev_id [B*N] int64, weight [P] float32)``."""
    _torch_check(tokens.is_cuda, "tokens must be on CUDA")
    _torch_check(merge_mask.is_cuda, "merge_mask must be on CUDA")
    _torch_check(tokens.dim() == 3, "tokens must be [B, N, C]")
    _torch_check(merge_mask.dim() == 2, "merge_mask must be [B, M]")
    start_index, group_size = int(start_index), int(group_size)
    tokens_c = tokens.contiguous()
    mask_c = merge_mask.to(torch.bool).contiguous()
    B, N, _ = tokens_c.shape
    M = mask_c.shape[1]
    _torch_check(mask_c.shape[0] == B, "merge_mask batch != tokens batch")
    _torch_check(start_index >= 0 and group_size > 0, "start_index must be >= 0 and group_size > 0")
    _torch_check(N == start_index + M * group_size, "N != start_index + M * group_size")
    out, offsets, rev, weight = _merge_impl(tokens_c, start_index, 1, group_size, 1 if M > 0 else 0,
                                            M * group_size, mask_c.view(torch.uint8), M, 0,
                                            torch.int64, torch.float32)
    return out, offsets, rev, weight


def co_me_token_split_cuda(merged_flat: torch.Tensor, rev_id: torch.Tensor, C: int) -> torch.Tensor:
    """Token split (inverse of merge): ``out[i, :] = merged_flat[rev_id[i], :]`` -> ``[total, C]``.
    ``rev_id`` may be int64 (as in the reference) or int32."""
    _torch_check(merged_flat.is_cuda, "merged_flat must be on CUDA")
    _torch_check(rev_id.is_cuda, "rev_id must be on CUDA")
    _torch_check(merged_flat.dim() == 2, "merged_flat must be [P, C]")
    _torch_check(merged_flat.shape[1] == C, "C mismatch")
    _torch_check(rev_id.dtype in (torch.int64, torch.int32), "rev_id must be int64 or int32")
    lib = _lib.load()
    merged_c = merged_flat.contiguous()
    rev_c = rev_id.contiguous().reshape(-1)
    total = rev_c.shape[0]
    dev = merged_c.device
    with torch.cuda.device(dev):
        out = torch.empty(total, C, dtype=merged_c.dtype, device=dev)
        r64 = rev_c.data_ptr() if rev_c.dtype == torch.int64 else None
        r32 = rev_c.data_ptr() if rev_c.dtype == torch.int32 else None
        _lib.check(lib.come_token_split(merged_c.data_ptr(), _lib.dtype_code(merged_c.dtype), merged_c.shape[0], C,
                                        r64, r32, total, out.data_ptr(), _lib.current_stream(dev)))
    return out


def co_me_token_split_pair_cuda(merged_a: torch.Tensor, merged_b: torch.Tensor, rev_id: torch.Tensor,
                                C: int) -> torch.Tensor:
    """Two token splits and the concatenation of their results in one launch:
    ``out[i] = cat(merged_a[rev_id[i]], merged_b[rev_id[i]])`` -> ``[total, 2 * C]``
    (the retained-layer step of the fused aggregator, reference ``vggt/fused.py:157-165``)."""
    _torch_check(merged_a.is_cuda and merged_b.is_cuda, "merged_a and merged_b must be on CUDA")
    _torch_check(rev_id.is_cuda, "rev_id must be on CUDA")
    _torch_check(merged_a.dim() == 2 and merged_a.shape[1] == C, "merged_a must be [P, C]")
    _torch_check(merged_b.shape == merged_a.shape and merged_b.dtype == merged_a.dtype
                 and merged_b.device == merged_a.device, "merged_b must match merged_a in shape, dtype and device")
    _torch_check(rev_id.dtype in (torch.int64, torch.int32), "rev_id must be int64 or int32")
    lib = _lib.load()
    a_c, b_c = merged_a.contiguous(), merged_b.contiguous()
    rev_c = rev_id.contiguous().reshape(-1)
    total = rev_c.shape[0]
    dev = a_c.device
    with torch.cuda.device(dev):
        out = torch.empty(total, 2 * C, dtype=a_c.dtype, device=dev)
        r64 = rev_c.data_ptr() if rev_c.dtype == torch.int64 else None
        r32 = rev_c.data_ptr() if rev_c.dtype == torch.int32 else None
        _lib.check(lib.come_token_split_pair(a_c.data_ptr(), b_c.data_ptr(), _lib.dtype_code(a_c.dtype),
                                             a_c.shape[0], C, r64, r32, total, out.data_ptr(),
                                             _lib.current_stream(dev)))
    return out


def co_me_token_merge_cuda_legacy(*args, **kwargs):
    """The reference still exports its first-generation pair (``co_me_cuext.pyi:22-46``) but calls it nowhere;
    it is not provided here."""
    raise RuntimeError("co_me_token_merge_cuda_legacy is not provided by the HIP build: use co_me_token_merge_cuda")


def co_me_token_merge_scan_legacy(*args, **kwargs):
    """See ``co_me_token_merge_cuda_legacy``."""
    raise RuntimeError("co_me_token_merge_scan_legacy is not provided by the HIP build: use co_me_token_merge_cuda")


def co_me_token_merge_2d_cuda(tokens: torch.Tensor, start_index: int, group_h: int, group_w: int, H: int, W: int,
                              merge_mask: torch.Tensor, index_dtype: torch.dtype = torch.int64,
                              count_dtype: torch.dtype = torch.float32):
    """2-D window merge straight from the image row-major token order (no permuted copy).

    ``tokens [B, start_index + H*W, C]``, ``merge_mask [B, (H//gh)*(W//gw)] bool``.  Grid positions
    outside the full windows are copied behind the windows.  Returns
    ``(out_flat [P,C], offsets [B+1] int32, index_map [B*N], counts [P])``.
    """
    _torch_check(tokens.is_cuda and merge_mask.is_cuda, "tokens and merge_mask must be on CUDA")
    _torch_check(tokens.dim() == 3 and merge_mask.dim() == 2, "tokens must be [B, N, C], merge_mask [B, M]")
    start_index, group_h, group_w, H, W = int(start_index), int(group_h), int(group_w), int(H), int(W)
    _torch_check(start_index >= 0 and group_h > 0 and group_w > 0 and H >= 0 and W >= 0, "bad geometry")
    tokens_c = tokens.contiguous()
    mask_c = merge_mask.to(torch.bool).contiguous()
    B, N, _ = tokens_c.shape
    M = (H // group_h) * (W // group_w)
    _torch_check(mask_c.shape[0] == B, "merge_mask batch != tokens batch")
    _torch_check(N == start_index + H * W, "N != start_index + H * W")
    _torch_check(mask_c.shape[1] == M, "M != (H // group_h) * (W // group_w)")
    tail = H * W - M * group_h * group_w
    return _merge_impl(tokens_c, start_index, group_h, group_w, H, W, mask_c.view(torch.uint8), M, tail,
                       index_dtype, count_dtype)


_MODES = {"pairwise-rank": 0, "abs_mse": 1, "mse": 2}


def co_me_select_windows(conf: torch.Tensor, batch: int, group_h: int, group_w: int, threshold: float,
                         mode: str = "pairwise-rank", return_means: bool = False):
    """Window confidence means + lowest-confidence selection.

    ``conf [batch*frames, H, W]`` bf16 or fp32 -> ``mask [batch*frames, M] bool``
    (and the window means as float32 when ``return_means``).
    """
    _torch_check(conf.is_cuda, "conf must be on CUDA")
    _torch_check(conf.dim() == 3, "conf must be [B*S, H, W]")
    _torch_check(mode in _MODES, f"unsupported confidence mode {mode!r}")
    _torch_check(conf.dtype in (torch.bfloat16, torch.float32), "conf must be bfloat16 or float32")
    rows, H, W = conf.shape
    _torch_check(batch > 0 and rows % batch == 0, "conf rows must be a multiple of batch")
    lib = _lib.load()
    conf_c = conf.contiguous()
    dev = conf.device
    M = (H // group_h) * (W // group_w)
    with torch.cuda.device(dev):
        mask = torch.empty(rows, M, dtype=torch.bool, device=dev)
        means = torch.empty(rows, M, dtype=torch.float32, device=dev)
        _lib.check(lib.come_select_windows(conf_c.data_ptr(), _lib.dtype_code(conf_c.dtype), batch, rows // batch,
                                           H, W, group_h, group_w, _MODES[mode], float(threshold),
                                           means.data_ptr(), mask.data_ptr(), None, 0, _lib.current_stream(dev)))
    return (mask, means) if return_means else mask


def co_me_select_merge_2d(tokens: torch.Tensor, conf: torch.Tensor, batch: int, start_index: int, group_h: int,
                          group_w: int, H: int, W: int, ratio: float, index_dtype: torch.dtype = torch.int32,
                          count_dtype: torch.dtype = torch.int32, mode: str = "pairwise-rank"):
    """Confidence-guided merge in one call: window means -> joint lowest-``ratio`` selection per
    batch element -> merge plan (one launch for all three when ``batch == 1``) -> gather-mean.  Returns
    ``(merged [P,C], index_map [B_eff*N], counts [P], cu_seqlens [B_eff+1] int32, mask [B_eff,M] bool)``.
    """
    _torch_check(tokens.is_cuda and conf.is_cuda, "tokens and conf must be on CUDA")
    _torch_check(tokens.dim() == 3, "tokens must be [B, N, C]")
    _torch_check(mode in _MODES, f"unsupported confidence mode {mode!r}")
    _torch_check(conf.dtype in (torch.bfloat16, torch.float32), "conf must be bfloat16 or float32")
    start_index, group_h, group_w, H, W = int(start_index), int(group_h), int(group_w), int(H), int(W)
    _torch_check(start_index >= 0 and group_h > 0 and group_w > 0 and H >= 0 and W >= 0, "bad geometry")
    rows, N, _ = tokens.shape
    M = (H // group_h) * (W // group_w)
    _torch_check(N == start_index + H * W, "N != start_index + H * W")
    _torch_check(batch > 0 and rows % batch == 0, "token rows must be a multiple of batch")
    _torch_check(conf.numel() == rows * H * W, "conf must hold one value per grid position")
    if M == 0 or rows == 0:         # nothing to select from: every token is kept
        mask = torch.zeros(rows, M, dtype=torch.bool, device=tokens.device)
        out, offsets, index_map, counts = co_me_token_merge_2d_cuda(tokens, start_index, group_h, group_w, H, W, mask,
                                                                     index_dtype=index_dtype, count_dtype=count_dtype)
        return out, index_map, counts, offsets, mask
    lib = _lib.load()
    dev = tokens.device
    tokens_c = tokens.contiguous()
    conf_c = conf.reshape(rows, H, W).contiguous()
    with torch.cuda.device(dev):
        mask = torch.empty(rows, M, dtype=torch.bool, device=dev)
        means = torch.empty(rows, M, dtype=torch.float32, device=dev)
        offsets = torch.empty(rows + 1, dtype=torch.int32, device=dev)
        prefix = torch.empty(rows, M, dtype=torch.int32, device=dev)
        _lib.check(lib.come_select_plan(conf_c.data_ptr(), _lib.dtype_code(conf_c.dtype), batch, rows // batch, H, W,
                                        group_h, group_w, _MODES[mode], float(ratio), start_index, means.data_ptr(),
                                        mask.data_ptr(), offsets.data_ptr(), prefix.data_ptr(), None, 0,
                                        _lib.current_stream(dev)))
    tail = H * W - M * group_h * group_w
    out, offsets, index_map, counts = _merge_impl(tokens_c, start_index, group_h, group_w, H, W, mask.view(torch.uint8),
                                                  M, tail, index_dtype, count_dtype, planned=(offsets, prefix))
    return out, index_map, counts, offsets, mask
