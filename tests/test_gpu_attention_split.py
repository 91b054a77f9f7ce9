"""Key-split tail of long launches (come_attn_varlen_fwd_ws): the query blocks of the partly filled last round of
workgroups are computed in several pieces over the keys and combined.  Checked against the closed form on
sampled rows and against the single-pass entry point (come_attn_varlen_fwd) on every row."""

import numpy as np
import pytest
import torch

from come_amd import _lib
from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias

pytestmark = pytest.mark.gpu
DEV = "cuda"
H, D = 16, 64


def single_pass(qkv, cu, max_len, bias):
    """The entry point without a work buffer."""
    lib = _lib.load()
    P = qkv.shape[0]
    q, k, v = qkv.unbind(1)
    out = torch.empty(P, H, D, dtype=qkv.dtype, device=qkv.device)
    lse = torch.empty(H, P, dtype=torch.float32, device=qkv.device)
    _lib.check(lib.come_attn_varlen_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.dtype_code(qkv.dtype),
                                        q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
                                        cu.data_ptr(), cu.numel() - 1, P, H, D, bias.data_ptr(), max_len, 0.125,
                                        out.data_ptr(), out.stride(0), out.stride(1), lse.data_ptr(), 0,
                                        _lib.current_stream(qkv.device)))
    return out, lse


@pytest.mark.parametrize("lens", [[9000], [6000, 5000], [9000, 700], [9000, 300], [25536]], ids=str)
def test_split_tail_matches_single_pass_and_closed_form(lens):
    lib = _lib.load()
    P = sum(lens)
    assert lib.come_attn_work_bytes(len(lens), P, H, max(lens)) > 0, "this shape is meant to use the key-split tail"
    g = torch.Generator().manual_seed(len(lens) * 1000 + lens[-1])
    qkv = torch.randn(P, 3, H, D, generator=g).bfloat16()
    bias = (torch.rand(P, generator=g) * 3).log().clamp(min=-4).bfloat16()
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens), perkey_bias=bias.to(DEV),
                                                                 softmax_scale=0.125, return_attn_probs=True)
    ref_out, ref_lse = single_pass(qkv.to(DEV), cu.to(DEV), max(lens), bias.to(DEV))
    assert bool(torch.isfinite(out).all())
    # the two entry points sum the same products in a different order
    torch.testing.assert_close(out.float(), ref_out.float(), atol=4e-3, rtol=2 ** -7)
    torch.testing.assert_close(lse, ref_lse, atol=2e-3, rtol=1e-4)
    # sampled rows (first and last rows of every segment, block borders of the tail) against the closed form
    out, lse = out.float().cpu(), lse.cpu()
    q, k, v = qkv.float().unbind(1)
    start = 0
    for L in lens:
        for local in sorted({0, L // 2, max(L - 1025, 0), max(L - 513, 0), max(L - 512, 0), L - 1}):
            row = start + local
            scores = torch.einsum("hd,khd->hk", q[row], k[start:start + L]) * 0.125 + bias.float()[None, start:start + L]
            ref = torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v[start:start + L])
            diff = (out[row] - ref).abs()
            assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3
            torch.testing.assert_close(lse[:, row], torch.logsumexp(scores, -1), atol=2e-3, rtol=1e-3)
        start += L


def test_work_buffer_rules():
    lib = _lib.load()
    assert lib.come_attn_work_bytes(1, 2000, 16, 2000) == 0          # short segments never split
    assert lib.come_attn_work_bytes(2, 47384, 16, 25536) == 0        # the benchmark shape fills its last round
    need = lib.come_attn_work_bytes(1, 9000, 16, 9000)
    assert need > 0
    # a buffer that is too small is ignored: same result as the single-pass entry point, bit for bit
    P = 9000
    qkv = torch.randn(P, 3, H, D, generator=torch.Generator().manual_seed(1)).bfloat16().to(DEV)
    bias = torch.zeros(P, dtype=torch.bfloat16, device=DEV)
    cu = torch.tensor([0, P], dtype=torch.int32, device=DEV)
    ref_out, _ = single_pass(qkv, cu, P, bias)
    q, k, v = qkv.unbind(1)
    out = torch.empty(P, H, D, dtype=qkv.dtype, device=DEV)
    small = torch.empty(1024, dtype=torch.uint8, device=DEV)
    _lib.check(lib.come_attn_varlen_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.COME_BF16, q.stride(0), q.stride(1),
                                           k.stride(0), k.stride(1), v.stride(0), v.stride(1), cu.data_ptr(), 1, P, H, D,
                                           bias.data_ptr(), P, 0.125, out.data_ptr(), out.stride(0), out.stride(1), None,
                                           small.data_ptr(), small.numel(), 0, _lib.current_stream(qkv.device)))
    assert torch.equal(out, ref_out)


@pytest.mark.parametrize("lens", [[700, 300, 812], [9000, 700], [6000, 5000]], ids=str)
def test_max_seqlen_may_be_any_upper_bound(lens):
    """A caller that does not want to read the longest segment back from the device (the per-layer ``.item()`` of
    reference flash_attn/__init__.py:21-33) passes a static bound such as the unmerged frame length or the total."""
    P = sum(lens)
    g = torch.Generator().manual_seed(P)
    qkv = torch.randn(P, 3, H, D, generator=g).bfloat16().to(DEV)
    bias = (torch.rand(P, generator=g) * 3).log().clamp(min=-4).bfloat16().to(DEV)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32).to(DEV)
    exact, exact_lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, max(lens), perkey_bias=bias,
                                                                        softmax_scale=0.125, return_attn_probs=True)
    for bound in (max(lens) + 1, max(lens) + 700, P, 2 * P):
        out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, bound, perkey_bias=bias,
                                                                     softmax_scale=0.125, return_attn_probs=True)
        # the launch plan (workgroup width, key-split tail) may differ with the bound: same products, other order
        torch.testing.assert_close(out.float(), exact.float(), atol=4e-3, rtol=2 ** -7)
        torch.testing.assert_close(lse, exact_lse, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("width", [64, 32, 128])
def test_every_block_count_covers_every_query_block_once(width):
    """The order in which a launch visits the query blocks of a unit depends on the parity of the block count
    (``max_seqlen`` / block rows): whatever the bound, every block is computed exactly once and the bits are the
    same.  Unit counts that are not multiples of 8 and a segment shorter than one block are included."""
    lens = [300, 77, 812, 5, 640]
    heads = 3
    P = sum(lens)
    g = torch.Generator().manual_seed(width)
    qkv = torch.randn(P, 3, heads, width, generator=g).bfloat16().to(DEV)
    bias = (torch.rand(P, generator=g) * 3).log().clamp(min=-4).bfloat16().to(DEV)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32).to(DEV)
    tight, tight_lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, max(lens), perkey_bias=bias,
                                                                        return_attn_probs=True)
    rows = 256 if width == 64 else 128
    for extra in range(1, 10):
        out = torch.full_like(tight, float("nan"))
        got, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, max(lens) + extra * rows,
                                                                     perkey_bias=bias, return_attn_probs=True)
        out.copy_(got)
        assert torch.equal(out, tight), f"{extra} more block rows"
        assert torch.equal(lse, tight_lse)
