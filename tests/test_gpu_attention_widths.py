"""GPU parity of the attention operator at head dimensions other than 64: 32 and 128 have their own kernel
instances, widths in between run zero-padded on the next one (the reference instantiates 32 ... 256,
flash_fwd_launch_template.h:174-330; its bias tests use 32 and 64, test_flex_attention_bias.py:247-266).

Checked against the fp32 closed-form oracle at the reference's tolerance (atol = rtol = 1e-2 per element) and at
the build target (max-abs <= 1e-2, mean-abs <= 1e-3).
"""

import math

import numpy as np
import pytest
import torch

import oracle
from come_amd import _lib
from come_amd.cuda_extension import (
    flash_attn_varlen_qkvpacked_func,
    flash_attn_varlen_qkvpacked_func_w_perkey_bias,
)

pytestmark = pytest.mark.gpu
DEV = "cuda"

SEGMENT_SETS = [[32, 48, 24, 24], [56, 49, 23], [128], [60, 40], [1], [3, 1, 2], [65], [129, 127], [257, 31],
                [700, 333, 64], [1000]]


def _cu(lens):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)


def _compare(out, ref, max_abs=1e-2, mean_abs=1e-3):
    out = out.float().cpu()
    diff = (out - ref).abs()
    assert float(diff.max()) <= max_abs, f"max-abs {float(diff.max())}"
    assert float(diff.mean()) <= mean_abs, f"mean-abs {float(diff.mean())}"
    torch.testing.assert_close(out, ref, atol=1e-2, rtol=1e-2)


def _inputs(lens, H, D, dtype, bias_kind, seed=0):
    g = torch.Generator().manual_seed(1000 * D + sum(lens) + seed)
    P = sum(lens)
    qkv = torch.randn(P, 3, H, D, generator=g).to(dtype)
    if bias_kind == "weights":
        bias = torch.rand(P, generator=g).clamp(min=1e-3).log().to(dtype)
    elif bias_kind == "counts":
        bias = torch.where(torch.rand(P, generator=g) < 0.3, math.log(9.0), 0.0).to(dtype)
    else:
        bias = None
    return qkv, bias, _cu(lens)


def _run(lens, H, D, dtype=torch.bfloat16, bias_kind="weights", scale=None, lse=False, max_seqlen=None):
    qkv, bias, cu = _inputs(lens, H, D, dtype, bias_kind)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias, softmax_scale=scale)
    args = (qkv.to(DEV), cu.to(DEV), max(lens) if max_seqlen is None else max_seqlen)
    if bias is None:
        res = flash_attn_varlen_qkvpacked_func(*args, softmax_scale=scale, return_attn_probs=lse)
    else:
        res = flash_attn_varlen_qkvpacked_func_w_perkey_bias(*args, perkey_bias=bias.to(DEV), softmax_scale=scale,
                                                             return_attn_probs=lse)
    if lse:
        out, got_lse, _ = res
        torch.testing.assert_close(got_lse.cpu(), ref_lse, atol=2e-3, rtol=1e-3)
    else:
        out = res
    assert out.shape == qkv[:, 0].shape and out.dtype == dtype and out.is_contiguous()
    _compare(out, ref)


@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("lens", SEGMENT_SETS, ids=str)
def test_bias_matches_closed_form(lens, D):
    _run(lens, H=3, D=D)


@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_dtypes_counts_plain_and_lse(dtype, D):
    _run([64, 64], H=4, D=D, dtype=dtype)                                   # test_flex_attention_bias.py:264-266
    _run([100, 150, 50], H=2, D=D, dtype=dtype, bias_kind="counts", lse=True)
    _run([300, 77], H=2, D=D, dtype=dtype, bias_kind=None, lse=True)


@pytest.mark.parametrize("D", [32, 128])
def test_long_segments_many_heads_and_other_scale(D):
    _run([3000, 1500], H=16, D=D, bias_kind="counts")
    _run([500, 260], H=3, D=D, scale=0.2)                                    # scale that is not a power of two
    _run([2048, 1111], H=2, D=D, lse=True, max_seqlen=5000)                  # max_seqlen is only an upper bound


@pytest.mark.parametrize("D", [32, 128])
def test_empty_segments_between_others(D):
    _run([40, 0, 90, 0], H=2, D=D, bias_kind="counts", lse=True)
    _run([0, 130], H=1, D=D, bias_kind=None)


@pytest.mark.parametrize("D", [8, 16, 24, 40, 72, 96, 120])
def test_widths_in_between_run_zero_padded(D):
    _run([56, 49, 23], H=2, D=D)
    _run([300], H=1, D=D, dtype=torch.float16, bias_kind="counts")


@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("dtype,jump", [(torch.bfloat16, 100.0), (torch.bfloat16, 300.0), (torch.float16, 12.0),
                                        (torch.float16, 30.0)], ids=["bf16+100", "bf16+300", "f16+12", "f16+30"])
def test_late_key_far_above_everything_before_it(dtype, jump, D):
    """A key whose score beats all earlier ones of its rows by `jump` nats, late in the segment: the running
    maximum has to move (and the accumulated output has to be rescaled) in the middle of the key loop."""
    L, H = 700, 2
    g = torch.Generator().manual_seed(int(jump) + D)
    qkv = torch.randn(L, 3, H, D, generator=g).to(dtype)
    bias = torch.zeros(L)
    bias[333] = jump
    bias[600] = jump - 0.5
    bias = bias.to(dtype)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, _cu([L]), bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), _cu([L]).to(DEV), L,
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True)
    assert bool(torch.isfinite(out).all())
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("D", [32, 128])
def test_growing_and_shrinking_scores(D):
    """Key norms that grow (the reference point moves again and again) or shrink (it never moves) along the segment."""
    L, H = 1500, 2
    for ramp in (torch.linspace(0.2, 5.0, L), torch.linspace(5.0, 0.2, L)):
        g = torch.Generator().manual_seed(D)
        qkv = torch.randn(L, 3, H, D, generator=g)
        qkv[:, 1] *= ramp[:, None, None]
        qkv = qkv.bfloat16()
        bias = torch.zeros(L).bfloat16()
        ref, _ = oracle.biased_varlen_attention(qkv, _cu([L]), bias)
        out = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), _cu([L]).to(DEV), L, perkey_bias=bias.to(DEV))
        _compare(out, ref, max_abs=2e-2)            # near-ties between keys of large norm: bf16 rounding of V decides


@pytest.mark.parametrize("D", [32, 128])
def test_bias_of_minus_infinity_masks_keys(D):
    L, H = 200, 2
    qkv, _, cu = _inputs([L], H, D, torch.bfloat16, None)
    bias = torch.zeros(L)
    bias[:70] = -math.inf                       # the whole first tile and a bit: rows start from masked keys only
    bias[150:] = -math.inf
    bias = bias.bfloat16()
    out = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L, perkey_bias=bias.to(DEV))
    ref, _ = oracle.biased_varlen_attention(qkv, cu, bias)
    _compare(out, ref)
    # the same rows attending to the kept keys only
    kept = qkv[70:150].float()
    scores = torch.einsum("qhd,khd->hqk", qkv[:, 0].float(), kept[:, 1]) * D ** -0.5
    want = torch.einsum("hqk,khd->qhd", torch.softmax(scores, -1), kept[:, 2])
    torch.testing.assert_close(out.float().cpu(), want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("D", [32, 128])
def test_strided_views_and_the_three_entry_points(D):
    """q, k, v as views of one wider tensor (row stride beyond 3 H D), through the C ABI directly: the plain entry,
    the one with a work buffer and the allocation-free one give the same bits (none of them uses a buffer here)."""
    lens, H = [400, 77, 300], 4
    P = sum(lens)
    g = torch.Generator().manual_seed(D)
    wide = torch.randn(P, 3 * H * D + 64, generator=g).bfloat16()
    qkv = wide[:, : 3 * H * D].view(P, 3, H, D)
    bias = torch.rand(P, generator=g).clamp(min=1e-3).log().bfloat16()
    cu = _cu(lens)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    dev_wide, dev_bias, dev_cu = wide.to(DEV), bias.to(DEV), cu.to(DEV)
    dq = dev_wide[:, : 3 * H * D].view(P, 3, H, D)
    q, k, v = dq.unbind(1)
    lib = _lib.load()
    outs = []
    for entry in ("plain", "ws", "static"):
        out = torch.empty(P, H, D, dtype=torch.bfloat16, device=DEV)
        lse = torch.empty(H, P, dtype=torch.float32, device=DEV)
        head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.dtype_code(torch.bfloat16), q.stride(0), q.stride(1),
                k.stride(0), k.stride(1), v.stride(0), v.stride(1), dev_cu.data_ptr(), len(lens), P, H, D,
                dev_bias.data_ptr(), max(lens), D ** -0.5, out.data_ptr(), out.stride(0), out.stride(1), lse.data_ptr())
        stream = _lib.current_stream(torch.device(DEV))
        if entry == "plain":
            rc = lib.come_attn_varlen_fwd(*head, 0, stream)
        elif entry == "ws":
            rc = lib.come_attn_varlen_fwd_ws(*head, None, 0, 0, stream)
        else:
            rc = lib.come_attn_varlen_fwd_static(*head, 0, stream)
        _lib.check(rc)
        torch.cuda.synchronize()
        _compare(out, ref)
        torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-3, rtol=1e-3)
        outs.append(out)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_unsupported_width_is_rejected_by_the_library():
    lib = _lib.load()
    t = torch.zeros(8, 3, 1, 96, dtype=torch.bfloat16, device=DEV)
    cu = _cu([8]).to(DEV)
    out = torch.empty(8, 1, 96, dtype=torch.bfloat16, device=DEV)
    q, k, v = t.unbind(1)
    rc = lib.come_attn_varlen_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.dtype_code(torch.bfloat16),
                                  q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
                                  cu.data_ptr(), 1, 8, 1, 96, None, 8, 0.1, out.data_ptr(), out.stride(0),
                                  out.stride(1), None, 0, _lib.current_stream(torch.device(DEV)))
    assert rc == 2                                           # COME_ERR_UNSUPPORTED
    assert b"head_dim" in lib.come_last_error()


@pytest.mark.parametrize("D,H", [(128, 8), (32, 16)])
def test_long_packed_sequences_sampled_rows(D, H):
    """Two packed sequences of 25 536 and 21 848 tokens (the lengths of the 64-wide benchmark workload), bias =
    log(count): the full fp32 oracle is too slow on a CPU at this size, so a sample of query rows is checked
    against the closed form, plus the logsumexp identity."""
    lens = [25536, 21848]
    P = sum(lens)
    g = torch.Generator().manual_seed(D)
    qkv = torch.randn(P, 3, H, D, generator=g).bfloat16()
    count = torch.ones(P)
    count[torch.randperm(P, generator=g)[:5000]] = 9.0
    bias = count.log().bfloat16()
    cu = _cu(lens)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens),
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True)
    out, lse = out.float().cpu(), lse.cpu()
    assert bool(torch.isfinite(out).all())
    q, k, v = qkv.float().unbind(1)
    for row in [0, 31, 32, 127, 128, 12345, 25535, 25536, 25537, 30000, P - 1]:
        s, e = (0, lens[0]) if row < lens[0] else (lens[0], P)
        scores = torch.einsum("hd,khd->hk", q[row], k[s:e]) * D ** -0.5 + bias.float()[None, s:e]
        ref = torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v[s:e])
        diff = (out[row] - ref).abs()
        assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3
        torch.testing.assert_close(lse[:, row], torch.logsumexp(scores, -1), atol=2e-3, rtol=1e-3)
