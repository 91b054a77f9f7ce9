"""GPU parity: forward varlen attention with a per-key bias through the C-ABI library
against the fp32 closed-form oracle.

Tolerances: the reference's own test uses atol = rtol = 1e-2 per element
(test_flex_attention_bias.py:20-21); the build target is max-abs <= 1e-2 and
mean-abs <= 1e-3 in bf16.  Both are asserted.
"""

import math

import numpy as np
import pytest
import torch

import oracle
from come_amd.cuda_extension import (
    flash_attn_varlen_qkvpacked_func,
    flash_attn_varlen_qkvpacked_func_w_perkey_bias,
    infer_flash_attn_varlen_max_seqlen,
)
from come_amd.cuda_extension.flash_attn import flash_attn_fwd_cuda

pytestmark = pytest.mark.gpu
DEV = "cuda"
MAX_ABS, MEAN_ABS = 1e-2, 1e-3

SEGMENT_SETS = [[32, 48, 24, 24], [56, 49, 23], [128], [60, 40], [50], [128, 256], [100, 150, 50], [64] * 4,
                [1], [3, 1, 2], [65], [257, 31], [700, 333, 64], [1000]]


# How softmax_scale reaches the scores is a per-call choice (``scale_mode``): "exact" - in fp32 on every score, the
# reference's arithmetic and what a tensor without a known logit bound gets ("auto"); "folded" - multiplied into a
# 16-bit q once, for logits within about +-10 nats.  Cases whose logits stay small run in both.
MODES = ["exact", "folded"]


def _cu(lens):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)


def _compare(out, ref):
    out = out.float().cpu()
    diff = (out - ref).abs()
    assert float(diff.max()) <= MAX_ABS, f"max-abs {float(diff.max())}"
    assert float(diff.mean()) <= MEAN_ABS, f"mean-abs {float(diff.mean())}"
    torch.testing.assert_close(out, ref, atol=1e-2, rtol=1e-2)


def _run(lens, H, dtype, bias_kind="weights", scale=None, return_lse=False, mode="auto"):
    P, D = sum(lens), 64
    qkv = torch.randn(P, 3, H, D).to(dtype)
    if bias_kind == "weights":
        bias = torch.rand(P).clamp(min=1e-3).log().to(dtype)
    elif bias_kind == "counts":
        bias = torch.where(torch.rand(P) < 0.3, math.log(9.0), 0.0).to(dtype)
    else:
        bias = None
    cu = _cu(lens)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias, softmax_scale=scale)
    args = (qkv.to(DEV), cu.to(DEV), max(lens))
    if bias is None:
        res = flash_attn_varlen_qkvpacked_func(*args, softmax_scale=scale, return_attn_probs=return_lse,
                                               scale_mode=mode)
    else:
        res = flash_attn_varlen_qkvpacked_func_w_perkey_bias(*args, perkey_bias=bias.to(DEV), softmax_scale=scale,
                                                             return_attn_probs=return_lse, scale_mode=mode)
    if return_lse:
        out, lse, _ = res
        # folded: the scaled q is rounded to 16 bits, a logit (and with it lse) moves by up to 2^-9 of its size
        torch.testing.assert_close(lse.cpu(), ref_lse, atol=1e-2 if mode == "folded" else 2e-3, rtol=1e-3)
    else:
        out = res
    assert out.shape == (P, H, D) and out.dtype == dtype
    _compare(out, ref)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("lens", SEGMENT_SETS, ids=[str(s) for s in SEGMENT_SETS])
def test_bias_matches_closed_form_bf16(lens, mode):
    _run(lens, H=4, dtype=torch.bfloat16, mode=mode, return_lse=True)


@pytest.mark.parametrize("mode", ["auto"] + MODES)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_dtypes(dtype, mode):
    _run([64, 64], H=4, dtype=dtype, mode=mode)
    _run([100, 150, 50], H=2, dtype=dtype, bias_kind="counts", mode=mode)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("lens", [[128, 256], [300, 77], [2048, 1111]])
def test_plain_attention_and_lse(lens, mode):
    _run(lens, H=2, dtype=torch.bfloat16, bias_kind=None, return_lse=True, mode=mode)
    _run(lens, H=2, dtype=torch.bfloat16, bias_kind="counts", return_lse=True, mode=mode)


@pytest.mark.parametrize("mode", MODES)
def test_sixteen_heads_long_segments_and_other_scale(mode):
    _run([3000, 1500], H=16, dtype=torch.bfloat16, bias_kind="counts", mode=mode)
    _run([500, 260], H=3, dtype=torch.bfloat16, scale=0.2, mode=mode)           # scale that is not a power of two


def test_scale_mode_is_validated_and_auto_follows_the_bound_on_the_tensor():
    """"auto" folds the scale only for a tensor that carries a small enough ``come_qk_bound`` (set by
    ``prepare_packed_self_attention_qkv``); results are bit-identical to the explicitly named mode."""
    lens, H = [700, 333], 4
    P = sum(lens)
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(P, 3, H, 64, generator=g).bfloat16().to(DEV)
    bias = torch.where(torch.rand(P, generator=g) < 0.3, math.log(9.0), 0.0).bfloat16().to(DEV)
    cu = _cu(lens).to(DEV)
    run = lambda t, **kw: flash_attn_varlen_qkvpacked_func_w_perkey_bias(t, cu, max(lens), perkey_bias=bias, **kw)
    exact, folded = run(qkv, scale_mode="exact"), run(qkv, scale_mode="folded")
    assert not torch.equal(exact, folded)
    assert torch.equal(run(qkv), exact)                         # no bound known: the reference's arithmetic
    tagged = qkv.clone()
    tagged.come_qk_bound = 64.0                                 # 64 * 0.125 = 8 nats
    assert torch.equal(run(tagged), folded)
    tagged.come_qk_bound = 256.0                                # 32 nats
    assert torch.equal(run(tagged), exact)
    assert torch.equal(run(tagged, scale_mode="folded"), folded)
    with pytest.raises(ValueError, match="scale_mode"):
        run(qkv, scale_mode="fast")


def test_zero_bias_equals_plain_operator():
    lens, H = [64, 64], 4
    P = sum(lens)
    qkv = torch.randn(P, 3, H, 64, device=DEV).half()
    cu = _cu(lens).to(DEV)
    plain = flash_attn_varlen_qkvpacked_func(qkv, cu, 64, softmax_scale=0.125)
    biased = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 64, perkey_bias=torch.zeros(P, device=DEV).half(),
                                                            softmax_scale=0.125)
    torch.testing.assert_close(plain, biased, atol=1e-4, rtol=1e-4)     # test_flex_attention_bias.py:279-300


def test_bias_has_effect():
    P, H = 128, 2
    qkv = torch.randn(P, 3, H, 64, device=DEV).half()
    cu = torch.tensor([0, 128], device=DEV, dtype=torch.int32)
    zero = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 128, perkey_bias=torch.zeros(P, device=DEV).half())
    some = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 128, perkey_bias=torch.randn(P, device=DEV).half())
    assert not torch.allclose(zero, some, atol=1e-4)


def test_count_bias_equals_key_duplication():
    L, H, c = 200, 2, 9
    qkv = torch.randn(L, 3, H, 64).bfloat16()
    count = torch.ones(L)
    count[17], count[150] = c, c
    a = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), _cu([L]).to(DEV), L,
                                                       perkey_bias=count.log().bfloat16().to(DEV))
    dup = torch.cat([qkv, qkv[17:18].repeat(c - 1, 1, 1, 1), qkv[150:151].repeat(c - 1, 1, 1, 1)])
    b = flash_attn_varlen_qkvpacked_func(dup.to(DEV), _cu([dup.shape[0]]).to(DEV), dup.shape[0])
    # log(9) rounded to bf16 is 2.203125 (exp -> 9.054): the identity holds to that rounding
    diff = (a.float() - b[:L].float()).abs()
    assert float(diff.max()) <= 2e-2 and float(diff.mean()) <= 2e-3


def test_sharp_logits_in_the_default_mode():
    """Logits of up to +-35 nats with near-ties between the leading keys (late_rows below) meet the ordinary tolerance
    in the default mode, where the scale is applied in fp32; folded into a 16-bit q the case needs 8e-2."""
    L, H = 1500, 2
    qkv = torch.randn(L, 3, H, 64).bfloat16()
    qkv[:, 1, :, :] *= torch.linspace(0.2, 6.0, L)[:, None, None].bfloat16()
    bias = torch.zeros(L).bfloat16()
    cu = _cu([L])
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L, perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True)
    diff = (out.float().cpu() - ref).abs()
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    assert float(diff.mean()) <= MEAN_ABS
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("gain", [1, 2, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_layernormed_qk_with_gains(gain, dtype):
    """What the real caller feeds the operator (reference vggt/module/bias_attention.py:100-137: q and k are
    LayerNorm'd per head, so |q| = |k| = 8 * gain and logits reach 8 * gain^2 nats), at the ordinary tolerance, through
    the default call."""
    _check_layernormed(gain, dtype)


def test_layernormed_qk_unit_gain_folded_mode():
    """With unit gains (logits within +-8 nats) folding the scale into a 16-bit q is inside the tolerance as well;
    from a gain of 2 on it is not (measured max-abs 2.3e-2 at gain 2, 1.2e-1 at gain 4 in bf16), which is why only
    tensors with a known small bound get it."""
    _check_layernormed(1, torch.bfloat16, mode="folded")
    _check_layernormed(1, torch.float16, mode="folded")


def _check_layernormed(gain, dtype, mode="auto"):
    lens, H = [700, 333, 64], 4
    P = sum(lens)
    g = torch.Generator().manual_seed(gain)
    x = torch.randn(P, 3, H, 64, generator=g)
    q = torch.nn.functional.layer_norm(x[:, 0], (64,)) * gain
    k = torch.nn.functional.layer_norm(x[:, 1], (64,)) * gain
    qkv = torch.stack((q, k, x[:, 2]), dim=1).to(dtype)
    bias = torch.where(torch.rand(P, generator=g) < 0.3, math.log(9.0), 0.0).to(dtype)
    cu = _cu(lens)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens),
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True,
                                                                 scale_mode=mode)
    diff = (out.float().cpu() - ref).abs()
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    assert float(diff.mean()) <= MEAN_ABS
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype,jump", [(torch.bfloat16, 100.0), (torch.bfloat16, 300.0), (torch.float16, 12.0),
                                        (torch.float16, 30.0)], ids=["bf16+100", "bf16+300", "f16+12", "f16+30"])
def test_late_key_beyond_the_range_of_the_stored_probabilities(dtype, jump, mode):
    """A late key whose logit exceeds everything before it by `jump` nats: relative to the lazily moved reference
    point its probability does not fit the 16-bit type (bf16: exp2 overflows from 88 nats on; fp16: the stored
    value saturates from about 11 nats on).  The workgroup notices and computes its block again with a running
    maximum, so the result meets the ordinary tolerance.  Several such keys, in the first tile, at tile borders and
    in a second, short segment (tail block)."""
    lens, H = [1500, 90], 2
    P = sum(lens)
    g = torch.Generator().manual_seed(int(jump))
    qkv = torch.randn(P, 3, H, 64, generator=g).to(dtype)
    bias = torch.zeros(P)
    bias[700] = jump                       # one step
    bias[1023] = 2 * jump                  # a second one on top, last key of a tile
    bias[1024] = 2 * jump - 1.0            # and a near-tie right behind it, first key of the next tile
    bias[1500 + 40] = jump                 # second segment: inside its only query block
    bias = bias.to(dtype)
    assert bool(torch.isfinite(bias.float()).all())
    cu = _cu(lens)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens),
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True,
                                                                 scale_mode=mode)
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    # two near-tied keys carry every row: the result is a 0.73 / 0.27 mix of two value rows, and rounding those
    # two probabilities and the result to 16 bits alone costs about 2^-9 of the value (as in the reference's kernel)
    diff = (out.float().cpu() - ref).abs()
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)     # the reference's own criterion
    assert float(diff.mean()) <= MEAN_ABS + 2.0 ** -9 * float(ref.abs().mean()), f"mean-abs {float(diff.mean())}"
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-2 if mode == "folded" else 5e-3, rtol=1e-3)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("jump", [80.0, 84.0, 87.0, 88.0])
def test_late_key_just_inside_the_float_range_with_large_values(jump, mode):
    """A late key that beats its row by 80 - 88 nats leaves a probability of 2^115 - 2^127 relative to the old reference
    point: still finite, so the row sum alone would not give it away, but multiplied by values of size 8 and added up
    over the keys of a step the fp32 outputs would overflow.  The redo threshold leaves that headroom."""
    L, H = 900, 2
    g = torch.Generator().manual_seed(int(jump))
    qkv = torch.randn(L, 3, H, 64, generator=g)
    qkv[:, 2] *= 8.0
    qkv = qkv.bfloat16()
    bias = torch.zeros(L)
    bias[500] = jump
    bias[501:520] = jump - 0.5             # a cluster right behind it: their products with v add up
    bias = bias.bfloat16()
    cu = _cu([L])
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L, perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True, scale_mode=mode)
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    # outputs are 8 times the usual size and their rounding errors with them: the usual bounds on out / 8
    torch.testing.assert_close(out.float().cpu() / 8, ref / 8, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-2 if mode == "folded" else 5e-3, rtol=1e-3)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("where", [1, 2, 31, 33, 40, 64, 65], ids=lambda w: f"last-{w}")
def test_key_beyond_the_range_in_the_last_tile_of_a_segment(where, mode):
    """The key that leaves the range of the stored probabilities is one of the last 65 keys of its segment (last
    key, last half-tile, the half-tile before it, the tile before), in a segment that ends on a tile border, one that
    ends one key behind it and a short second one: the sums of the last slots are looked at behind the loop."""
    lens, H = [1536, 1473, 100], 2
    P = sum(lens)
    g = torch.Generator().manual_seed(where)
    qkv = torch.randn(P, 3, H, 64, generator=g).bfloat16()
    bias = torch.zeros(P)
    end = 0
    for L in lens:
        end += L
        bias[end - where] = 150.0
    bias = bias.bfloat16()
    cu = _cu(lens)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens),
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True,
                                                                 scale_mode=mode)
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-2 if mode == "folded" else 5e-3, rtol=1e-3)


def test_key_beyond_the_range_inside_a_key_split_piece():
    """The same situation in a launch whose last query blocks are cut along the keys (long single segment with a work
    buffer): the piece that meets the key computes its share again; pieces are combined as usual."""
    L, H = 12288, 16
    g = torch.Generator().manual_seed(9)
    qkv = torch.randn(L, 3, H, 64, generator=g).bfloat16()
    bias = torch.zeros(L)
    bias[9000], bias[11500] = 120.0, 250.0
    bias = bias.bfloat16()
    from come_amd import _lib
    assert _lib.load().come_attn_work_bytes(1, L, H, L) > 0
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), _cu([L]).to(DEV), L,
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True)
    out, lse = out.float().cpu(), lse.cpu()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    q, k, v = qkv.float().unbind(1)
    for row in [0, 255, 5000, 8999, 9000, 11776, 12000, 12287]:          # the last blocks are the split ones
        scores = torch.einsum("hd,khd->hk", q[row], k) * 0.125 + bias.float()[None]
        ref = torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v)
        diff = (out[row] - ref).abs()
        assert float(diff.max()) <= MAX_ABS and float(diff.mean()) <= MEAN_ABS
        torch.testing.assert_close(lse[:, row], torch.logsumexp(scores, -1), atol=2e-2, rtol=1e-3)


@pytest.mark.parametrize("kind", ["ramp", "jump", "late_rows", "descending", "plateau"])
def test_reference_point_moves(kind):
    """Scores that grow by many orders of magnitude along the keys: the kernel keeps probabilities relative
    to a per-row reference point taken from the first keys and has to move it (rare path) without losing
    accuracy.  Checked against the closed form like every other case."""
    L, H = 1500, 2
    qkv = torch.randn(L, 3, H, 64).bfloat16()
    if kind == "ramp":
        bias = torch.linspace(-30.0, 30.0, L)
    elif kind == "jump":
        bias = torch.zeros(L)
        bias[700], bias[701], bias[1333] = 40.0, 25.0, 55.0
    elif kind == "late_rows":
        bias = torch.zeros(L)
        qkv[:, 1, :, :] *= torch.linspace(0.2, 6.0, L)[:, None, None].bfloat16()     # later keys score far higher
    elif kind == "plateau":
        # 22 nats up from key 200 on and staying there: no 32 keys add up to 2^40 times the first keys' sum, but the
        # running row sum passes it some 300 keys later, and again never after the reference point has moved
        bias = torch.zeros(L)
        bias[200:] = 22.0
    else:
        bias = torch.linspace(40.0, -40.0, L)
    bias = bias.bfloat16()
    cu = _cu([L])
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L, perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True)
    assert bool(torch.isfinite(out).all())
    if kind != "late_rows":
        _compare(out, ref)
    else:
        # sharp rows whose outputs reach 4: a bf16 output in [2, 4) is only known to 2^-7 = 7.8e-3, and two leading
        # probabilities rounded to bf16 (as in the reference's kernel) add as much, so the absolute bound cannot hold
        # there; the reference's own criterion (atol = rtol = 1e-2 per element) and the mean bound do
        torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)
        assert float((out.float().cpu() - ref).abs().mean()) <= MEAN_ABS
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=5e-3, rtol=1e-3)
    if kind == "late_rows":
        # logits of up to +-35 nats with near-ties between the leading keys: with softmax_scale * log2(e) folded into
        # a 16-bit q the error in a logit grows with its magnitude (about 1e-3 * |logit| / sqrt(head_dim) bits) and
        # shows as a few 1e-2 at this extreme - the case the default mode exists for
        out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L,
                                                                     perkey_bias=bias.to(DEV), return_attn_probs=True,
                                                                     scale_mode="folded")
        diff = (out.float().cpu() - ref).abs()
        assert float(diff.max()) <= 8e-2 and float(diff.mean()) <= 5e-3, (float(diff.max()), float(diff.mean()))
        torch.testing.assert_close(lse.cpu(), ref_lse, atol=5e-2, rtol=2e-3)


def test_fp16_reference_point_moves_within_its_narrow_range():
    """fp16 stores the probabilities in fp16, so its reference points move much earlier (row sums above 2^5, rows
    more than 2^4 below the workgroup's reference keep their own offset).  A slowly rising bias (20 nats over the
    segment) and rows of different scale exercise both paths inside the range fp16 can hold."""
    L, H = 1500, 2
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(L, 3, H, 64, generator=g).half()
    qkv[::3, 0] = (qkv[::3, 0].float() * 2).half()
    bias = torch.linspace(-10.0, 10.0, L).half()
    cu = _cu([L])
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L, perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True)
    assert bool(torch.isfinite(out).all())
    _compare(out, ref)
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=5e-3, rtol=1e-3)


def test_rows_of_very_different_magnitude_in_one_workgroup():
    """Every 7th query carries a large component along a direction in which all keys are equal, which lifts all
    of its logits by 80 nats (115 in log2 units) without widening them: row maxima inside one workgroup then
    differ by far more than 2^64, and the rows far below the workgroup's shared reference point keep their own
    offset (the per-row correction path).  Same tolerance as everywhere else."""
    L, H = 1100, 2
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn(L, 3, H, 64, generator=g).bfloat16()
    big = torch.zeros(L, dtype=torch.bool)
    big[::7] = True
    qkv[:, 1, :, 0] = 4.0
    qkv[big, 0, :, 0] = 160.0
    bias = torch.rand(L, generator=g).log().clamp(min=-5).bfloat16()
    cu = _cu([L])
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L, perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True)
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    _compare(out, ref)
    torch.testing.assert_close(lse.cpu()[:, ~big], ref_lse[:, ~big], atol=5e-3, rtol=1e-3)
    torch.testing.assert_close(lse.cpu()[:, big], ref_lse[:, big], atol=2e-2, rtol=1e-3)  # 80 nats


def test_strided_views_and_separate_tensors():
    lens, H = [90, 41], 4
    P = sum(lens)
    qkv = torch.randn(P, 3, H, 64).bfloat16()
    bias = torch.randn(P).bfloat16()
    cu = _cu(lens)
    ref, _ = oracle.biased_varlen_attention(qkv, cu, bias)
    q, k, v = (qkv[:, i].contiguous().to(DEV) for i in range(3))      # contiguous [P, H, D] tensors
    out = flash_attn_fwd_cuda.varlen_fwd_w_perkey_bias(q, k, v, None, cu.to(DEV), cu.to(DEV), None, None, None, None,
                                                       bias.to(DEV), 90, 90, 0.0, 0.125, False, False, -1, -1, 0.0,
                                                       False, None)
    assert len(out) == 4 and out[1].shape == (H, P) and out[1].dtype == torch.float32
    _compare(out[0], ref)
    big = torch.zeros(P, 5, H, 72).bfloat16()                          # odd strides: row 5*H*72, head 72
    big[:, 1:4, :, :64] = qkv
    out2 = flash_attn_varlen_qkvpacked_func_w_perkey_bias(big.to(DEV)[:, 1:4, :, :64], cu.to(DEV), 90,
                                                          perkey_bias=bias.to(DEV))
    _compare(out2, ref)


@pytest.mark.parametrize("pad,offset", [(4, 0), (8, 4), (12, 0)], ids=["stride68", "stride72+4", "stride76"])
def test_output_views_that_do_not_allow_16_byte_stores(pad, offset):
    """``out_`` may be a view whose head stride or start is only a multiple of 8 bytes: the kernel then writes its
    rows in 8-byte pieces.  Same bits as into a contiguous output; the padding of the view stays untouched."""
    lens, H = [300, 77, 513], 3
    P = sum(lens)
    g = torch.Generator().manual_seed(pad)
    qkv = torch.randn(P, 3, H, 64, generator=g).bfloat16().to(DEV)
    bias = torch.where(torch.rand(P, generator=g) < 0.3, math.log(9.0), 0.0).bfloat16().to(DEV)
    cu = _cu(lens).to(DEV)
    q, k, v = qkv.unbind(1)
    call = lambda out_: flash_attn_fwd_cuda.varlen_fwd_w_perkey_bias(
        q, k, v, out_, cu, cu, None, None, None, None, bias, max(lens), max(lens), 0.0, 0.125, False, False, -1, -1,
        0.0, False, None)[0]
    want = call(None)
    wide = torch.full((P, H, 64 + pad), 7.0, dtype=torch.bfloat16, device=DEV)
    view = wide[:, :, offset:offset + 64]
    assert view.stride(1) % 8 != 0 or view.data_ptr() % 16 != 0
    got = call(view)
    assert got.data_ptr() == view.data_ptr()
    assert torch.equal(got, want)
    untouched = torch.ones(64 + pad, dtype=torch.bool)
    untouched[offset:offset + 64] = False
    assert bool((wide[:, :, untouched.to(DEV)] == 7.0).all())


def test_max_seqlen_helper_and_empty_segment():
    lens = [40, 0, 90]
    cu = _cu(lens).to(DEV)
    assert infer_flash_attn_varlen_max_seqlen(cu) == 90
    P = sum(lens)
    qkv = torch.randn(P, 3, 2, 64).bfloat16()
    bias = torch.randn(P).bfloat16()
    ref, _ = oracle.biased_varlen_attention(qkv, _cu(lens), bias)
    out = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu, 90, perkey_bias=bias.to(DEV))
    _compare(out, ref)


def test_unsupported_arguments_raise():
    P = 64
    cu = torch.tensor([0, 64], device=DEV, dtype=torch.int32)
    qkv = torch.randn(P, 3, 2, 64, device=DEV).bfloat16()
    bias = torch.zeros(P, device=DEV).bfloat16()
    with pytest.raises(RuntimeError, match="causal"):
        flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 64, perkey_bias=bias, causal=True)
    with pytest.raises(RuntimeError, match="dropout"):
        flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 64, perkey_bias=bias, dropout_p=0.1)
    with pytest.raises(RuntimeError, match="head_dim"):
        flash_attn_varlen_qkvpacked_func(torch.randn(P, 3, 2, 136, device=DEV).half(), cu, 64)
    with pytest.raises(RuntimeError, match="dtype"):
        flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 64, perkey_bias=bias.half())
    with pytest.raises(RuntimeError, match="shape"):
        flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 64, perkey_bias=bias[:10])
    with pytest.raises(RuntimeError, match="fp16 and bf16"):
        flash_attn_varlen_qkvpacked_func(qkv.float(), cu, 64)
    q = qkv.clone().requires_grad_(True)
    out = flash_attn_varlen_qkvpacked_func_w_perkey_bias(q, cu, 64, perkey_bias=bias)
    with pytest.raises(RuntimeError, match="backward is not supported"):
        out.sum().backward()


def test_full_size_c3_rows_against_oracle_rows():
    """Benchmark attention configuration: 16 heads x 64, two packed sequences of 25 536 and 21 848 tokens,
    bias = log(count), count in {1, 9}.  The full fp32 oracle is too slow on a CPU at this size, so a
    sample of query rows is checked against the closed form, plus the logsumexp identity."""
    H, D = 16, 64
    lens = [25536, 21848]
    P = sum(lens)
    g = torch.Generator().manual_seed(0)
    qkv = torch.randn(P, 3, H, D, generator=g).bfloat16()
    count = torch.ones(P)
    count[torch.randperm(lens[0], generator=g)[:2304]] = 9.0
    count[lens[0] + torch.randperm(lens[1], generator=g)[:2765]] = 9.0
    bias = count.log().bfloat16()
    cu = _cu(lens)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens),
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True)
    out, lse = out.float().cpu(), lse.cpu()
    assert bool(torch.isfinite(out).all())
    rows = [0, 1, 31, 32, 255, 256, 12345, 25535, 25536, 25537, 30000, P - 1]
    q, k, v = qkv.float().unbind(1)
    for row in rows:
        s, e = (0, lens[0]) if row < lens[0] else (lens[0], P)
        scores = torch.einsum("hd,khd->hk", q[row], k[s:e]) * 0.125 + bias.float()[None, s:e]
        ref = torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v[s:e])
        diff = (out[row] - ref).abs()
        assert float(diff.max()) <= MAX_ABS and float(diff.mean()) <= MEAN_ABS
        torch.testing.assert_close(lse[:, row], torch.logsumexp(scores, -1), atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("L", [8192, 8129, 8127, 8064, 7999], ids=lambda L: f"L{L}")
def test_long_segment_launch_with_every_remainder_of_its_four_tile_loop(L, mode):
    """One segment that fills a round of 512-query workgroups (16 heads x 16 blocks = 256): the instantiation whose
    key loop takes four 64-key tiles per turn.  128, 128 (one key into the last tile), 127, 126 and 125 tiles leave
    0, 0, 3, 2 and 1 tiles behind the last full turn; rows sampled over the segment against the closed form."""
    H = 16
    g = torch.Generator().manual_seed(L)
    qkv = torch.randn(L, 3, H, 64, generator=g).bfloat16()
    bias = torch.where(torch.rand(L, generator=g) < 0.3, 2.197, 0.0).bfloat16()
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), _cu([L]).to(DEV), L, perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True, scale_mode=mode)
    out, lse = out.float().cpu(), lse.cpu()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    q, k, v = qkv.float().unbind(1)
    for row in [0, 33, 511, 512, 4000, L - 513, L - 65, L - 64, L - 1]:
        scores = torch.einsum("hd,khd->hk", q[row], k) * 0.125 + bias.float()[None]
        ref = torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v)
        diff = (out[row] - ref).abs()
        assert float(diff.max()) <= MAX_ABS and float(diff.mean()) <= MEAN_ABS, (row, float(diff.max()))
        torch.testing.assert_close(lse[:, row], torch.logsumexp(scores, -1), atol=4e-3, rtol=1e-3)


BORDER_LENGTHS = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 512, 513, 767, 769, 1023, 1025]


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_with_lengths_at_tile_borders(seed):
    """Seeded sweep: segment lengths drawn from the borders of the 32 / 64-key tiles and the 256 / 512-query blocks,
    1 to 6 segments (some empty), several head counts, both dtypes, bias kinds and scales; q, k, v either views
    of one packed tensor or separate tensors with strides of their own; ``out_`` either fresh or supplied."""
    g = torch.Generator().manual_seed(1000 + seed)
    pick = lambda seq: seq[int(torch.randint(len(seq), (1,), generator=g))]
    n_seq = pick([1, 2, 3, 4, 6])
    lens = [pick(BORDER_LENGTHS + [0]) for _ in range(n_seq)]
    if sum(lens) == 0:
        lens[0] = 65
    H = pick([1, 2, 3, 5, 16])
    dtype = pick([torch.bfloat16, torch.bfloat16, torch.float16])
    scale = pick([0.125, 0.1, 0.2])
    P = sum(lens)
    qkv = torch.randn(P, 3, H, 64, generator=g).to(dtype)
    kind = pick(["counts", "weights", None])
    if kind == "counts":
        bias = torch.where(torch.rand(P, generator=g) < 0.3, math.log(9.0), 0.0).to(dtype)
    elif kind == "weights":
        bias = torch.rand(P, generator=g).clamp(min=1e-3).log().to(dtype)
    else:
        bias = None
    cu = _cu(lens)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias, softmax_scale=scale)
    max_len = max(lens)
    if pick([True, False]):
        q, k, v = qkv.to(DEV).unbind(1)                                            # views into the packed tensor
    else:
        pad = [torch.zeros(P, H, 64 + 8 * (i + 1), dtype=dtype, device=DEV) for i in range(3)]
        for i in range(3):
            pad[i][..., :64] = qkv[:, i].to(DEV)
        q, k, v = (t[..., :64] for t in pad)                                         # three row / head strides
    out_ = torch.full((P, H, 64), float("nan"), dtype=dtype, device=DEV) if pick([True, False]) else None
    fold = seed % 2 == 1                   # alternate between the two ways of applying the scale
    out, lse, _, _ = flash_attn_fwd_cuda.varlen_fwd_w_perkey_bias(
        q, k, v, out_, cu.to(DEV), cu.to(DEV), None, None, None, None, None if bias is None else bias.to(DEV),
        max_len, max_len, 0.0, scale, False, False, -1, -1, 0.0, False, None, fold_scale=fold)
    if out_ is not None:
        assert out.data_ptr() == out_.data_ptr()
    assert bool(torch.isfinite(out).all())
    # short segments and sharp softmaxes (scale 0.2) give outputs of size 1 to 4, where rounding the result to 16
    # bits alone costs up to 2^-9 of the value (2^-10 on average): the bounds are the reference's own
    # (test_flex_attention_bias.py:20-21, atol = rtol = 1e-2) and the mean bound with that allowance
    diff = (out.float().cpu() - ref).abs()
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    assert float(diff.mean()) <= MEAN_ABS + 2.0 ** -9 * float(ref.abs().mean()), f"mean-abs {float(diff.mean())}"
    # the row sum is taken from the probabilities as rounded to 16 bits (so that numerator and denominator of the
    # output agree): for rows of one or two keys that is up to 2^-9 of the sum, 2e-3 in lse, on top of the rest
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=1e-2 if fold else 4e-3, rtol=1e-3)


def test_bias_of_minus_infinity_masks_keys():
    """A caller may mask keys with a bias of -inf (the Co-Me path never does: log(count) >= 0).  Masked keys get
    probability exactly 0, also when every one of the first keys of a segment - from which the kernel takes its
    reference points - is masked."""
    lens, H = [700, 90], 3
    P = sum(lens)
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(P, 3, H, 64, generator=g).bfloat16()
    bias = torch.where(torch.rand(P, generator=g) < 0.3, -math.inf, 0.0)
    bias[:40] = -math.inf                                              # the whole first 32-key step of segment 0
    bias[40] = 0.0
    bias[700:730] = -math.inf                                          # most of the first step of segment 1
    bias = bias.bfloat16()
    cu = _cu(lens)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    assert bool(torch.isfinite(ref).all())
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), 700, perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True)
    assert bool(torch.isfinite(out).all())
    _compare(out, ref)
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=1e-2, rtol=1e-3)
    # a masked key cannot reach the output: changing its value row changes nothing, bit for bit
    qkv2 = qkv.clone()
    qkv2[:40, 2] = 1000.0
    out2 = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv2.to(DEV), cu.to(DEV), 700, perkey_bias=bias.to(DEV))
    assert torch.equal(out2, out)


@pytest.mark.parametrize("lens", [[32, 48, 24, 24], [56, 49, 23], [128], [60, 40]], ids=str)
def test_reference_test_shapes_with_narrow_heads(lens):
    """The reference's own CUDA tests use heads of 32 (test_flex_attention_bias.py:247-262: H=2, D=32)."""
    P, H, D = sum(lens), 2, 32
    g = torch.Generator().manual_seed(P)
    qkv = torch.randn(P, 3, H, D, generator=g).bfloat16()
    bias = torch.rand(P, generator=g).clamp(min=1e-3).log().bfloat16()
    cu = _cu(lens)
    scale = D ** -0.5
    out = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens), perkey_bias=bias.to(DEV))
    assert out.shape == (P, H, D) and out.is_contiguous()
    q, k, v = qkv.float().unbind(1)
    start = 0
    for L in lens:
        sl = slice(start, start + L)
        scores = torch.einsum("qhd,khd->hqk", q[sl], k[sl]) * scale + bias.float()[None, None, sl]
        ref = torch.einsum("hqk,khd->qhd", torch.softmax(scores, -1), v[sl])
        torch.testing.assert_close(out[sl].float().cpu(), ref, atol=1e-2, rtol=1e-2)
        start += L
    with pytest.raises(RuntimeError, match="head_dim 256"):
        flash_attn_varlen_qkvpacked_func(torch.zeros(8, 3, 2, 256, device=DEV).bfloat16(), _cu([8]).to(DEV), 8)
