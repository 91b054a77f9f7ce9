"""The q half of the attention prologue applied inside the attention kernel (``come_attn_varlen_fwd_qp``).

The reference normalises and rotates q and k in a step of the caller (``src/accelerate/common/qkv.py:31-39``) right in
front of the operator (``src/accelerate/vggt/module/bias_attention.py:100-137``).  With ``defer_q=True`` only k goes
through that step and the kernel treats its query fragments as it loads them.  The bar is the strictest there is: the
same bits as the two-step path (whose own parity against the oracle is tested elsewhere), on outputs and
log-sum-exps, because the kernel runs the same arithmetic in the same summation order; one case also goes against
the oracle directly.
"""

import copy
import ctypes

import pytest
import torch

import oracle
from come_amd import _lib
from come_amd.common import RotaryPositionEmbedding2D, prepare_packed_self_attention_qkv
from come_amd.cuda_extension import (flash_attn_varlen_qkvpacked_func,
                                     flash_attn_varlen_qkvpacked_func_w_perkey_bias)

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _cu(lens):
    return torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)


def _inputs(lens, H, dtype, seed, affine=True):
    P = sum(lens)
    g = torch.Generator().manual_seed(seed)
    qkv = (torch.randn(P, 3, H, 64, generator=g) * 1.5 + 0.3).to(dtype)
    norms = []
    for _ in range(2):
        n = torch.nn.LayerNorm(64, eps=1e-5)
        if affine:
            with torch.no_grad():
                n.weight.copy_(torch.rand(64, generator=g) + 0.5)
                n.bias.copy_(torch.randn(64, generator=g) * 0.2)
        norms.append(n.to(dtype))
    pos = torch.randint(0, 38, (P, 2), generator=g)
    counts = torch.where(torch.rand(P, generator=g) < 0.3, 9.0, 1.0)
    return qkv, norms, pos, counts.log().to(dtype)


def _both_ways(qkv, q_norm, k_norm, rope, pos, bias, lens, dtype, **kw):
    """(out, lse) of prologue-then-attention and of the deferred q prologue, on copies of the same raw tensor."""
    cu = _cu(lens).to(DEV)
    results = []
    for defer in (False, True):
        t = qkv.clone().to(DEV)
        with torch.no_grad():
            t = prepare_packed_self_attention_qkv(t, q_norm, k_norm, rope, None if pos is None else pos.to(DEV), dtype,
                                                  max_position=40, defer_q=defer)
        if defer:
            assert torch.equal(t[:, 0].cpu(), qkv[:, 0]), "q must stay the raw projection"
            assert hasattr(t, "come_q_prologue")
        else:
            assert not hasattr(t, "come_q_prologue")
        if bias is None:
            out, lse, _ = flash_attn_varlen_qkvpacked_func(t, cu, max(lens), return_attn_probs=True, **kw)
        else:
            out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(t, cu, max(lens), perkey_bias=bias.to(DEV),
                                                                         return_attn_probs=True, **kw)
        results.append((out, lse, t))
    return results


@pytest.mark.parametrize("mode", ["exact", "folded"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("lens,H", [([300, 77], 3), ([2048, 1111, 1], 4), ([686, 862, 700, 768, 769], 16), ([5000], 2)],
                         ids=["two_short", "ragged", "frames", "long"])
def test_same_bits_as_the_two_step_path(lens, H, dtype, mode):
    qkv, (qn, kn), pos, bias = _inputs(lens, H, dtype, seed=len(lens) + H)
    qn, kn = copy.deepcopy(qn).cuda(), copy.deepcopy(kn).cuda()
    (out_a, lse_a, t_a), (out_b, lse_b, t_b) = _both_ways(qkv, qn, kn, RotaryPositionEmbedding2D(100.0), pos, bias, lens,
                                                         dtype, scale_mode=mode)
    assert torch.equal(t_a[:, 1], t_b[:, 1]) and torch.equal(t_a[:, 2], t_b[:, 2])      # k, v: the same either way
    assert torch.equal(out_a, out_b)
    assert torch.equal(lse_a, lse_b)


def test_norm_only_rope_only_plain_affine_free_and_auto_mode():
    dtype = torch.bfloat16
    lens, H = [513, 300], 4
    qkv, (qn, kn), pos, bias = _inputs(lens, H, dtype, seed=21)
    qn, kn = qn.cuda(), kn.cuda()
    ident = torch.nn.Identity()
    rope = RotaryPositionEmbedding2D(100.0)
    plain = [torch.nn.LayerNorm(64, eps=1e-6, elementwise_affine=False).to(dtype).cuda() for _ in range(2)]
    for q_norm, k_norm, r, p, b in [(qn, kn, None, None, bias), (ident, ident, rope, pos, bias), (qn, kn, rope, pos, None),
                                    (plain[0], plain[1], rope, pos, bias)]:
        (out_a, lse_a, _), (out_b, lse_b, _) = _both_ways(qkv, q_norm, k_norm, r, p, b, lens, dtype)
        assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    # neither norm nor rotation: nothing to defer, the tensor carries no prologue
    t = prepare_packed_self_attention_qkv(qkv.clone().to(DEV), ident, ident, None, None, dtype, defer_q=True)
    assert not hasattr(t, "come_q_prologue") and torch.equal(t.cpu(), qkv)
    # a second, non-deferred pass over a tensor that carried a prologue drops it
    t = prepare_packed_self_attention_qkv(qkv.clone().to(DEV), qn, kn, rope, pos.to(DEV), dtype, defer_q=True)
    assert hasattr(t, "come_q_prologue")
    t = prepare_packed_self_attention_qkv(t, ident, ident, None, None, dtype)
    assert not hasattr(t, "come_q_prologue")


def test_key_split_tail_of_a_long_launch():
    """A launch that finishes its last query blocks in key-split pieces (work buffer): every piece prepares the same
    query rows again."""
    dtype = torch.bfloat16
    lens, H = [12288], 16
    assert _lib.load().come_attn_work_bytes(1, lens[0], H, lens[0]) > 0
    qkv, (qn, kn), pos, bias = _inputs(lens, H, dtype, seed=5)
    (out_a, lse_a, _), (out_b, lse_b, _) = _both_ways(qkv, qn.cuda(), kn.cuda(), RotaryPositionEmbedding2D(100.0), pos, bias,
                                                     lens, dtype)
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)


def test_same_bits_at_the_size_of_the_benchmark_workload():
    """16 heads, two packed sequences of 25 536 and 21 848 rows (the 512-query workgroups with their four-tile loop,
    full rounds and a key-split tail)."""
    dtype = torch.bfloat16
    lens, H = [25536, 21848], 16
    qkv, (qn, kn), pos, bias = _inputs(lens, H, dtype, seed=1)
    (out_a, lse_a, t_a), (out_b, lse_b, t_b) = _both_ways(qkv, qn.cuda(), kn.cuda(), RotaryPositionEmbedding2D(100.0), pos, bias,
                                                         lens, dtype)
    assert torch.equal(t_a[:, 1], t_b[:, 1])
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    assert bool(torch.isfinite(out_b).all())


@torch.no_grad()
def test_against_the_oracle():
    """Prologue and attention of the oracle on the raw tensor against the deferred path, at the operator's tolerance.
    (Unit-size gains: the oracle's prologue and the kernel's differ by a unit in the last place of some q / k elements,
    which is part of the prologue's own tolerance; with large gains the softmax amplifies that beyond the operator's,
    whichever way q was prepared - what the bit-identity tests above pin is that the deferred path adds nothing.)"""
    dtype = torch.bfloat16
    lens, H = [700, 333], 4
    qkv, (qn, kn), pos, bias = _inputs(lens, H, dtype, seed=33)
    prepared = oracle.qk_norm_rope(qkv, qn.weight, qn.bias, kn.weight, kn.bias, 1e-5, pos, 100.0)
    ref, ref_lse = oracle.biased_varlen_attention(prepared, _cu(lens), bias)
    t = prepare_packed_self_attention_qkv(qkv.clone().to(DEV), qn.cuda(), kn.cuda(), RotaryPositionEmbedding2D(100.0),
                                          pos.to(DEV), dtype, defer_q=True)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(t, _cu(lens).to(DEV), max(lens), perkey_bias=bias.to(DEV),
                                                                 return_attn_probs=True)
    diff = (out.float().cpu() - ref).abs()
    assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3, (float(diff.max()), float(diff.mean()))
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-2, rtol=1e-3)


def test_what_the_deferred_prologue_refuses():
    dtype = torch.bfloat16
    lens, H = [300, 200], 2
    qkv, (qn, kn), pos, bias = _inputs(lens, H, dtype, seed=2)
    rope = RotaryPositionEmbedding2D(100.0)
    t = prepare_packed_self_attention_qkv(qkv.clone().to(DEV), qn.cuda(), kn.cuda(), rope, pos.to(DEV), dtype, defer_q=True)
    cu = _cu(lens).to(DEV)
    with pytest.raises(RuntimeError, match="COME_ATTN_WORK_QUEUE"):
        flash_attn_varlen_qkvpacked_func(t, cu, max(lens), work_queue=True)
    wide = torch.randn(64, 3, 2, 128).to(dtype).to(DEV)
    with pytest.raises(RuntimeError, match="head_dim"):
        prepare_packed_self_attention_qkv(wide, torch.nn.Identity(), torch.nn.Identity(), rope,
                                          torch.zeros(64, 2, dtype=torch.int64, device=DEV), dtype, defer_q=True)


def test_c_abi_null_prologue_equals_ws_and_bad_descriptors_are_refused():
    dtype = torch.bfloat16
    lens, H = [400, 90], 2
    P = sum(lens)
    qkv, _, pos, bias = _inputs(lens, H, dtype, seed=8)
    qkv, bias, cu = qkv.to(DEV), bias.to(DEV), _cu(lens).to(DEV)
    lib = _lib.load()
    q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]
    stream = _lib.current_stream(qkv.device)

    def run(fn, *extra):
        out = torch.empty(P, H, 64, dtype=dtype, device=DEV)
        lse = torch.empty(H, P, dtype=torch.float32, device=DEV)
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.COME_BF16, q.stride(0), q.stride(1), k.stride(0), k.stride(1),
                v.stride(0), v.stride(1), cu.data_ptr(), len(lens), P, H, 64, bias.data_ptr(), max(lens), 0.125,
                out.data_ptr(), out.stride(0), out.stride(1), lse.data_ptr(), None, 0, *extra, 0, stream)
        return rc, out, lse

    rc_a, out_a, lse_a = run(lib.come_attn_varlen_fwd_ws)
    rc_b, out_b, lse_b = run(lib.come_attn_varlen_fwd_qp, None)
    assert rc_a == 0 and rc_b == 0
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    # a descriptor that neither normalises nor rotates changes nothing either
    rc_c, out_c, _ = run(lib.come_attn_varlen_fwd_qp, ctypes.byref(_lib.QPrologue(0, 0.0, None, None, None, None, None, 0)))
    assert rc_c == 0 and torch.equal(out_a, out_c)
    # positions without tables, a negative eps, a misaligned gain
    positions = pos.to(DEV)
    rc, _, _ = run(lib.come_attn_varlen_fwd_qp, ctypes.byref(_lib.QPrologue(0, 0.0, None, None, positions.data_ptr(), None, None, 0)))
    assert rc != 0 and b"tables" in lib.come_last_error()
    rc, _, _ = run(lib.come_attn_varlen_fwd_qp, ctypes.byref(_lib.QPrologue(1, -1.0, None, None, None, None, None, 0)))
    assert rc != 0 and b"eps" in lib.come_last_error()
    gain = torch.ones(72, dtype=dtype, device=DEV)
    rc, _, _ = run(lib.come_attn_varlen_fwd_qp, ctypes.byref(_lib.QPrologue(1, 1e-5, gain.data_ptr() + 2, None, None, None, None, 0)))
    assert rc != 0 and b"aligned" in lib.come_last_error()
