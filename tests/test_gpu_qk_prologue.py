"""HIP q/k LayerNorm + 2-D RoPE prologue against the oracle, through the C ABI.

Tolerance: the kernel and the oracle round at the same points (after the normalisation, after each
product, after the sum), but their fp32 arithmetic differs in the last bit, which can move a result by
one unit in the last place of the storage dtype at a rounding step: rtol = 2^-6 (two bf16 ulps),
atol = 1e-2, and mean-abs <= 1e-3 over the tensor.
"""

import copy
import types

import pytest
import torch

import oracle
from come_amd.common import RotaryPositionEmbedding2D, prepare_packed_self_attention_qkv

pytestmark = pytest.mark.gpu


def make(P, H, dtype, seed, affine=True):
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
    return qkv, norms, pos


def gpu(module):
    return copy.deepcopy(module).cuda()


def check(got, want, dtype):
    got, want = got.float().cpu(), want.float()
    rtol = 2.0 ** -6 if dtype == torch.bfloat16 else 2.0 ** -9
    torch.testing.assert_close(got, want, rtol=rtol, atol=1e-2)
    assert (got - want).abs().mean() < 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("P,H", [(1, 1), (37, 3), (1000, 16), (4099, 16)])
def test_norm_and_rope(P, H, dtype):
    qkv, (qn, kn), pos = make(P, H, dtype, seed=P + H)
    want = oracle.qk_norm_rope(qkv, qn.weight, qn.bias, kn.weight, kn.bias, 1e-5, pos, 100.0)
    dev = qkv.cuda()
    with torch.no_grad():
        out = prepare_packed_self_attention_qkv(dev, gpu(qn), gpu(kn), RotaryPositionEmbedding2D(100.0), pos.cuda(), dtype)
    assert out.data_ptr() == dev.data_ptr()                       # in place
    assert torch.equal(out[:, 2].cpu(), qkv[:, 2])                # v untouched
    check(out[:, :2], want[:, :2], dtype)


def test_norm_only_rope_only_and_max_position():
    dtype = torch.bfloat16
    qkv, (qn, kn), pos = make(513, 4, dtype, seed=9)
    with torch.no_grad():
        a = prepare_packed_self_attention_qkv(qkv.cuda(), gpu(qn), gpu(kn), None, None, dtype)
        check(a[:, :2], oracle.qk_norm_rope(qkv, qn.weight, qn.bias, kn.weight, kn.bias, 1e-5, None)[:, :2], dtype)
        ident = torch.nn.Identity()
        rope = RotaryPositionEmbedding2D(100.0)
        b = prepare_packed_self_attention_qkv(qkv.cuda(), ident, ident, rope, pos.cuda(), dtype, max_position=40)
        want = oracle.qk_norm_rope(qkv, None, None, None, None, 0.0, pos, 100.0, apply_norm=False)
        check(b[:, :2], want[:, :2], dtype)
        # rotation with exact tables: position 0 leaves a row bit-identical
        zero = prepare_packed_self_attention_qkv(qkv.cuda(), ident, ident, rope, torch.zeros_like(pos).cuda(), dtype)
        assert torch.equal(zero.cpu(), qkv)
        # a [1, P, 2] position tensor (as the reference passes it) is accepted
        c = prepare_packed_self_attention_qkv(qkv.cuda(), ident, ident, rope, pos[None].cuda(), dtype)
        assert torch.equal(c, b)
        # rope modules of the reference are recognised by their attribute: VGGT / DA3 `base_frequency`, Pi3 `base`
        for foreign in (types.SimpleNamespace(base_frequency=100.0), types.SimpleNamespace(base=100.0, F0=1.0)):
            d = prepare_packed_self_attention_qkv(qkv.cuda(), ident, ident, foreign, pos.cuda(), dtype)
            assert torch.equal(d, b)
        with pytest.raises(RuntimeError, match="base frequency"):
            prepare_packed_self_attention_qkv(qkv.cuda(), ident, ident, object(), pos.cuda(), dtype)


def test_strided_views_of_a_wider_buffer():
    dtype = torch.bfloat16
    qkv, (qn, kn), pos = make(300, 2, dtype, seed=4)
    wide = torch.zeros(300, 3, 5, 64, dtype=dtype)                # heads 1..2 of a 5-head buffer
    wide[:, :, 1:3] = qkv
    dev = wide.cuda()
    view = dev[:, :, 1:3]
    with torch.no_grad():
        prepare_packed_self_attention_qkv(view, gpu(qn), gpu(kn), RotaryPositionEmbedding2D(100.0), pos.cuda(), dtype)
    want = oracle.qk_norm_rope(qkv, qn.weight, qn.bias, kn.weight, kn.bias, 1e-5, pos, 100.0)
    check(dev[:, :2, 1:3], want[:, :2], dtype)
    rest = dev.cpu().clone()
    rest[:, :, 1:3] = 0
    assert not rest.any()                                         # nothing outside the view was written


def test_rejects_what_it_does_not_implement():
    qkv = torch.randn(8, 3, 2, 32).bfloat16().cuda()
    ident = torch.nn.Identity()
    with torch.no_grad(), pytest.raises(RuntimeError, match="head_dim 64"):
        prepare_packed_self_attention_qkv(qkv, torch.nn.LayerNorm(32).cuda().bfloat16(),
                                          torch.nn.LayerNorm(32).cuda().bfloat16(), None, None, torch.bfloat16)
    with torch.no_grad(), pytest.raises(RuntimeError, match="same kind"):
        prepare_packed_self_attention_qkv(torch.randn(8, 3, 2, 64).bfloat16().cuda(),
                                          torch.nn.LayerNorm(64).cuda().bfloat16(), ident, None, None, torch.bfloat16)
    with pytest.raises(RuntimeError, match="bf16 / fp16"):
        prepare_packed_self_attention_qkv(torch.randn(8, 3, 2, 64).cuda(), ident, ident, None, None, torch.float32)
