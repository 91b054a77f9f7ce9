"""Drives the library through the kind of Python glue the reference wraps around its extension modules.

The reference does not call its pybind modules directly.  Its token-merger module builds two wrappers on the raw
operators and attaches them to the extension module with ``setattr`` (src/accelerate/token_merger/co_me.py:131-149,
225-238), and a dispatch decorator looks them up by name with ``getattr`` when the accelerated function is defined and
chooses between them and the torch fallback at call time (src/utility/feature.py:154-166).  Its attention module
prepares the packed qkv, derives ``cu_seqlens`` / ``max_seqlen`` / the per-key bias from the jagged tokens and calls the
biased operator (src/accelerate/vggt/module/bias_attention.py:100-137).  The same pattern is written out here from
scratch on ``come_amd.cuda_extension`` alone - attributes attached to this package's ``co_me_cuext`` module, name-based
dispatch, an attention module of that shape - and checked against the oracle.
"""

import math

import pytest
import torch

import oracle
from come_amd import cuda_extension
from come_amd.common import prepare_packed_self_attention_qkv
from come_amd.interface import JaggedTokens

pytestmark = pytest.mark.gpu
DEV = "cuda"


class Extension:
    """Name-based dispatch onto the extension module, with a switch back to the fallback."""

    force_disabled = False

    @classmethod
    def accelerate(cls, name):
        def decorator(fallback):
            fast = getattr(cuda_extension.co_me_cuext, name)          # resolved once, by name, when decorated

            def dispatch(*args, **kwargs):
                return fallback(*args, **kwargs) if cls.force_disabled else fast(*args, **kwargs)

            return dispatch

        return decorator


@pytest.fixture
def glue():
    """Attaches the two wrappers to the extension module and defines the two dispatched functions, as a caller's
    module would at import time; detaches them afterwards."""
    ext = cuda_extension.co_me_cuext

    def merge_entry(tokens, start_index, group_size, merge_mask):
        flat, offsets, rev_id, weight = ext.co_me_token_merge_cuda(tokens.contiguous(), start_index, group_size,
                                                                   merge_mask.contiguous())
        return JaggedTokens(tokens=flat.unsqueeze(0), weight=weight, offset=offsets.long()), rev_id

    def split_entry(tokens, rev_id, bsnc_shape):
        B, S, N, C = bsnc_shape
        return ext.co_me_token_split_cuda(tokens.tokens.squeeze(0).contiguous(), rev_id.contiguous(), C).reshape(B * S, N, C)

    setattr(ext, "merge_entry_of_the_caller", merge_entry)
    setattr(ext, "split_entry_of_the_caller", split_entry)

    @Extension.accelerate("merge_entry_of_the_caller")
    def token_merge(tokens, start_index, group_size, merge_mask):      # fallback: the oracle on the CPU
        jag, rev = oracle.token_merge_1d(tokens.cpu(), start_index, group_size, merge_mask.cpu())
        return JaggedTokens(tokens=jag.tokens, weight=jag.weight, offset=jag.offset), rev

    @Extension.accelerate("split_entry_of_the_caller")
    def token_split(tokens, rev_id, bsnc_shape):
        jag = oracle.JaggedTokens(tokens=tokens.tokens.cpu(), weight=tokens.weight.cpu(), offset=tokens.offset.cpu())
        return oracle.token_split(jag, rev_id.cpu(), bsnc_shape)

    yield token_merge, token_split
    delattr(ext, "merge_entry_of_the_caller")
    delattr(ext, "split_entry_of_the_caller")
    Extension.force_disabled = False


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_attached_wrappers_dispatch_by_name(glue, dtype):
    token_merge, token_split = glue
    B, S, M, G, S0, C = 1, 3, 40, 4, 2, 256
    N = S0 + M * G
    g = torch.Generator().manual_seed(0)
    tokens = torch.randn(B * S, N, C, generator=g).to(dtype).to(DEV)
    mask = (torch.rand(B * S, M, generator=g) < 0.5).to(DEV)

    fast, fast_rev = token_merge(tokens, S0, G, mask)
    assert fast.tokens.is_cuda and fast.offset.dtype == torch.int64 and fast_rev.dtype == torch.int64
    assert fast.weight.dtype == torch.float32 and fast.tokens.dim() == 3 and fast.tokens.shape[0] == 1
    Extension.force_disabled = True
    slow, slow_rev = token_merge(tokens, S0, G, mask)
    Extension.force_disabled = False
    assert not slow.tokens.is_cuda
    assert torch.equal(fast.offset.cpu(), slow.offset) and torch.equal(fast_rev.cpu(), slow_rev)
    assert torch.equal(fast.weight.cpu(), slow.weight)
    torch.testing.assert_close(fast.tokens.cpu().float(), slow.tokens.float(), atol=1e-2 if dtype != torch.float32 else 1e-5,
                               rtol=1e-2 if dtype != torch.float32 else 1e-5)

    restored = token_split(fast, fast_rev, (B, S, N, C))
    Extension.force_disabled = True
    want = token_split(fast, fast_rev, (B, S, N, C))
    Extension.force_disabled = False
    assert restored.shape == (B * S, N, C) and torch.equal(restored.cpu(), want)


class AttentionOfTheCaller(torch.nn.Module):
    """Attention module of the shape the reference wraps around the operator: qkv projection, q / k LayerNorm, packed
    preparation, offsets -> int32 cu_seqlens, max_seqlen read from them, bias = log(weight) in the run dtype."""

    def __init__(self, dim, heads, run_dtype):
        super().__init__()
        self.num_heads, self.head_dim, self.scale, self.run_dtype = heads, dim // heads, (dim // heads) ** -0.5, run_dtype
        self.qkv = torch.nn.Linear(dim, 3 * dim)
        self.q_norm, self.k_norm = torch.nn.LayerNorm(self.head_dim), torch.nn.LayerNorm(self.head_dim)
        self.proj = torch.nn.Linear(dim, dim)
        self.to(run_dtype)

    def forward(self, x: JaggedTokens, operator=None):
        tokens = x.tokens.squeeze(0)
        P, C = tokens.shape
        qkv = self.qkv(tokens).reshape(P, 3, self.num_heads, self.head_dim)
        qkv = prepare_packed_self_attention_qkv(qkv=qkv, q_norm=self.q_norm, k_norm=self.k_norm, rope=None, pos=None,
                                                run_dtype=self.run_dtype)
        cu_seqlens = x.offset.to(torch.int32)
        max_seqlen = cuda_extension.infer_flash_attn_varlen_max_seqlen(cu_seqlens)
        perkey_bias = x.weight.float().log().to(dtype=self.run_dtype)
        if operator is None:
            out = cuda_extension.flash_attn_varlen_qkvpacked_func_w_perkey_bias(
                qkv, cu_seqlens, max_seqlen, perkey_bias=perkey_bias, dropout_p=0.0, softmax_scale=self.scale)
        else:
            out = operator(qkv, cu_seqlens, perkey_bias, self.scale)
        out = self.proj(out.reshape(P, C))
        return JaggedTokens(tokens=out.unsqueeze(0), weight=x.weight, offset=x.offset)


@pytest.mark.parametrize("gain", [1.0, 3.0])
def test_attention_module_of_the_callers_shape(gain):
    """Unit gains: the prepared tensor carries a bound of about 8 nats and the operator folds the scale; gains of 3:
    72 nats, the scale is applied in fp32.  Either way the module matches the same module on the oracle operator."""
    dim, heads = 256, 4
    torch.manual_seed(1)
    module = AttentionOfTheCaller(dim, heads, torch.bfloat16).to(DEV).eval()
    with torch.no_grad():
        module.q_norm.weight.mul_(gain)
        module.k_norm.weight.mul_(gain)
    lens = [300, 77, 512]
    P = sum(lens)
    g = torch.Generator().manual_seed(2)
    x = JaggedTokens(tokens=torch.randn(1, P, dim, generator=g).bfloat16().to(DEV),
                     weight=torch.where(torch.rand(P, generator=g) < 0.3, 9.0, 1.0).to(DEV),
                     offset=torch.tensor([0, 300, 377, 889], device=DEV))

    def oracle_operator(qkv, cu, bias, scale):
        out, _ = oracle.biased_varlen_attention(qkv.cpu(), cu.cpu(), bias.cpu(), scale)
        return out.to(device=qkv.device, dtype=qkv.dtype)

    with torch.no_grad():
        got = module(x)
        want = module(x, operator=oracle_operator)
    assert got.tokens.shape == (1, P, dim) and got.offset is x.offset
    diff = (got.tokens.float() - want.tokens.float()).abs()
    assert float(diff.max()) <= 2e-2 and float(diff.mean()) <= 2e-3, (float(diff.max()), float(diff.mean()))
    bound = (math.sqrt(64) * gain) ** 2 * 0.125
    assert (bound <= cuda_extension.flash_attn.FOLD_SCALE_MAX_LOGIT) == (gain == 1.0)
