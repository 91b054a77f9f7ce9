"""Packed ("jagged") self-attention on the HIP kernels against the same attention run sample by sample, as in the
reference's test/auto_test/test_jagged_attention.py:75-153 (packing isolation, qk-norm and 2-D RoPE on packed
rows).  head_dim is 64 here (the reference's toy case uses 16, which this build does not instantiate).  The
per-sample side is computed in fp32 on the CPU from the same fp16 weights and inputs; tolerance atol = 5e-3,
rtol = 1e-2 for fp16 outputs of magnitude ~0.3 (the reference compares two fp16 GPU paths at 1e-3)."""

import pytest
import torch

import oracle
from come_amd.common import RotaryPositionEmbedding2D, prepare_packed_self_attention_qkv
from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func, infer_flash_attn_varlen_max_seqlen

pytestmark = pytest.mark.gpu
DEV, DTYPE = "cuda", torch.float16
DIM, HEADS, HEAD_DIM = 256, 4, 64


class Attention(torch.nn.Module):
    """qkv Linear -> optional q/k LayerNorm -> optional 2-D RoPE -> softmax attention -> proj."""

    def __init__(self, qk_norm: bool, rope: bool):
        super().__init__()
        self.qkv = torch.nn.Linear(DIM, 3 * DIM)
        self.proj = torch.nn.Linear(DIM, DIM)
        self.q_norm = torch.nn.LayerNorm(HEAD_DIM) if qk_norm else torch.nn.Identity()
        self.k_norm = torch.nn.LayerNorm(HEAD_DIM) if qk_norm else torch.nn.Identity()
        if qk_norm:
            with torch.no_grad():
                for n in (self.q_norm, self.k_norm):
                    n.weight.uniform_(0.5, 1.5)
                    n.bias.normal_(0, 0.1)
        self.rope = RotaryPositionEmbedding2D(100.0) if rope else None

    def per_sample(self, x: torch.Tensor, pos: torch.Tensor | None) -> torch.Tensor:
        """Dense reference for one sample ``x [n, DIM]`` on the CPU in fp32 arithmetic, rounding where the packed
        path stores 16-bit tensors (qkv, normalised / rotated q and k, attention output)."""
        w = {k: v.detach().cpu() for k, v in self.state_dict().items()}
        qkv = torch.nn.functional.linear(x.float(), w["qkv.weight"].float(), w["qkv.bias"].float()).to(DTYPE)
        qkv = qkv.view(-1, 3, HEADS, HEAD_DIM)
        norm = isinstance(self.q_norm, torch.nn.LayerNorm)
        qkv = oracle.qk_norm_rope(qkv, w.get("q_norm.weight"), w.get("q_norm.bias"), w.get("k_norm.weight"),
                                  w.get("k_norm.bias"), 1e-5, pos if self.rope is not None else None, 100.0,
                                  apply_norm=norm)
        out, _ = oracle.biased_varlen_attention(qkv, torch.tensor([0, x.shape[0]]), None, HEAD_DIM ** -0.5)
        out = out.to(DTYPE).reshape(-1, DIM)
        return torch.nn.functional.linear(out.float(), w["proj.weight"].float(), w["proj.bias"].float())

    @torch.no_grad()
    def packed(self, tokens: torch.Tensor, offset: torch.Tensor, pos: torch.Tensor | None) -> torch.Tensor:
        """``tokens [P, DIM]`` on the GPU, all samples at once."""
        P = tokens.shape[0]
        qkv = self.qkv(tokens).view(P, 3, HEADS, HEAD_DIM)
        qkv = prepare_packed_self_attention_qkv(qkv, self.q_norm, self.k_norm, self.rope, pos, DTYPE)
        cu = offset.to(torch.int32)
        out = flash_attn_varlen_qkvpacked_func(qkv, cu, infer_flash_attn_varlen_max_seqlen(cu),
                                               softmax_scale=HEAD_DIM ** -0.5)
        return self.proj(out.reshape(P, DIM))


def run_case(qk_norm, rope, grids):
    torch.manual_seed(42)
    attn = Attention(qk_norm, rope).to(DEV, DTYPE).eval()
    samples = [torch.randn(h * w, DIM).to(DTYPE) for h, w in grids]
    positions = None
    if rope:
        positions = [torch.stack(torch.meshgrid(torch.arange(h), torch.arange(w), indexing="ij"), -1).reshape(-1, 2)
                     for h, w in grids]
    lens = [s.shape[0] for s in samples]
    offset = torch.tensor([0] + lens).cumsum(0)
    packed = attn.packed(torch.cat(samples).to(DEV), offset.to(DEV),
                         torch.cat(positions).to(DEV) if rope else None).float().cpu()
    for i, x in enumerate(samples):
        ref = attn.per_sample(x, positions[i] if rope else None)
        torch.testing.assert_close(packed[offset[i]:offset[i + 1]], ref, atol=5e-3, rtol=1e-2)


def test_basic_no_rope_no_qknorm():
    run_case(False, False, [(2, 5), (4, 5), (3, 5), (2, 4)])


def test_with_qknorm():
    run_case(True, False, [(2, 5), (4, 5), (3, 5), (2, 4)])


def test_with_rope():
    run_case(False, True, [(2, 5), (4, 5), (3, 5), (2, 4)])


def test_with_qknorm_and_rope_longer_samples():
    run_case(True, True, [(12, 13), (9, 31), (37, 28), (5, 5)])


def test_single_sample():
    run_case(False, False, [(5, 5)])


def test_uniform_length():
    run_case(False, False, [(4, 4)] * 4)
