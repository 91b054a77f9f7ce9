"""The work-queue launch of the varlen attention (``COME_ATTN_WORK_QUEUE``): a one-workgroup kernel turns ``cu_seqlens``
into per-XCD lists of (segment, head, query block) items without empty entries, resident workgroups claim items from
them and keep their K / V ring running from one item to the next.  Whatever the schedule, every query block is computed
exactly once with the same arithmetic: the outputs equal those of the default launch (one workgroup per query block)
bit for bit, which in turn is checked against the closed form everywhere else; a few cases are compared with the oracle
here as well."""

import math

import numpy as np
import pytest
import torch

import oracle
from come_amd import _lib
from come_amd.cuda_extension import (flash_attn_varlen_qkvpacked_func,
                                     flash_attn_varlen_qkvpacked_func_w_perkey_bias)

pytestmark = pytest.mark.gpu
DEV = "cuda"

CASES = [
    ([32, 48, 24, 24], 4), ([1], 1), ([3, 1, 2], 2), ([65], 3), ([257, 31], 5), ([700, 333, 64], 4), ([1000], 16),
    ([300, 0, 77, 812, 5, 640, 0], 3),                  # empty segments, 21 units (not a multiple of 8)
    ([256] * 9, 2), ([255, 256, 257, 511, 512, 513, 1023, 1024, 1025], 1), ([2048, 2047, 1], 2),
    ([686, 862, 733, 790] * 8, 16),                     # the benchmark's frames: 512 units of 3 - 4 blocks
    ([305 + 7 * i for i in range(26)] * 5, 16),         # 130 short segments: several items per resident workgroup
]


def _cu(lens):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)


def _inputs(lens, H, dtype, seed, bias_kind="counts"):
    g = torch.Generator().manual_seed(seed)
    P = sum(lens)
    qkv = torch.randn(P, 3, H, 64, generator=g).to(dtype)
    if bias_kind == "counts":
        bias = torch.where(torch.rand(P, generator=g) < 0.3, math.log(9.0), 0.0).to(dtype)
    else:
        bias = None
    return qkv, bias, _cu(lens)


def _both(qkv, bias, cu, max_len, **kw):
    run = flash_attn_varlen_qkvpacked_func if bias is None else flash_attn_varlen_qkvpacked_func_w_perkey_bias
    extra = {} if bias is None else {"perkey_bias": bias}
    plain = run(qkv, cu, max_len, return_attn_probs=True, **extra, **kw)
    queued = run(qkv, cu, max_len, return_attn_probs=True, work_queue=True, **extra, **kw)
    return plain, queued


@pytest.mark.parametrize("mode", ["exact", "folded"])
@pytest.mark.parametrize("lens,H", CASES, ids=[f"{len(c[0])}seg-max{max(c[0])}-h{c[1]}" for c in CASES])
def test_queue_launch_equals_default_launch_bit_for_bit(lens, H, mode):
    qkv, bias, cu = _inputs(lens, H, torch.bfloat16, seed=len(lens) * 131 + H)
    qkv, bias, cu = qkv.to(DEV), bias.to(DEV), cu.to(DEV)
    assert _lib.load().come_attn_queue_bytes(len(lens), H, max(lens)) > 0
    (out, lse, _), (out_q, lse_q, _) = _both(qkv, bias, cu, max(lens), scale_mode=mode)
    assert bool(torch.isfinite(out_q).all()) and bool(torch.isfinite(lse_q).all())
    assert torch.equal(out_q, out)
    assert torch.equal(lse_q, lse)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_queue_launch_against_the_oracle(dtype):
    lens, H = [700, 333, 64, 1, 513], 4
    qkv, bias, cu = _inputs(lens, H, dtype, seed=5)
    ref, ref_lse = oracle.biased_varlen_attention(qkv, cu, bias)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens),
                                                                 perkey_bias=bias.to(DEV), return_attn_probs=True,
                                                                 work_queue=True)
    diff = (out.float().cpu() - ref).abs()
    assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=4e-3, rtol=1e-3)


def test_any_upper_bound_of_the_lengths_and_no_bias():
    """The list holds the blocks that exist, however far ``max_seqlen`` lies above the segments (up to the 2048 keys
    the queue launch is built for; beyond that the flag is ignored and the default launch runs)."""
    lens, H = [300, 77, 812, 5, 640], 3
    qkv, _, cu = _inputs(lens, H, torch.bfloat16, seed=9, bias_kind=None)
    qkv, cu = qkv.to(DEV), cu.to(DEV)
    tight = flash_attn_varlen_qkvpacked_func(qkv, cu, max(lens))
    for bound in (813, 1024, 1500, 2048, 2049, 4000):
        assert (_lib.load().come_attn_queue_bytes(len(lens), H, bound) > 0) == (bound <= 2048)
        got = flash_attn_varlen_qkvpacked_func(qkv, cu, bound, work_queue=True)
        assert torch.equal(got, tight), f"max_seqlen {bound}"


def test_block_that_has_to_be_computed_again_inside_the_queue_launch():
    """A late key far beyond the range of the stored probabilities makes its workgroup compute the block again, which
    uses the ring stages for itself: the next item of that workgroup starts from scratch.  Items before and after it
    are unaffected."""
    lens, H = [1500, 90, 700, 700, 300, 1200], 2
    P = sum(lens)
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(P, 3, H, 64, generator=g).bfloat16()
    bias = torch.zeros(P)
    bias[700], bias[1023], bias[1500 + 40] = 100.0, 200.0, 100.0
    bias[1590 + 1400 + 150] = 300.0
    bias = bias.bfloat16()
    cu = _cu(lens)
    ref, _ = oracle.biased_varlen_attention(qkv, cu, bias)
    (out, lse, _), (out_q, lse_q, _) = _both(qkv.to(DEV), bias.to(DEV), cu.to(DEV), max(lens))
    assert torch.equal(out_q, out) and torch.equal(lse_q, lse)
    torch.testing.assert_close(out_q.float().cpu(), ref, atol=1e-2, rtol=1e-2)


def test_c_abi_flag_buffer_rules_and_the_built_in_array():
    """Through the C ABI: the flag needs ``come_attn_queue_bytes`` of buffer (a smaller one: the default launch, same
    bits), the allocation-free entry point keeps the queue in its own array, unknown flag bits are rejected."""
    lib = _lib.load()
    lens, H = [700, 300, 1000, 77], 16
    qkv, bias, cu = _inputs(lens, H, torch.bfloat16, seed=2)
    qkv, bias, cu = qkv.to(DEV), bias.to(DEV), cu.to(DEV)
    P = sum(lens)
    need = lib.come_attn_queue_bytes(len(lens), H, max(lens))
    assert need == 4 * (16 + 8 * ((len(lens) * H + 7) // 8) * ((max(lens) + 255) // 256))
    assert lib.come_attn_queue_bytes(1, 16, 25536) == 0 and lib.come_attn_queue_bytes(70000, 1, 512) == 0
    q, k, v = qkv.unbind(1)

    def call(entry, work, flags):
        out = torch.full((P, H, 64), float("nan"), dtype=torch.bfloat16, device=DEV)
        lse = torch.full((H, P), float("nan"), dtype=torch.float32, device=DEV)
        args = [q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.COME_BF16, q.stride(0), q.stride(1), k.stride(0),
                k.stride(1), v.stride(0), v.stride(1), cu.data_ptr(), len(lens), P, H, 64, bias.data_ptr(), max(lens),
                0.125, out.data_ptr(), out.stride(0), out.stride(1), lse.data_ptr()]
        stream = _lib.current_stream(qkv.device)
        if entry == "static":
            rc = lib.come_attn_varlen_fwd_static(*args, flags, stream)
        else:
            rc = lib.come_attn_varlen_fwd_ws(*args, _lib.ptr(work), 0 if work is None else work.numel(), flags, stream)
        torch.cuda.synchronize()
        return rc, out, lse

    rc, want, want_lse = call("ws", None, 0)
    assert rc == 0
    work = torch.full((need,), 0xAB, dtype=torch.uint8, device=DEV)       # no particular contents are expected
    for _ in range(2):                                                    # the counters are reset by every call
        rc, out, lse = call("ws", work, _lib.COME_ATTN_WORK_QUEUE)
        assert rc == 0 and torch.equal(out, want) and torch.equal(lse, want_lse)
    rc, out, _ = call("ws", work[: need - 16], _lib.COME_ATTN_WORK_QUEUE)  # too small: flag ignored
    assert rc == 0 and torch.equal(out, want)
    rc, out, _ = call("ws", None, _lib.COME_ATTN_WORK_QUEUE)
    assert rc == 0 and torch.equal(out, want)
    for _ in range(2):
        rc, out, lse = call("static", None, _lib.COME_ATTN_WORK_QUEUE | _lib.COME_ATTN_FOLD_SCALE)
        rc2, want_f, want_f_lse = call("ws", None, _lib.COME_ATTN_FOLD_SCALE)
        assert rc == 0 and rc2 == 0 and torch.equal(out, want_f) and torch.equal(lse, want_f_lse)
    rc, _, _ = call("ws", None, 8)
    assert rc == 1 and b"flags" in lib.come_last_error()
