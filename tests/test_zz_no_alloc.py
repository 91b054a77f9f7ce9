"""GPU test of the allocation-free attention entry point ``come_attn_varlen_fwd_static``: called through the C ABI
and compared bit for bit with ``come_attn_varlen_fwd_ws`` (the same kernels over a caller-supplied buffer) on two
calls in a row, the second on a smaller input, then on a shape whose pieces do not fit the built-in array."""

import pytest
import torch

from come_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"
HEADS, D = 16, 64


def _inputs(lengths, seed, heads=HEADS):
    g = torch.Generator().manual_seed(seed)
    total = sum(lengths)
    qkv = torch.randn(total, 3, heads, D, generator=g).bfloat16().to(DEV)
    counts = torch.where(torch.rand(total, generator=g) < 0.1, 9.0, 1.0)
    bias = counts.log().bfloat16().to(DEV)
    cu = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32, device=DEV)
    return qkv, bias, cu


def _call(entry, qkv, bias, cu, max_len, work=None, flags=0, out=None, lse=None):
    lib = _lib.load()
    total, _, heads, _ = qkv.shape
    q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]
    if out is None:
        out = torch.full((total, heads, D), float("nan"), dtype=qkv.dtype, device=DEV)
        lse = torch.full((heads, total), float("nan"), dtype=torch.float32, device=DEV)
    args = [q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.dtype_code(qkv.dtype),
            q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
            cu.data_ptr(), cu.numel() - 1, total, heads, D, bias.data_ptr(), max_len, 0.125,
            out.data_ptr(), out.stride(0), out.stride(1), lse.data_ptr()]
    stream = _lib.current_stream(qkv.device)
    if entry == "static":
        status = lib.come_attn_varlen_fwd_static(*args, flags, stream)
    else:
        status = lib.come_attn_varlen_fwd_ws(*args, _lib.ptr(work), 0 if work is None else work.numel(), flags, stream)
    return status, out, lse


def test_static_matches_workspace_entry_twice_then_rejects_oversize():
    lib = _lib.load()
    limit = lib.come_attn_static_work_bytes()
    assert limit == 64 << 20
    # first a 25 536-token segment, then a smaller one (12 288): both shapes use the key-split tail, i.e. the buffer
    # (the second shape also with the other way of applying the scale: the flag travels through this entry point too)
    for seed, lengths, flags in ((0, [25536], 0), (1, [12288], 0), (1, [12288], _lib.COME_ATTN_FOLD_SCALE)):
        need = lib.come_attn_work_bytes(len(lengths), sum(lengths), HEADS, max(lengths))
        assert 0 < need <= limit, "the shape must exercise the work buffer"
        qkv, bias, cu = _inputs(lengths, seed)
        work = torch.empty(need, dtype=torch.uint8, device=DEV)
        st_ws, out_ws, lse_ws = _call("ws", qkv, bias, cu, max(lengths), work, flags)
        st, out, lse = _call("static", qkv, bias, cu, max(lengths), None, flags)
        assert st_ws == 0 and st == 0, lib.come_last_error()
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
        assert torch.equal(out, out_ws)
        assert torch.equal(lse, lse_ws)
        # the call itself takes no device memory: with its outputs already there, the free memory the driver
        # reports and what torch's allocator holds are the same before and after a (warm) call
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        free_before, held_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
        st, _, _ = _call("static", qkv, bias, cu, max(lengths), None, flags, out=out, lse=lse)
        torch.cuda.synchronize()
        assert st == 0
        assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == held_before
        assert torch.equal(out, out_ws)
        # and it differs from a launch that never used a buffer only by rounding (not by garbage from the array)
        st_plain, out_plain, _ = _call("ws", qkv, bias, cu, max(lengths), None)
        assert st_plain == 0
        diff = (out.float() - out_plain.float()).abs()
        assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3

    # a shape that uses no buffer at all runs as the plain entry point does
    qkv, bias, cu = _inputs([700, 300, 1000], 2)
    assert lib.come_attn_work_bytes(3, 2000, HEADS, 1000) == 0
    st, out, lse = _call("static", qkv, bias, cu, 1000)
    st_ws, out_ws, lse_ws = _call("ws", qkv, bias, cu, 1000, None)
    assert st == 0 and st_ws == 0
    assert torch.equal(out, out_ws) and torch.equal(lse, lse_ws)

    # pieces beyond the built-in array: a clear error, nothing enqueued
    lengths, heads = [51712] * 3, 2
    assert lib.come_attn_work_bytes(3, sum(lengths), heads, max(lengths)) > limit
    qkv, bias, cu = _inputs(lengths, 3, heads=heads)
    st, out, _ = _call("static", qkv, bias, cu, max(lengths))
    assert st == 2
    msg = lib.come_last_error().decode()
    assert "come_attn_varlen_fwd_static" in msg and "come_attn_varlen_fwd_ws" in msg and str(limit) in msg
    torch.cuda.synchronize()
    assert torch.isnan(out.float()).all()                         # untouched


def test_static_entry_point_inside_a_captured_graph():
    """The caller the entry point exists for: the launch is recorded into a HIP graph (the address of the built-in
    array is looked up before the capture through ``come_attn_static_work_bytes``) and replayed several times, with
    eager work and synchronisations of the program between the replays; every replay reproduces the eager result bit
    for bit, on changed inputs as well."""
    lib = _lib.load()
    assert lib.come_attn_static_work_bytes() == 64 << 20          # also resolves the array's address on this device
    lengths = [12288]                                             # uses the key-split tail, i.e. the array
    assert lib.come_attn_work_bytes(1, 12288, HEADS, 12288) > 0
    qkv, bias, cu = _inputs(lengths, 7)
    total = sum(lengths)
    out = torch.empty(total, HEADS, D, dtype=qkv.dtype, device=DEV)
    lse = torch.empty(HEADS, total, dtype=torch.float32, device=DEV)
    st, want, want_lse = _call("static", qkv, bias, cu, max(lengths))
    assert st == 0
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        st, _, _ = _call("static", qkv, bias, cu, max(lengths), out=out, lse=lse)      # warm-up on the capturing stream
        assert st == 0
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            st, _, _ = _call("static", qkv, bias, cu, max(lengths), out=out, lse=lse)
        assert st == 0, lib.come_last_error()
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        out.fill_(float("nan"))
        lse.fill_(float("nan"))
        scratch_work = torch.randn(1 << 20, device=DEV).sum()      # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(lse, want_lse), f"replay {replay}"
        assert bool(torch.isfinite(scratch_work))
    # new inputs in the same buffers: the graph holds pointers, not data
    qkv2, bias2, _ = _inputs(lengths, 8)
    st, want2, want2_lse = _call("static", qkv2, bias2, cu, max(lengths))
    torch.cuda.synchronize()
    qkv.copy_(qkv2)
    bias.copy_(bias2)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want2) and torch.equal(lse, want2_lse)
