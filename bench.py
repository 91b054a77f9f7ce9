"""Benchmark of the Co-Me hot path on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints ONE JSON line.

Headline ("step"): one forward pass of the biased varlen attention over the benchmark
attention configuration (16 heads x 64, two packed sequences of 25 536 and 21 848 tokens after a
50 % / 60 % 3x3 merge of 32 frames of 37x37 patches, bias = log(count), bf16).  Its throughput is
algorithmic flops (sum over segments of 4 L^2 d H) per second.

The same line carries, under ``other``, the merge / unmerge microbenchmark (16 frames of 37x37,
C = 1024, bf16, 3x3 windows, ratio 0.5) as GB/s of algorithmic bytes with its own roofline, and
the rate of the whole confidence-guided merge (selection + plan in one launch, then the gather-mean).

``roofline`` times the dominant kernel with HIP events on the launch stream; ``cpu_baseline`` times
the reference's PyTorch CPU path (SDPA with the bias as attn_mask) on the same workload on the host
cores, stopped after about 20 s of work.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0       # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E

# HBM bytes per launch of each kernel on exactly the workloads built below, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE passes (KiB per dispatch), FETCH_SIZE scaled by 2.000 and WRITE_SIZE by 1.000 -- the factors a 256 MiB
# device copy (``--only copy``) gives for the same counters.  Each entry names the summary under profiles/ that holds
# the run it was read from; a kernel change means a new run of the commands written there and new numbers here.
TRAFFIC = {
    "attn": {"bytes": int((266508 * 2.000 + 97733) * 1024), "source": "profiles/attn_fwd_c3.txt"},
    "merge": {"bytes": int((22072 * 2.000 + 25943) * 1024), "source": "profiles/merge_c2_r050.txt"},
    "unmerge": {"bytes": int((13632 * 2.000 + 43970) * 1024), "source": "profiles/unmerge_c2_r050.txt"},
}
TRAFFIC_BYTES = {k: v["bytes"] for k, v in TRAFFIC.items()}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-CPU baseline leg")
    ap.add_argument("--no-other", action="store_true", help="skip the merge / unmerge microbenchmarks")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end aggregator leg")
    ap.add_argument("--scale-mode", choices=["auto", "exact", "folded"], default="auto",
                    help="with --only frame / stress_frames: how softmax_scale is applied (one kernel per profiler run)")
    ap.add_argument("--only", choices=["stress_frames", "attn", "merge", "unmerge", "pair", "dtypes", "bias", "refmerge", "prologue", "prologue_k", "copy", "exact", "folded", "widths", "select", "e2e", "stress", "stress_e2e", "frame"], default=None,
                    help="run a single kernel in a loop (for profilers); prints a short JSON line")
    return ap.parse_args()


# ------------------------------------------------------------------------------------------
# synthetic workloads
# ------------------------------------------------------------------------------------------

def packed_counts(frames: int, windows: int, specials: int, leftover: int, merged_windows: int, gen):
    """Counts (1 or 9) of one packed sequence in layout order: per frame
    [specials | windows (one 9 or nine 1s) | leftover positions]; ``merged_windows`` windows are chosen
    jointly over all frames."""
    import torch

    chosen = torch.zeros(frames * windows, dtype=torch.bool)
    chosen[torch.randperm(frames * windows, generator=gen)[:merged_windows]] = True
    chosen = chosen.reshape(frames, windows)
    parts = []
    for f in range(frames):
        parts.append(torch.ones(specials))
        w = torch.where(chosen[f][:, None], torch.tensor([9.0] + [0.0] * 8), torch.ones(9)).reshape(-1)
        parts.append(w[w > 0])
        parts.append(torch.ones(leftover))
    return torch.cat(parts)


def make_attention_workload(device):
    import torch

    gen = torch.Generator().manual_seed(0)
    H, D = 16, 64
    counts0 = packed_counts(32, 144, 5, 73, 2304, gen)      # ratio 0.50 -> 25 536 tokens
    counts1 = packed_counts(32, 144, 5, 73, 2765, gen)      # ratio 0.60 -> 21 848 tokens
    lens = [counts0.numel(), counts1.numel()]
    assert lens == [25536, 21848], lens
    P = sum(lens)
    torch.manual_seed(0)
    qkv = torch.randn(P, 3, H, D, device=device, dtype=torch.float32).bfloat16()
    bias = torch.cat([counts0, counts1]).log().bfloat16().to(device)
    cu = torch.tensor([0, lens[0], P], dtype=torch.int32, device=device)
    flops = sum(4.0 * L * L * D * H for L in lens)
    return dict(qkv=qkv, bias=bias, cu=cu, lens=lens, flops=flops, H=H, D=D)


def smooth_confidence(frames, H, W, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    a = torch._standard_gamma(torch.full((frames, H, W), 2.0), generator=g)
    b = torch._standard_gamma(torch.full((frames, H, W), 5.0), generator=g)
    x = a / (a + b)                                            # Beta(2, 5)
    r = 9
    ker = torch.exp(-torch.arange(-r, r + 1).float() ** 2 / (2 * 3.0 ** 2))
    ker = ker / ker.sum()
    y = torch.nn.functional.pad(x[:, None], (r, r, r, r), mode="reflect")
    y = torch.nn.functional.conv2d(y, ker.view(1, 1, 1, -1))
    y = torch.nn.functional.conv2d(y, ker.view(1, 1, -1, 1))[:, 0]
    return 0.5 * x + 0.5 * y


# ------------------------------------------------------------------------------------------
# timed legs
# ------------------------------------------------------------------------------------------

def time_loop(fn, steps, warmup):
    """Returns (wall seconds for `steps` calls, HIP-event milliseconds for the same region)."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, start.elapsed_time(stop)


def bench_attention(steps, warmup, device, scale_mode="auto"):
    """The headline: the operator as a caller without any knowledge of its logits calls it (``scale_mode="auto"`` on
    a plain tensor: softmax_scale applied in fp32 to every score, the reference's arithmetic)."""
    from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias

    w = make_attention_workload(device)
    max_len = max(w["lens"])

    def step():
        return flash_attn_varlen_qkvpacked_func_w_perkey_bias(w["qkv"], w["cu"], max_len, perkey_bias=w["bias"],
                                                              softmax_scale=0.125, scale_mode=scale_mode)

    wall, ev_ms = time_loop(step, steps, warmup)
    return w, wall, ev_ms


def jittered_frame_masks(conf, ratio, jitter, seed):
    """Per-frame selection for the stress workload: frame f merges its ``round(r_f * M)`` lowest-confidence 3x3
    windows with ``r_f = ratio + U(-jitter, jitter)`` (workload synthesis on the host side of the bench, torch)."""
    import torch

    frames, H, W = conf.shape
    mh, mw = H // 3, W // 3
    means = conf[:, : mh * 3, : mw * 3].reshape(frames, mh, 3, mw, 3).mean(dim=(2, 4)).reshape(frames, mh * mw)
    g = torch.Generator().manual_seed(seed)
    r = ratio + (torch.rand(frames, generator=g) * 2 - 1) * jitter
    k = (r * mh * mw).round().long().clamp(0, mh * mw)
    order = means.argsort(dim=1)
    rank = torch.empty_like(order)
    rank.scatter_(1, order, torch.arange(mh * mw).expand(frames, -1))
    return rank < k[:, None]


def merge_workload(device, ratio=0.5, sets=None, frames=16, H=37, W=37, jitter=None, dtype=None, C=1024):
    """Merge microbenchmark: 16 frames, 37x37 patches + 5 specials, C = 1024, bf16, over rotating input / output
    buffer sets.  Every stream has to come from HBM, not from the 256 MB Infinity Cache, so the sets of each tensor a
    kernel reads must exceed the cache on their own: ``sets=None`` takes as many as bring the packed rows (the
    smallest stream, read by the unmerge) to 320 MB, at least 8.  (With 8 sets = 209 MB of packed rows at ratio 0.5
    the unmerge read them from the cache and measured 6.2 instead of 4.7 TB/s.)  With ``jitter`` the mask comes from
    ``jittered_frame_masks`` instead of the joint quantile selection."""
    import torch
    from come_amd import _lib

    S0 = 5
    N = S0 + H * W
    dtype = torch.bfloat16 if dtype is None else dtype
    code, esize = _lib.dtype_code(dtype), torch.empty(0, dtype=dtype).element_size()
    lib = _lib.load()
    conf = smooth_confidence(frames, H, W, seed=0).to(device)
    M = (H // 3) * (W // 3)
    tail = H * W - M * 9
    mask = torch.empty(frames, M, dtype=torch.uint8, device=device)
    means = torch.empty(frames, M, dtype=torch.float32, device=device)
    offsets = torch.empty(frames + 1, dtype=torch.int32, device=device)
    prefix = torch.empty(frames, M, dtype=torch.int32, device=device)
    stream = _lib.current_stream(device)

    if jitter is not None:
        mask.copy_(jittered_frame_masks(conf.cpu(), ratio, jitter, seed=1).to(torch.uint8))

    def select_and_plan():
        if jitter is None:         # confidence -> mask -> plan in one launch
            _lib.check(lib.come_select_plan(conf.data_ptr(), _lib.COME_F32, 1, frames, H, W, 3, 3, 0, ratio, S0,
                                            means.data_ptr(), mask.data_ptr(), offsets.data_ptr(), prefix.data_ptr(),
                                            None, 0, stream))
        else:
            _lib.check(lib.come_merge_plan(mask.data_ptr(), frames, M, S0, 9, tail, offsets.data_ptr(),
                                           prefix.data_ptr(), stream))

    select_and_plan()
    P = int(offsets[-1].item())
    if sets is None:
        packed_bytes = P * C * esize
        sets = 2 if packed_bytes < (1 << 20) else max(8, -(-320_000_000 // packed_bytes))
    torch.manual_seed(0)
    tokens = [torch.randn(frames, N, C, device=device).to(dtype) for _ in range(sets)]
    outs = [torch.empty(P, C, dtype=dtype, device=device) for _ in range(sets)]
    index_map = torch.empty(frames * N, dtype=torch.int32, device=device)
    counts = torch.empty(P, dtype=torch.int32, device=device)
    restored = [torch.empty(frames * N, C, dtype=dtype, device=device) for _ in range(sets)]
    state = {"i": 0}

    def merge_only():
        i = state["i"] = (state["i"] + 1) % sets
        _lib.check(lib.come_token_merge(tokens[i].data_ptr(), code, frames, N, C, S0, 3, 3, H, W,
                                        mask.data_ptr(), offsets.data_ptr(), prefix.data_ptr(), outs[i].data_ptr(), P,
                                        None, index_map.data_ptr(), None, counts.data_ptr(), stream))

    def pipeline():
        select_and_plan()
        merge_only()

    def split_only():
        i = state["i"] = (state["i"] + 1) % sets
        _lib.check(lib.come_token_split(outs[i].data_ptr(), code, P, C, None, index_map.data_ptr(),
                                        frames * N, restored[i].data_ptr(), stream))

    merge_bytes = (frames * N * C * esize + P * C * esize + frames * N * 4 + P * 4 + frames * H * W * 4
                   + (frames + 1) * 4)
    split_bytes = P * C * esize + frames * N * 4 + frames * N * C * esize
    return dict(merge_only=merge_only, pipeline=pipeline, select_and_plan=select_and_plan, split_only=split_only, P=P, merge_bytes=merge_bytes,
                split_bytes=split_bytes, frames=frames, N=N, C=C, ratio=ratio, tokens=tokens, conf=conf,
                counts=counts, offsets=offsets, outs=outs, restored=restored, index_map=index_map,
                keep=(mask, means, prefix))


def bench_merge_unmerge(device, iters=200, warmup=20):
    w = merge_workload(device)
    for _ in range(len(w["outs"])):
        w["merge_only"]()                                       # fill every output set before unmerge reads it
    _, merge_ms = time_loop(w["merge_only"], iters, warmup)
    _, pipe_ms = time_loop(w["pipeline"], iters, warmup)
    _, select_plan_ms = time_loop(w["select_and_plan"], iters, warmup)
    _, split_ms = time_loop(w["split_only"], iters, warmup)
    merge_gbs = w["merge_bytes"] / (merge_ms / iters * 1e-3) / 1e9
    split_gbs = w["split_bytes"] / (split_ms / iters * 1e-3) / 1e9
    return w, {
        "merge": {"workload": "C2 merge: 16 frames 37x37+5, C=1024 bf16, 3x3, ratio 0.5, P=%d" % w["P"],
                  "value": round(merge_gbs, 1), "unit": "GB/s", "us_per_call": round(merge_ms / iters * 1e3, 2),
                  "algorithmic_bytes": w["merge_bytes"], "iters": iters, "rotating_buffer_sets": len(w["outs"]),
                  "roofline": {"bound": "hbm", "achieved": round(merge_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                               "frac": round(merge_gbs / PEAK_HBM_GBS, 4), "traffic": TRAFFIC_BYTES["merge"],
                               "traffic_source": TRAFFIC["merge"]["source"]},
                  # confidence -> mask -> plan (one launch, come_select_plan) -> gather-mean: the whole
                  # confidence-guided merge, same algorithmic bytes (the selection reads the confidence map and
                  # writes a few KB of bookkeeping, both already counted)
                  "select_plan_merge": {"us_per_call": round(pipe_ms / iters * 1e3, 2),
                                        "value": round(w["merge_bytes"] / (pipe_ms / iters * 1e-3) / 1e9, 1), "unit": "GB/s",
                                        "frac": round(w["merge_bytes"] / (pipe_ms / iters * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)},
                  "select_plan_us": round(select_plan_ms / iters * 1e3, 2)},
        "unmerge": {"workload": "C2 unmerge: P=%d -> %d rows, C=1024 bf16" % (w["P"], w["frames"] * w["N"]),
                    "value": round(split_gbs, 1), "unit": "GB/s", "us_per_call": round(split_ms / iters * 1e3, 2),
                    "algorithmic_bytes": w["split_bytes"], "iters": iters, "rotating_buffer_sets": len(w["outs"]),
                    "roofline": {"bound": "hbm", "achieved": round(split_gbs, 1), "peak": PEAK_HBM_GBS,
                                 "unit": "GB/s", "frac": round(split_gbs / PEAK_HBM_GBS, 4),
                                 "traffic": TRAFFIC_BYTES["unmerge"],
                                 "traffic_source": TRAFFIC["unmerge"]["source"]}},
    }


def bench_merge_operator(device, w, iters=200, warmup=20):
    """The confidence-guided merge as a caller of ``co_me_cuext.co_me_select_merge_2d`` sees it: selection + plan,
    the 4-byte device-to-host read of the packed row count that sizes the output, the allocations from torch's caching
    allocator and the gather-mean, per call on the wall clock (the read makes every call synchronous), over the
    rotating token sets of the microbenchmark.  Next to it the reference-shaped chain of two calls
    (``co_me_select_windows`` then ``co_me_token_merge_2d_cuda``), which plans in a launch of its own."""
    import torch
    from come_amd.cuda_extension import co_me_cuext

    tokens, conf, sets = w["tokens"], w["conf"], len(w["tokens"])
    frames, H, W = w["frames"], 37, 37
    state = {"i": 0}

    def fused():
        i = state["i"] = (state["i"] + 1) % sets
        return co_me_cuext.co_me_select_merge_2d(tokens[i], conf, 1, 5, 3, 3, H, W, w["ratio"])

    def two_calls():
        i = state["i"] = (state["i"] + 1) % sets
        mask = co_me_cuext.co_me_select_windows(conf, 1, 3, 3, w["ratio"])
        return co_me_cuext.co_me_token_merge_2d_cuda(tokens[i], 5, 3, 3, H, W, mask, index_dtype=torch.int32,
                                                     count_dtype=torch.int32)

    def median_us(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(iters):
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e6)
        return sorted(times)[len(times) // 2]

    fused_us, two_us = median_us(fused), median_us(two_calls)
    assert fused()[0].shape[0] == w["P"]
    return {"co_me_select_merge_2d_us": round(fused_us, 1),
            "GBs": round(w["merge_bytes"] / (fused_us * 1e-6) / 1e9, 1),
            "frac": round(w["merge_bytes"] / (fused_us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4),
            "select_then_merge_calls_us": round(two_us, 1), "statistic": "median wall time per call, synchronised",
            "includes": "selection + plan launch, 4-byte read of the packed row count, output allocation, merge launch"}


def bench_write_floor(device, nbytes, iters=200, warmup=20):
    """A plain fill of ``nbytes`` over rotating buffers: what this part sustains for a stream of writes of the size
    of the unmerge's output, the dominant stream of that kernel."""
    import torch

    sets = max(8, -(-320_000_000 // nbytes))
    bufs = [torch.empty(nbytes // 4, dtype=torch.int32, device=device) for _ in range(sets)]
    state = {"i": 0}

    def fill():
        i = state["i"] = (state["i"] + 1) % sets
        bufs[i].fill_(1)

    _, ms = time_loop(fill, iters, warmup)
    return {"bytes": nbytes, "us_per_call": round(ms / iters * 1e3, 2), "GBs": round(nbytes / (ms / iters * 1e-3) / 1e9, 1),
            "kernel": "torch fill_", "rotating_buffer_sets": sets}


def bench_merge_caller_dtypes(device, iters=200, warmup=20):
    """The two other tensors the fused aggregator of the reference merges (vggt/fused.py:126-129): the fp32 residual
    stream [frames, N, 1024] and the bf16 positions [frames, N, 2] (element-wise kernels: rows of 4 bytes)."""
    import torch

    out = {}
    for name, dtype, C in (("fp32_c1024", torch.float32, 1024), ("bf16_c2", torch.bfloat16, 2)):
        w = merge_workload(device, dtype=dtype, C=C)
        for _ in range(len(w["outs"])):
            w["merge_only"]()
        _, m_ms = time_loop(w["merge_only"], iters, warmup)
        _, s_ms = time_loop(w["split_only"], iters, warmup)
        out[name] = {"rotating_buffer_sets": len(w["outs"]),
                     "merge_us": round(m_ms / iters * 1e3, 2), "merge_bytes": w["merge_bytes"],
                     "merge_GBs": round(w["merge_bytes"] / (m_ms / iters * 1e-3) / 1e9, 1),
                     "unmerge_us": round(s_ms / iters * 1e3, 2), "unmerge_bytes": w["split_bytes"],
                     "unmerge_GBs": round(w["split_bytes"] / (s_ms / iters * 1e-3) / 1e9, 1)}
        del w
        torch.cuda.empty_cache()
    return out


def bench_reference_merge_shapes(device):
    """The shapes of the reference's own merge / split microbenchmark (test/benchmark/bench_token_merge.py:18-23:
    1-D groups of 4, fp32 tokens, random mask at 0.5), timed as that script times them: the whole Python call
    (``func_token_merge`` including its read of the packed row count, ``func_token_split``), synchronised, median."""
    import torch
    from come_amd.token_merger import func_token_merge, func_token_split

    def median_ms(fn, reps):
        fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
        return sorted(times)[len(times) // 2]

    out = {}
    for label, B, M, G, S, C in (("Small", 1, 256, 4, 0, 512), ("Medium", 32, 1024, 4, 2, 1024),
                                 ("Large", 128, 2048, 4, 2, 2048)):
        N = S + M * G
        torch.manual_seed(0)
        tokens = torch.randn(B, N, C, device=device)
        mask = torch.rand(B, M, device=device) < 0.5
        jag, rev = func_token_merge(tokens, S, G, mask)
        P = jag.tokens.shape[1]
        reps = 200 if label == "Small" else (50 if label == "Medium" else 10)
        m_ms = median_ms(lambda: func_token_merge(tokens, S, G, mask), reps)
        s_ms = median_ms(lambda: func_token_split(jag, rev, (1, B, N, C)), reps)
        nbytes = (B * N + P) * C * 4
        out[label] = {"shape": "B=%d N=%d C=%d G=%d fp32, P=%d" % (B, N, C, G, P), "merge_ms": round(m_ms, 4),
                      "merge_GBs": round(nbytes / (m_ms * 1e-3) / 1e9, 1), "split_ms": round(s_ms, 4),
                      "split_GBs": round(nbytes / (s_ms * 1e-3) / 1e9, 1)}
        del tokens, jag, rev
        torch.cuda.empty_cache()
    return out


def bench_unmerge_pair(device, w, iters=200, warmup=20):
    """Retained-layer step of the fused aggregator: two packed tensors restored to the dense grid side by side
    (``come_token_split_pair``), next to two ``come_token_split`` launches followed by ``torch.cat``."""
    import torch
    from come_amd import _lib

    lib, stream = _lib.load(), _lib.current_stream(device)
    rows, C, P, sets = w["frames"] * w["N"], w["C"], w["P"], len(w["outs"])
    wide = [torch.empty(rows, 2 * C, dtype=torch.bfloat16, device=device) for _ in range(sets)]
    far = sets // 2                     # the second source was last touched half a rotation (> 256 MB of traffic) ago
    state = {"i": 0}

    def pair():
        i = state["i"] = (state["i"] + 1) % sets
        _lib.check(lib.come_token_split_pair(w["outs"][i].data_ptr(), w["outs"][(i + far) % sets].data_ptr(),
                                             _lib.COME_BF16, P, C, None, w["index_map"].data_ptr(), rows,
                                             wide[i].data_ptr(), stream))

    def two_and_cat():
        i = state["i"] = (state["i"] + 1) % sets
        for j in (i, (i + far) % sets):
            _lib.check(lib.come_token_split(w["outs"][j].data_ptr(), _lib.COME_BF16, P, C, None,
                                            w["index_map"].data_ptr(), rows, w["restored"][j].data_ptr(), stream))
        torch.cat((w["restored"][i], w["restored"][(i + far) % sets]), dim=-1, out=wide[i])

    _, pair_ms = time_loop(pair, iters, warmup)
    _, cat_ms = time_loop(two_and_cat, iters, warmup)
    nbytes = 2 * P * C * 2 + rows * 4 + rows * 2 * C * 2
    gbs = nbytes / (pair_ms / iters * 1e-3) / 1e9
    return {"workload": "two packed [%d, %d] bf16 -> dense [%d, %d]" % (P, C, rows, 2 * C),
            "us_per_call": round(pair_ms / iters * 1e3, 2), "algorithmic_bytes": nbytes, "GBs": round(gbs, 1),
            "frac": round(gbs / PEAK_HBM_GBS, 4), "two_splits_and_cat_us": round(cat_ms / iters * 1e3, 2)}


def bench_merge_ratios(device, iters=200, warmup=20):
    """The merge / unmerge microbenchmark at the other two ratios of the configuration."""
    import torch

    out = {}
    for ratio in (0.25, 0.75):
        w = merge_workload(device, ratio=ratio)
        for _ in range(len(w["outs"])):
            w["merge_only"]()
        _, m_ms = time_loop(w["merge_only"], iters, warmup)
        _, s_ms = time_loop(w["split_only"], iters, warmup)
        out["r%03d" % round(ratio * 100)] = {
            "P": w["P"], "merge_us": round(m_ms / iters * 1e3, 2), "merge_bytes": w["merge_bytes"],
            "merge_GBs": round(w["merge_bytes"] / (m_ms / iters * 1e-3) / 1e9, 1),
            "merge_frac": round(w["merge_bytes"] / (m_ms / iters * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "unmerge_us": round(s_ms / iters * 1e3, 2), "unmerge_bytes": w["split_bytes"],
            "unmerge_GBs": round(w["split_bytes"] / (s_ms / iters * 1e-3) / 1e9, 1),
            "unmerge_frac": round(w["split_bytes"] / (s_ms / iters * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
        del w
        torch.cuda.empty_cache()
    return out


def attention_case(device, lens, counts, steps, warmup, H=16, D=64, scale_mode="auto", work_queue=False):
    """Times the biased attention on packed segments ``lens`` with per-key counts; returns (ms, TFLOP/s)."""
    import torch
    from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias

    P = sum(lens)
    torch.manual_seed(1)
    qkv = torch.randn(P, 3, H, D, device=device, dtype=torch.float32).bfloat16()
    bias = counts.float().log().bfloat16().to(device)
    bounds = [0]
    for n in lens:
        bounds.append(bounds[-1] + n)
    cu = torch.tensor(bounds, dtype=torch.int32, device=device)
    max_len = max(lens)
    _, ms = time_loop(lambda: flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, max_len, perkey_bias=bias,
                                                                             softmax_scale=0.125,
                                                                             scale_mode=scale_mode,
                                                                             work_queue=work_queue), steps, warmup)
    flops = sum(4.0 * n * n * D * H for n in lens)
    return ms / steps, flops / (ms / steps * 1e-3) / 1e12, flops


def bench_bias_overhead(device):
    """What the reference's own microbenchmark checks (test/benchmark/bench_flash_attn_w_bias.py: the per-key bias
    must cost next to nothing over the plain kernel): its head_dim 64, non-causal shapes and the headline shape,
    with and without bias."""
    import torch
    from come_amd.cuda_extension import (flash_attn_varlen_qkvpacked_func,
                                         flash_attn_varlen_qkvpacked_func_w_perkey_bias)

    out = {}
    shapes = (("tiny b=4 s=128 h=8 fp16", [128] * 4, 8, torch.float16), ("small b=8 s=256 h=16 fp16", [256] * 8, 16, torch.float16),
              ("small b=8 s=256 h=16 bf16", [256] * 8, 16, torch.bfloat16), ("headline L={25536,21848} h=16 bf16", [25536, 21848], 16, torch.bfloat16))
    for name, lens, H, dtype in shapes:
        P = sum(lens)
        torch.manual_seed(2)
        qkv = torch.randn(P, 3, H, 64, device=device).to(dtype)
        bias = (torch.randn(P, device=device) * 0.1).to(dtype)
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=device)
        steps = 200 if P < 10000 else 10
        _, plain_ms = time_loop(lambda: flash_attn_varlen_qkvpacked_func(qkv, cu, max(lens)), steps, 5)
        _, bias_ms = time_loop(lambda: flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, max(lens), perkey_bias=bias),
                               steps, 5)
        out[name] = {"plain_us": round(plain_ms / steps * 1e3, 2), "with_bias_us": round(bias_ms / steps * 1e3, 2),
                     "ratio": round(plain_ms / bias_ms, 4)}
    return out


def bench_qk_prologue(device, rows=(25536, 43968), iters=200, warmup=20, k_only=False):
    """q / k LayerNorm + 2-D RoPE in place on the packed ``qkv [P, 3, 16, 64]`` bf16 (one launch through the C ABI),
    over 4 rotating tensors (each launch touches 2/3 of 157 MB at P = 25 536).  Algorithmic bytes: q and k read and
    written once.  ``k_only``: the same launch with a null q (half the bytes), what remains of the pass when the q half
    is left to the attention kernel (``defer_q``)."""
    import torch
    from come_amd import _lib
    from come_amd.common import RotaryPositionEmbedding2D

    lib, stream = _lib.load(), _lib.current_stream(device)
    out = {}
    for P in rows:
        H = 16
        torch.manual_seed(3)
        sets = [torch.randn(P, 3, H, 64, device=device).bfloat16() for _ in range(4)]
        params = [torch.randn(64, device=device).bfloat16() for _ in range(4)]
        cos_t, sin_t = RotaryPositionEmbedding2D(100.0).tables(64, 38, device, torch.bfloat16)
        pos = torch.randint(0, 38, (P, 2), device=device)
        state = {"i": 0}

        def step():
            i = state["i"] = (state["i"] + 1) % 4
            q, k = sets[i][:, 0], sets[i][:, 1]
            _lib.check(lib.come_qk_norm_rope(None if k_only else q.data_ptr(), k.data_ptr(), _lib.COME_BF16, q.stride(0), q.stride(1),
                                             k.stride(0), k.stride(1), P, H, 64, 1, params[0].data_ptr(),
                                             params[1].data_ptr(), params[2].data_ptr(), params[3].data_ptr(), 1e-5,
                                             pos.data_ptr(), cos_t.data_ptr(), sin_t.data_ptr(), 38, stream))

        _, ms = time_loop(step, iters, warmup)
        nbytes = P * (1 if k_only else 2) * H * 64 * 2 * 2
        gbs = nbytes / (ms / iters * 1e-3) / 1e9
        out["P=%d" % P] = {"us_per_call": round(ms / iters * 1e3, 2), "algorithmic_bytes": nbytes, "GBs": round(gbs, 1),
                           "frac": round(gbs / PEAK_HBM_GBS, 4)}
        del sets
        torch.cuda.empty_cache()
    return out


def bench_frame_attention(device, w, only_mode=None):
    """Frame-mode attention of the headline workload's first sequence: 32 segments of about 798 tokens.
    ``only_mode``: time that scale mode alone (profiler runs)."""
    import torch

    counts = packed_counts(32, 144, 5, 73, 2304, torch.Generator().manual_seed(0))
    # a frame ends where its counts add up to its 5 + 73 + 144 * 9 source tokens
    ends = (counts.cumsum(0) % (5 + 73 + 144 * 9) == 0).nonzero().flatten() + 1
    lens = torch.diff(ends, prepend=torch.zeros(1, dtype=ends.dtype)).tolist()
    assert len(lens) == 32 and sum(lens) == counts.numel()
    # launches of 0.1 - 0.2 ms: the figure settles only after some tens of milliseconds under load (142 us with 10
    # warm-up launches, 119 us from about 200 on), hence the long warm-up
    if only_mode is not None:
        ms, tflops, flops = attention_case(device, lens, counts, steps=200, warmup=300, scale_mode=only_mode)
        return {"scale_mode": only_mode, "us_per_call": round(ms * 1e3, 1), "value": round(tflops, 1), "unit": "TFLOP/s",
                "algorithmic_flops": flops, "frac": round(tflops / PEAK_BF16_TFLOPS, 4)}
    ms, tflops, flops = attention_case(device, lens, counts, steps=200, warmup=300)
    ms_f, tflops_f, _ = attention_case(device, lens, counts, steps=200, warmup=100, scale_mode="folded")
    ms_q, tflops_q, _ = attention_case(device, lens, counts, steps=200, warmup=100, work_queue=True)
    return {"workload": "frame attention: 32 segments of %d..%d packed tokens (same tokens as the headline sequence 0)"
                        % (min(lens), max(lens)), "us_per_call": round(ms * 1e3, 1), "value": round(tflops, 1),
            "unit": "TFLOP/s", "algorithmic_flops": flops, "frac": round(tflops / PEAK_BF16_TFLOPS, 4),
            "folded_scale": {"us_per_call": round(ms_f * 1e3, 1), "value": round(tflops_f, 1),
                             "frac": round(tflops_f / PEAK_BF16_TFLOPS, 4)},
            # the opt-in launch of resident workgroups fed from a device-side work list (list kernel included)
            "work_queue": {"us_per_call": round(ms_q * 1e3, 1), "value": round(tflops_q, 1),
                           "frac": round(tflops_q / PEAK_BF16_TFLOPS, 4)}}


def bench_stress(device, frames_only_mode=None):
    """Long-sequence stress configuration at kernel level: 128 frames of 37x28 patches + 5 specials (133 248
    tokens), 3x3 merge at ratio 0.75 with per-frame jitter +-0.1.  ``frames_only_mode``: only the frame attention of
    that workload, in that scale mode (profiler runs)."""
    import torch

    w = merge_workload(device, ratio=0.75, sets=4, frames=128, H=37, W=28, jitter=0.1)   # 4 x 102 MB of packed rows
    for _ in range(4):
        w["merge_only"]()
    _, m_ms = time_loop(w["merge_only"], 50, 10)
    _, s_ms = time_loop(w["split_only"], 50, 10)
    offsets = w["offsets"].cpu().tolist()
    counts = w["counts"].cpu()
    frame_lens = [b - a for a, b in zip(offsets[:-1], offsets[1:])]
    res = {"workload": "stress: 128 frames 37x28+5 (133248 tokens), 3x3 merge r=0.75 +-0.1 per frame -> P=%d, "
                       "frame segments %d..%d" % (w["P"], min(frame_lens), max(frame_lens)),
           "merge_us": round(m_ms / 50 * 1e3, 1), "merge_bytes": w["merge_bytes"],
           "merge_GBs": round(w["merge_bytes"] / (m_ms / 50 * 1e-3) / 1e9, 1),
           "unmerge_us": round(s_ms / 50 * 1e3, 1), "unmerge_bytes": w["split_bytes"],
           "unmerge_GBs": round(w["split_bytes"] / (s_ms / 50 * 1e-3) / 1e9, 1), "rotating_buffer_sets": 4}
    P = w["P"]
    del w
    torch.cuda.empty_cache()
    if frames_only_mode is not None:
        ms, tflops, flops = attention_case(device, frame_lens, counts, steps=200, warmup=300, scale_mode=frames_only_mode)
        return {"workload": res["workload"], "scale_mode": frames_only_mode, "us_per_call": round(ms * 1e3, 1),
                "TFLOPs": round(tflops, 1), "algorithmic_flops": flops, "frac": round(tflops / PEAK_BF16_TFLOPS, 4)}
    ms, tflops, flops = attention_case(device, frame_lens, counts, steps=200, warmup=300)
    ms_f, tflops_f, _ = attention_case(device, frame_lens, counts, steps=200, warmup=100, scale_mode="folded")
    ms_q, tflops_q, _ = attention_case(device, frame_lens, counts, steps=200, warmup=100, work_queue=True)
    res["frame_attention"] = {"us_per_call": round(ms * 1e3, 1), "TFLOPs": round(tflops, 1), "algorithmic_flops": flops,
                              "frac": round(tflops / PEAK_BF16_TFLOPS, 4),
                              "folded_scale": {"us_per_call": round(ms_f * 1e3, 1), "TFLOPs": round(tflops_f, 1),
                                               "frac": round(tflops_f / PEAK_BF16_TFLOPS, 4)},
                              "work_queue": {"us_per_call": round(ms_q * 1e3, 1), "TFLOPs": round(tflops_q, 1),
                                             "frac": round(tflops_q / PEAK_BF16_TFLOPS, 4)}}
    ms, tflops, flops = attention_case(device, [P], counts, steps=5, warmup=2)
    res["global_attention"] = {"ms_per_call": round(ms, 3), "TFLOPs": round(tflops, 1), "algorithmic_flops": flops,
                               "frac": round(tflops / PEAK_BF16_TFLOPS, 4)}
    return res


def bench_scale_mode(device, mode, steps=10, warmup=3):
    """The headline workload with the way softmax_scale reaches the scores named explicitly: ``"exact"`` (in fp32 on
    every score, the reference's arithmetic and the default for a tensor without a known logit bound) or ``"folded"``
    (multiplied into a 16-bit q once: what tensors with a small ``come_qk_bound`` get)."""
    w, _, ms = bench_attention(steps, warmup, device, scale_mode=mode)
    tflops = w["flops"] / (ms / steps * 1e-3) / 1e12
    return {"ms_per_call": round(ms / steps, 4), "value": round(tflops, 1), "unit": "TFLOP/s",
            "frac": round(tflops / PEAK_BF16_TFLOPS, 4),
            "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tflops / PEAK_BF16_TFLOPS, 4),
                         "kernel": "attn_fwd_pipe_kernel<bf16, 8, %s>" % ("true" if mode == "exact" else "false")}}


def bench_deferred_q_prologue(device, steps=20, warmup=5):
    """The headline workload with the q half of the prologue (LayerNorm + 2-D rotary embedding) done by the attention
    kernel on the query fragments it loads (``prepare_packed_self_attention_qkv(..., defer_q=True)``), next to the
    two-step path on the same tensors: per layer call, full in-place pass + attention against k-only pass + attention
    with the prologue.  fp32 scale on every score in both."""
    import torch
    from come_amd.common import RotaryPositionEmbedding2D, prepare_packed_self_attention_qkv
    from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias

    w = make_attention_workload(device)
    P, max_len = w["qkv"].shape[0], max(w["lens"])
    norms = [torch.nn.LayerNorm(64, eps=1e-6).to(device=device, dtype=torch.bfloat16) for _ in range(2)]
    rope = RotaryPositionEmbedding2D(100.0)
    pos = torch.randint(0, 38, (P, 2), device=device)
    res = {}
    for name, defer in (("two_step", False), ("deferred_q", True)):
        # the pass rewrites q / k in place: every step works on a LayerNorm'd tensor again, which is what it would see
        qkv = w["qkv"].clone()

        def prologue():
            return prepare_packed_self_attention_qkv(qkv, norms[0], norms[1], rope, pos, torch.bfloat16, max_position=37,
                                                     defer_q=defer)

        def attention():
            return flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, w["cu"], max_len, perkey_bias=w["bias"],
                                                                  softmax_scale=0.125, scale_mode="exact")

        with torch.no_grad():
            prologue()
            _, ms_p = time_loop(prologue, 10 * steps, 10 * warmup)
            _, ms_a = time_loop(attention, steps, warmup)
        res[name] = {"prologue_us": round(ms_p / (10 * steps) * 1e3, 1), "attention_ms": round(ms_a / steps, 4),
                     "sum_ms": round(ms_p / (10 * steps) + ms_a / steps, 4)}
    res["saved_us_per_layer_call"] = round((res["two_step"]["sum_ms"] - res["deferred_q"]["sum_ms"]) * 1e3, 1)
    res["workload"] = "headline attention workload (P = 47384 packed rows, 16 heads x 64), q / k LayerNorm + 2-D RoPE"
    return res


def bench_other_widths(device, steps=20, warmup=40):
    """The biased varlen attention at the head dimensions beside 64 that have their own kernel instance (32 and 128):
    one segment of 16 384 tokens, 16 heads, bf16, bias log(count) on 30 % of the keys."""
    import torch
    from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias

    res = {}
    L, H = 16384, 16
    for D in (32, 128):
        g = torch.Generator(device="cpu").manual_seed(D)
        qkv = torch.randn(L, 3, H, D, generator=g).bfloat16().to(device)
        bias = torch.where(torch.rand(L, generator=g) < 0.3, math.log(9.0), 0.0).bfloat16().to(device)
        cu = torch.tensor([0, L], dtype=torch.int32, device=device)

        def step():
            return flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, L, perkey_bias=bias)

        _, ms = time_loop(step, steps, warmup)
        tflops = 4.0 * L * L * D * H / (ms / steps * 1e-3) / 1e12
        res[f"head_dim_{D}"] = {"ms_per_call": round(ms / steps, 4), "value": round(tflops, 1), "unit": "TFLOP/s",
                                "frac": round(tflops / PEAK_BF16_TFLOPS, 4)}
    res["workload"] = "1 segment x 16384 tokens, 16 heads, bf16, per-key bias"
    return res


def bench_gemm_reference(device):
    """Library bf16 GEMM (8192^3, N(0,1) operands, torch.matmul -> hipBLASLt) in the same run: what the matrix
    cores of this box sustain on data of the same kind, next to the nominal 2.5 PFLOP/s used for ``frac``."""
    import torch

    torch.manual_seed(0)
    a = torch.randn(8192, 8192, device=device).bfloat16()
    b = torch.randn(8192, 8192, device=device).bfloat16()
    _, ms = time_loop(lambda: a @ b, 20, 5)
    tflops = 2.0 * 8192 ** 3 / (ms / 20 * 1e-3) / 1e12
    return {"workload": "torch.matmul bf16 8192x8192x8192, N(0,1) operands", "value": round(tflops, 1), "unit": "TFLOP/s",
            "frac_of_nominal_peak": round(tflops / PEAK_BF16_TFLOPS, 4)}


def bench_e2e(device, frames=32, depth=24, reps=5, height=518, width=518, ratio=0.5):
    """End-to-end aggregator (random init, bf16): 24 frame + 24 global blocks, dim 1024, 16 heads x 64, MLP 4096,
    32 frames of 518x518; 3x3 merge from block 4 onward at ratio 0.5 against the same model without merging.
    (``frames=128, depth=36, width=392, ratio=0.75``: the long-sequence stress configuration, 133 248 tokens.)
    ``within_tolerance`` says whether the merged model stayed within the stated relative L1 of the unmerged one on
    the pixels of unmerged windows; the same check is an assertion in tests/test_gpu_e2e_full.py."""
    import torch
    from come_amd.harness import AggregatorConfig, AlternatingAggregator, deferred_q_prologue, relative_l1
    from come_amd.token_merger import CoMe_2D_TokenMerger

    torch.manual_seed(0)
    cfg = AggregatorConfig(depth=depth)
    model = AlternatingAggregator(cfg).eval().to(device=device, dtype=torch.bfloat16)
    images = torch.rand(1, frames, 3, height, width, generator=torch.Generator().manual_seed(0)).to(device)
    merger = CoMe_2D_TokenMerger(cfg.specials, 3, 3, ratio, allow_remainder=True)
    gh, gw = height // 14, width // 14

    def timed(m, prologue=None):
        out = model(images, merger=m, prologue=prologue)        # warm-up (allocator, GEMM heuristics)
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            out = model(images, merger=m, prologue=prologue)
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
        return out, sorted(times)[len(times) // 2]

    dense, dense_ms = timed(None)
    merged, merged_ms = timed(merger)
    # the same forward with the q half of every attention prologue left to the attention kernel: the same bits
    fused, fused_ms = timed(merger, deferred_q_prologue)
    mh, mw = gh // 3, gw // 3
    mask = merged["merge_mask"].reshape(frames, mh, mw)
    keep = torch.ones(frames, gh, gw, dtype=torch.bool, device=device)
    keep[:, :mh * 3, :mw * 3] = ~mask.repeat_interleave(3, 1).repeat_interleave(3, 2)
    keep_px = keep.repeat_interleave(14, 1).repeat_interleave(14, 2)[None, :, None]
    rel = relative_l1(merged["maps"], dense["maps"], keep_px)
    return {"workload": f"VGGT-style aggregator, random init, bf16: {depth} frame + {depth} global blocks, dim 1024, "
                        f"16 heads x 64, MLP 4096, S={frames} frames {height}x{width} ({dense['tokens_dense']} tokens); "
                        f"3x3 merge from block {cfg.merge_block} at r={ratio} ({merged['tokens_packed']} packed tokens)",
            "merged_ms": round(merged_ms, 2), "unmerged_ms": round(dense_ms, 2),
            "speedup": round(dense_ms / merged_ms, 3), "reps": reps, "statistic": "median wall time per forward",
            "merged_deferred_q_prologue_ms": round(fused_ms, 2),
            "deferred_q_prologue_same_bits": bool(torch.equal(fused["maps"], merged["maps"])),
            "rel_l1_unmerged_windows": round(rel, 5), "rel_l1_tolerance": 5e-2, "within_tolerance": bool(rel <= 5e-2),
            "finite": bool(torch.isfinite(merged["maps"]).all())}


# ------------------------------------------------------------------------------------------
# host-CPU baseline (the reference's PyTorch path on the CPU), bounded sample
# ------------------------------------------------------------------------------------------

def cpu_baseline_attention(w, min_s=10.0, budget_s=20.0, q_chunk=4096):
    """The reference's PyTorch CPU path for this operator (per segment, SDPA in bf16 with the bias as
    attn_mask, queries in chunks of ``q_chunk``) over the same workload, repeated until ``min_s`` seconds are
    sampled and stopped after ``budget_s``.  Same flop formula as the GPU figure (4 * rows * L * d * H per chunk)."""
    import torch
    import oracle

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    qkv, bias = w["qkv"].cpu(), w["bias"].cpu()
    bounds = [0, w["lens"][0], w["lens"][0] + w["lens"][1]]
    flops, spent, rows, passes = 0.0, 0.0, 0, 0
    while spent < min_s:                                       # whole passes until enough time is sampled
        for s, e in zip(bounds[:-1], bounds[1:]):
            for c0 in range(s, e, q_chunk):
                if spent >= budget_s:
                    break
                c1 = min(e, c0 + q_chunk)
                t0 = time.perf_counter()
                oracle.sdpa_bf16_chunk(qkv, bias, s, e, c0, c1, 0.125)
                spent += time.perf_counter() - t0
                flops += 4.0 * (c1 - c0) * (e - s) * w["D"] * w["H"]
                rows += c1 - c0
        passes += 1
    total_rows = bounds[-1]
    return {"value": round(flops / spent / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"torch CPU SDPA bf16 + attn_mask bias on the same workload, {rows} query rows of "
                      f"{total_rows} per pass ({passes} passes; all keys of their segment, 16 heads) in {spent:.1f} s, "
                      f"chunks of {q_chunk} queries"}


def cpu_baseline_merge(mw):
    import torch
    import oracle

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    tokens = mw["tokens"][0].cpu()
    conf = mw["conf"].cpu()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        mask = oracle.select_lowest_confidence(conf, 1, 3, 3, mw["ratio"])
        jag, rev = oracle.token_merge_2d(tokens, 5, 3, 3, 37, 37, mask, allow_remainder=True)
        times.append(time.perf_counter() - t0)
    t_merge = sorted(times)[1]
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        oracle.token_split(jag, rev, (1, mw["frames"], mw["N"], mw["C"]))
        times.append(time.perf_counter() - t0)
    t_split = sorted(times)[1]
    return {"merge_GBs": round(mw["merge_bytes"] / t_merge / 1e9, 3), "unmerge_GBs": round(mw["split_bytes"] / t_split / 1e9, 3),
            "cores": threads, "kind": "port",
            "sample": f"oracle select+merge ({t_merge * 1e3:.0f} ms) and split ({t_split * 1e3:.0f} ms) of the full C2 "
                      "workload on the CPU in bf16, median of 3"}


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "multi-GPU sharding is a design note, not code. Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from come_amd import _lib

    _lib.load()                                                  # fails loudly when the HIP library is missing
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.only:
        if args.only == "stress":
            print(json.dumps({"only": "stress", **bench_stress(device)}))
        elif args.only == "frame":
            print(json.dumps({"only": "frame", **bench_frame_attention(
                device, None, None if args.scale_mode == "auto" else args.scale_mode)}))
        elif args.only == "stress_frames":
            print(json.dumps({"only": "stress_frames", **bench_stress(
                device, "exact" if args.scale_mode == "auto" else args.scale_mode)}))
        elif args.only == "e2e":
            print(json.dumps({"only": "e2e", **bench_e2e(device, reps=max(1, args.steps))}))
        elif args.only == "stress_e2e":                          # seconds per forward: not part of the default run
            print(json.dumps({"only": "stress_e2e", **bench_e2e(device, frames=128, depth=36, width=392, ratio=0.75,
                                                                  reps=max(1, min(args.steps, 3)))}))
        elif args.only == "copy":
            # plain device copy of known size: the yardstick the HBM byte counters are scaled by
            nbytes = 256 << 20
            src = torch.empty(nbytes, dtype=torch.uint8, device=device).random_(0, 255)
            dst = torch.empty_like(src)
            _, ms = time_loop(lambda: dst.copy_(src), args.steps, args.warmup)
            print(json.dumps({"only": "copy", "bytes_read": nbytes, "bytes_written": nbytes,
                              "us_per_call": ms / args.steps * 1e3,
                              "GBs": 2 * nbytes / (ms / args.steps * 1e-3) / 1e9}))
        elif args.only == "attn":
            w, wall, ev_ms = bench_attention(args.steps, args.warmup, device)
            print(json.dumps({"only": "attn", "ms_per_call": ev_ms / args.steps,
                              "tflops": w["flops"] / (ev_ms / args.steps * 1e-3) / 1e12}))
        elif args.only in ("exact", "folded"):
            print(json.dumps({"only": args.only, **bench_scale_mode(device, args.only, args.steps, args.warmup)}))
        elif args.only == "widths":
            print(json.dumps({"only": "widths", **bench_other_widths(device, args.steps, args.warmup)}))
        elif args.only == "prologue":
            print(json.dumps({"only": "prologue", **bench_qk_prologue(device, iters=args.steps, warmup=args.warmup)}))
        elif args.only == "prologue_k":
            print(json.dumps({"only": "prologue_k", **bench_qk_prologue(device, iters=args.steps, warmup=args.warmup, k_only=True),
                              "q_half_in_attention": bench_deferred_q_prologue(device)}))
        elif args.only == "refmerge":
            print(json.dumps({"only": "refmerge", **bench_reference_merge_shapes(device)}))
        elif args.only == "bias":
            print(json.dumps({"only": "bias", **bench_bias_overhead(device)}))
        elif args.only == "dtypes":
            print(json.dumps({"only": "dtypes", **bench_merge_caller_dtypes(device, args.steps, args.warmup)}))
        elif args.only == "pair":
            mw = merge_workload(device)
            for _ in range(len(mw["outs"])):
                mw["merge_only"]()
            print(json.dumps({"only": "pair", **bench_unmerge_pair(device, mw, args.steps, args.warmup)}))
        elif args.only == "select":
            mw = merge_workload(device)
            _, ms = time_loop(mw["select_and_plan"], args.steps, args.warmup)
            print(json.dumps({"only": "select", "us_per_call": ms / args.steps * 1e3}))
        else:
            mw = merge_workload(device)
            for _ in range(len(mw["outs"])):
                mw["merge_only"]()
            fn = mw["merge_only"] if args.only == "merge" else mw["split_only"]
            _, ms = time_loop(fn, args.steps, args.warmup)
            nbytes = mw["merge_bytes"] if args.only == "merge" else mw["split_bytes"]
            print(json.dumps({"only": args.only, "us_per_call": ms / args.steps * 1e3,
                              "GBs": nbytes / (ms / args.steps * 1e-3) / 1e9}))
        return

    w, wall, ev_ms = bench_attention(args.steps, args.warmup, device)
    ms_per_step = wall / args.steps * 1e3
    value = w["flops"] / (wall / args.steps) / 1e12
    kernel_tflops = w["flops"] / (ev_ms / args.steps * 1e-3) / 1e12

    result = {
        "metric": "biased-attn TFLOP/s",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "C3 biased varlen flash-attention fwd: 16 heads x 64, packed L = {25536, 21848} "
                               "(32 frames 37x37 after 3x3 merge at r = 0.5 / 0.6), bias = log(count in {1,9}), "
                               "scale 0.125, non-causal",
                   "algorithmic_flops_per_step": w["flops"]},
        "roofline": {"bound": "mfma", "achieved": round(kernel_tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(kernel_tflops / PEAK_BF16_TFLOPS, 4), "traffic": TRAFFIC_BYTES["attn"],
                     "traffic_source": TRAFFIC["attn"]["source"],
                     "kernel": "attn_fwd_pipe_kernel<bf16, 8, true>", "scale_mode": "auto -> exact (fp32 scale on every score)",
                     "ms_per_launch": round(ev_ms / args.steps, 4)},
    }
    mw = None
    if not args.no_other:
        mw, other = bench_merge_unmerge(device)
        result["other"] = other
        other["merge"]["operator"] = bench_merge_operator(device, mw)
        other["unmerge"]["write_floor"] = bench_write_floor(device, mw["frames"] * mw["N"] * mw["C"] * 2)
        other["unmerge_pair"] = bench_unmerge_pair(device, mw)
        other["library_gemm_reference"] = bench_gemm_reference(device)
        other["merge_other_ratios"] = bench_merge_ratios(device)
        other["merge_caller_dtypes"] = bench_merge_caller_dtypes(device)
        other["reference_merge_microbench_shapes"] = bench_reference_merge_shapes(device)
        other["qk_prologue"] = bench_qk_prologue(device)
        other["qk_prologue"]["k_only"] = bench_qk_prologue(device, k_only=True)
        other["qk_prologue"]["q_half_in_attention"] = bench_deferred_q_prologue(device)
        other["frame_attention"] = bench_frame_attention(device, w)
        other["bias_overhead"] = bench_bias_overhead(device)
        other["attention_exact_scale"] = bench_scale_mode(device, "exact")
        other["attention_folded_scale"] = bench_scale_mode(device, "folded")
        other["attention_other_widths"] = bench_other_widths(device)
        other["stress"] = bench_stress(device)
    if not args.no_e2e:
        result.setdefault("other", {})["e2e"] = bench_e2e(device)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_attention(w)
        if mw is not None:
            result["other"]["cpu_baseline"] = cpu_baseline_merge(mw)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
