"""Independent pure-Python restatements used to pin the oracle on tiny inputs.

They share no code with ``oracle/``: plain loops over frames, groups and
tokens, float64 arithmetic, Python lists for the layout.
"""

import math

import numpy as np


def merge_1d_loops(tokens, start_index, G, mask, tail=0):
    """tokens: np [B,N,C] float64, mask: np [B,M] bool -> (out [P,C], offset, rev, weight)."""
    B, N, C = tokens.shape
    M = mask.shape[1]
    out, weight, rev, offset = [], [], [], [0]
    for b in range(B):
        for s in range(start_index):
            rev.append(len(out)); out.append(tokens[b, s].copy()); weight.append(1.0)
        for m in range(M):
            src = [start_index + m * G + g for g in range(G)]
            if mask[b, m]:
                acc = np.zeros(C)
                for n in src:
                    acc += tokens[b, n]
                    rev.append(len(out))
                out.append(acc / G); weight.append(float(G))
            else:
                for n in src:
                    rev.append(len(out)); out.append(tokens[b, n].copy()); weight.append(1.0)
        for t in range(tail):
            rev.append(len(out)); out.append(tokens[b, start_index + M * G + t].copy()); weight.append(1.0)
        offset.append(len(out))
    return np.array(out).reshape(len(out), C), np.array(offset), np.array(rev), np.array(weight)


def merge_2d_loops(tokens, start_index, gh, gw, H, W, mask):
    """2-D windows incl. remainder positions; rev is reported in image row-major order."""
    B, N, C = tokens.shape
    mh, mw = H // gh, W // gw
    out, weight, offset = [], [], [0]
    rev = np.full((B, N), -1, dtype=np.int64)
    for b in range(B):
        for s in range(start_index):
            rev[b, s] = len(out); out.append(tokens[b, s].copy()); weight.append(1.0)
        for wy in range(mh):
            for wx in range(mw):
                members = [start_index + (wy * gh + dy) * W + (wx * gw + dx) for dy in range(gh) for dx in range(gw)]
                if mask[b, wy * mw + wx]:
                    row = len(out)
                    out.append(sum(tokens[b, n] for n in members) / (gh * gw)); weight.append(float(gh * gw))
                    for n in members:
                        rev[b, n] = row
                else:
                    for n in members:
                        rev[b, n] = len(out); out.append(tokens[b, n].copy()); weight.append(1.0)
        for y in range(H):
            for x in range(W):
                if y >= mh * gh or x >= mw * gw:
                    n = start_index + y * W + x
                    rev[b, n] = len(out); out.append(tokens[b, n].copy()); weight.append(1.0)
        offset.append(len(out))
    assert (rev >= 0).all()
    return np.array(out).reshape(len(out), C), np.array(offset), rev.reshape(-1), np.array(weight)


def attention_loops(q, k, v, bias, scale):
    """One segment, one head; q,k,v: np [L,D] float64; bias [L]."""
    L, D = q.shape
    out = np.zeros((L, D))
    lse = np.zeros(L)
    for i in range(L):
        s = [scale * float(np.dot(q[i], k[j])) + float(bias[j]) for j in range(L)]
        m = max(s)
        e = [math.exp(x - m) for x in s]
        z = sum(e)
        lse[i] = m + math.log(z)
        for j in range(L):
            out[i] += (e[j] / z) * v[j]
    return out, lse


def zscore_window_means_loops(conf, batch, gh, gw):
    """Normalised-score window means by plain loops in float64.

    conf: np [batch * frames, H, W].  Per batch element: mean over all of its positions, standard
    deviation with the n - 1 divisor, z = (x - mean) / (std + 1e-3); then the mean of z over every
    full gh x gw window (block-row-major).  Returns np [batch * frames, M].
    """
    F, H, W = conf.shape
    frames = F // batch
    mh, mw = H // gh, W // gw
    out = np.zeros((F, mh * mw))
    for b in range(batch):
        vals = [float(conf[b * frames + f, y, x]) for f in range(frames) for y in range(H) for x in range(W)]
        n = len(vals)
        mean = sum(vals) / n
        var = sum((v - mean) * (v - mean) for v in vals) / (n - 1)
        denom = math.sqrt(var) + 1e-3
        for f in range(frames):
            for wy in range(mh):
                for wx in range(mw):
                    acc = 0.0
                    for dy in range(gh):
                        for dx in range(gw):
                            acc += (float(conf[b * frames + f, wy * gh + dy, wx * gw + dx]) - mean) / denom
                    out[b * frames + f, wy * mw + wx] = acc / (gh * gw)
    return out
