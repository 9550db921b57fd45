"""TEST INFRASTRUCTURE ONLY — loop-level fp64 evaluation of the textbook definitions, for tiny inputs.

Independent of oracle/mops_torch.py on purpose (no shared helper, no matmul, no library softmax): it is
what pins that file's attention functions, so a dropped scale, a wrong head map, an off-by-one in the
causal rule or a transposed operand there fails against these loops.
"""
from __future__ import annotations

import math

import numpy as np


def attention_row(q_row: np.ndarray, keys: np.ndarray, values: np.ndarray, scale: float) -> np.ndarray:
    """softmax(scale * q . k_j) weighted sum of v_j, one query row, fp64. keys/values: [L, D]."""
    L, D = keys.shape
    logits = [scale * sum(float(q_row[d]) * float(keys[j, d]) for d in range(D)) for j in range(L)]
    mx = max(logits)
    w = [math.exp(x - mx) for x in logits]
    z = sum(w)
    out = np.zeros(D, dtype=np.float64)
    for j in range(L):
        for d in range(D):
            out[d] += (w[j] / z) * float(values[j, d])
    return out


def varlen_causal(q: np.ndarray, k: np.ndarray, v: np.ndarray, cu_seqlens, scale: float) -> np.ndarray:
    """q [T,Hq,D], k/v [T,Hkv,D]; query i of a sequence sees keys 0..i of the same sequence; query head h
    uses kv head h // (Hq // Hkv)."""
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    rep = Hq // Hkv
    out = np.zeros((T, Hq, D), dtype=np.float64)
    for s in range(len(cu_seqlens) - 1):
        lo, hi = int(cu_seqlens[s]), int(cu_seqlens[s + 1])
        for i in range(lo, hi):
            for h in range(Hq):
                g = h // rep
                out[i, h] = attention_row(q[i, h], k[lo:i + 1, g], v[lo:i + 1, g], scale)
    return out


def varlen_causal_prefix(q: np.ndarray, k: np.ndarray, v: np.ndarray, cu_q, cu_k, scale: float) -> np.ndarray:
    """As varlen_causal, but sequence s has Lk >= Lq keys (k/v packed by cu_k): its query i, counted from
    the first NEW token, sits at absolute position i + (Lk - Lq) and sees the keys at positions <= that."""
    T, Hq, D = q.shape
    rep = Hq // k.shape[1]
    out = np.zeros((T, Hq, D), dtype=np.float64)
    for s in range(len(cu_q) - 1):
        q_lo, q_hi, k_lo, k_hi = int(cu_q[s]), int(cu_q[s + 1]), int(cu_k[s]), int(cu_k[s + 1])
        first_new = (k_hi - k_lo) - (q_hi - q_lo)
        for i in range(q_hi - q_lo):
            last_visible = first_new + i
            for h in range(Hq):
                out[q_lo + i, h] = attention_row(q[q_lo + i, h], k[k_lo:k_lo + last_visible + 1, h // rep],
                                                 v[k_lo:k_lo + last_visible + 1, h // rep], scale)
    return out


def paged_decode(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, cache_seqlens, block_table,
                 scale: float) -> np.ndarray:
    """q [B,Hq,D]; caches [NB,BS,Hkv,D]; token t of sequence b is cache[block_table[b][t // BS], t % BS]."""
    B, Hq, D = q.shape
    BS, Hkv = k_cache.shape[1], k_cache.shape[2]
    rep = Hq // Hkv
    out = np.zeros((B, Hq, D), dtype=np.float64)
    for b in range(B):
        n = int(cache_seqlens[b])
        if n == 0:
            continue
        for h in range(Hq):
            g = h // rep
            keys = np.stack([k_cache[int(block_table[b][t // BS]), t % BS, g] for t in range(n)])
            vals = np.stack([v_cache[int(block_table[b][t // BS]), t % BS, g] for t in range(n)])
            out[b, h] = attention_row(q[b, h], keys, vals, scale)
    return out


def rms(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """x * w / sqrt(mean(x^2) + eps) in fp64 with no intermediate rounding."""
    x = x.astype(np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w.astype(np.float64)
