"""TEST INFRASTRUCTURE ONLY — the parity oracle: a CPU-capable restatement of the reference's `torch`
backend for the six hot operators, registered under the backend name "torch" of the build's registry so
that tests read `get_op(name, "torch")` against `get_op(name, "hip")`.

Why a restatement: the reference's torch backend cannot run without a GPU and two absent packages — its
store_kvcache is a Triton kernel (mops/torch/ops.py:62-65 -> mops/triton/attention.py:7-38) and both
attention ops call the un-vendored, unpinned `flash-attn` library (mops/torch/ops.py:68-76).  The
reference ships no tests, golden vectors or fixtures for any of these ops.

What pins each function (all in tests/test_oracle.py, none of it a retyped copy of the formula below):
  rms_forward / add_rms_forward  fp64 closed form within 1 bf16 ulp; constant row and zero row special
                                 cases; add with zero residual reduces to rms_forward; residual output
                                 equals the bf16 sum.
  embedding                      equality with torch.nn.functional.embedding and with W[ids].
  store_kvcache                  equality with Tensor.index_copy_ on the flattened cache; sentinel slots
                                 untouched; -1 slots skipped; strided V source.
  flash_attn_varlen_func         fp64 loop-level brute force on tiny inputs (oracle/bruteforce.py);
                                 torch.nn.functional.scaled_dot_product_attention(is_causal=True) per
                                 sequence; L=1 -> o=v; constant V -> o=V.
  flash_attn_with_kvcache        fp64 brute force; equals the last row of causal prefill over the same
                                 K/V; invariant under a joint permutation of cache blocks and block_table;
                                 NaN sentinels beyond cache_seqlens do not reach the output.
  apply_rotary_emb               complex multiplication in fp64; identity at angle 0 and the quarter turn
                                 (x1, x2) -> (-x2, x1), both bit for bit; pair-norm preservation; R(t)R(-t) = I.
  siluAndMul                     fp64 x / (1 + e^-x) with the two bf16 roundings; the single-rounding variant differs.
  sampler_forward                brute-force first-maximum loop, with ties, the last column and an all-equal row.
  qk_norm_rope_store             fp64 loops on a tiny input with norm weights that vary along the head, so that
                                 rotary-before-norm fails; raw v and rotated k in their slots; slot -1 skipped.
The rounding internal to flash-attn itself (P cast to bf16 before PV, exp2 softmax) is pinned by no file
available here: attention parity is therefore stated with the tolerance max-abs 2e-2 / mean-abs 2e-3.
"""
from __future__ import annotations

import math

import torch

from nano_vllm_ninetoothed_amd.mops.registry import _BACKEND_REGISTRY, register_op

register_torch_op = register_op("torch")


def _fresh(func):
    """Registers func under "torch", replacing an earlier registration (module reloads in tests)."""
    _BACKEND_REGISTRY["torch"].pop(func.__name__, None)
    return register_torch_op(func)


@_fresh
def rms_forward(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """mops/torch/ops.py:9-16 — fp32 statistics, round to the input dtype, then multiply by the weight
    in the input dtype (second rounding)."""
    xf = x.to(torch.float32)
    mean_sq = (xf * xf).mean(dim=-1, keepdim=True)
    normed = (xf * torch.rsqrt(mean_sq + eps)).to(x.dtype)
    return normed * weight


@_fresh
def add_rms_forward(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """mops/torch/ops.py:18-30 — the sum is formed in fp32; the returned residual is that sum rounded,
    the normalisation uses the unrounded sum."""
    s = x.to(torch.float32) + residual.to(torch.float32)
    new_residual = s.to(x.dtype)
    mean_sq = (s * s).mean(dim=-1, keepdim=True)
    normed = (s * torch.rsqrt(mean_sq + eps)).to(x.dtype)
    return normed * weight, new_residual


@_fresh
def embedding(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """mops/torch/ops.py:57-59."""
    return weight[x.long()]


@_fresh
def store_kvcache(key, value, k_cache, v_cache, slot_mapping) -> None:
    """mops/triton/attention.py:18-38 — row i of key/value goes to flat cache row slot_mapping[i];
    slot -1 is skipped; caches are mutated in place."""
    n, heads, dim = key.shape
    row = heads * dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == dim and value.stride(1) == dim
    assert k_cache.stride(1) == row and v_cache.stride(1) == row
    assert slot_mapping.numel() == n
    slots = slot_mapping.long()
    keep = slots != -1
    kflat = k_cache.view(-1, row)
    vflat = v_cache.view(-1, row)
    kflat[slots[keep]] = key.reshape(n, row)[keep]
    vflat[slots[keep]] = value.reshape(n, row)[keep]


def _attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, causal_offset: int | None):
    """softmax(scale * q k^T + mask) v in fp32 for one sequence.  q [Lq, Hq, D], k/v [Lk, Hkv, D];
    query head h reads kv head h // (Hq // Hkv) (mops/triton/attention.py:117-119).  With
    causal_offset = Lk - Lq, key j is visible to query i iff j <= i + causal_offset."""
    lq, hq, _ = q.shape
    lk, hkv, _ = k.shape
    rep = hq // hkv
    qf = q.to(torch.float32).transpose(0, 1)                                  # [Hq, Lq, D]
    kf = k.to(torch.float32).transpose(0, 1).repeat_interleave(rep, dim=0)    # [Hq, Lk, D]
    vf = v.to(torch.float32).transpose(0, 1).repeat_interleave(rep, dim=0)
    scores = torch.matmul(qf, kf.transpose(1, 2)) * scale
    if causal_offset is not None:
        i = torch.arange(lq, device=q.device).unsqueeze(1)
        j = torch.arange(lk, device=q.device).unsqueeze(0)
        scores = scores.masked_fill(j > i + causal_offset, float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    return torch.matmul(probs, vf).transpose(0, 1)                            # [Lq, Hq, D] fp32


@_fresh
def flash_attn_varlen_func(q, k, v, max_seqlen_q=None, cu_seqlens_q=None, max_seqlen_k=None, cu_seqlens_k=None,
                           softmax_scale=None, causal=True, block_table=None, **kwargs):
    """Packed causal attention, semantics of flash_attn.flash_attn_varlen_func as used at
    nanovllm/layers/attention.py:34-37 and restated by mops/triton/attention.py:59-102,110-146.  When a
    sequence has more keys than queries (cached prefix), the causal mask is aligned to the bottom right:
    query i sees keys 0 .. i + (Lk - Lq)."""
    if cu_seqlens_k is None:
        cu_seqlens_k = cu_seqlens_q
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(q.shape[-1])
    out = torch.zeros_like(q)
    cq = cu_seqlens_q.tolist()
    ck = cu_seqlens_k.tolist()
    for s in range(len(cq) - 1):
        qs = q[cq[s]:cq[s + 1]]
        n_k = ck[s + 1] - ck[s]
        if qs.shape[0] == 0 or n_k <= 0:
            continue
        if block_table is None:
            ks, vs = k[ck[s]:ck[s + 1]], v[ck[s]:ck[s + 1]]
        else:   # k, v are the paged caches (nanovllm/layers/attention.py:32-33): gather this sequence's keys
            bs = k.shape[1]
            nblk = (n_k + bs - 1) // bs
            blocks = block_table[s, :nblk].long()
            ks = k[blocks].reshape(nblk * bs, *k.shape[2:])[:n_k]
            vs = v[blocks].reshape(nblk * bs, *v.shape[2:])[:n_k]
        off = (ks.shape[0] - qs.shape[0]) if causal else None
        out[cq[s]:cq[s + 1]] = _attend(qs, ks, vs, scale, off).to(q.dtype)
    return out


@_fresh
def flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=None, block_table=None, softmax_scale=None,
                            causal=True, **kwargs):
    """One query token per sequence against the paged cache: token t of sequence b lives at
    cache[block_table[b, t // BS], t % BS] (mops/torch/ops.py:96-99); q [B, 1, Hq, D] -> [B, 1, Hq, D]."""
    bsz, one, hq, d = q.shape
    assert one == 1
    bs = k_cache.shape[1]
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    out = torch.zeros_like(q)
    lens = cache_seqlens.tolist()
    for b in range(bsz):
        n = lens[b]
        if n <= 0:
            continue
        nblk = (n + bs - 1) // bs
        blocks = block_table[b, :nblk].long()
        kb = k_cache[blocks].reshape(nblk * bs, *k_cache.shape[2:])[:n]
        vb = v_cache[blocks].reshape(nblk * bs, *v_cache.shape[2:])[:n]
        out[b] = _attend(q[b], kb, vb, scale, None).to(q.dtype)
    return out


# Non-hot names, so that a whole decoder-layer sequence can be replayed on the oracle backend.

@_fresh
def linear(x, weight, bias=None):
    return torch.nn.functional.linear(x, weight, bias)


@_fresh
def siluAndMul(x, y):
    return torch.nn.functional.silu(x) * y


@_fresh
def sampler_forward(logits, temperatures):
    return torch.argmax(torch.softmax(logits.float() / temperatures.unsqueeze(1), dim=-1), dim=-1)


@_fresh
def apply_rotary_emb(x, cos, sin):
    x1, x2 = torch.chunk(x.float(), 2, dim=-1)
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).to(x.dtype)


@_fresh
def qk_norm_rope_store(qkv, q_weight, k_weight, eps, cos, sin, k_cache, v_cache, slot_mapping, num_heads, num_kv_heads,
                       need_k=True):
    """The hip backend's extension op, restated as the sequence it fuses: q_norm, k_norm, rotary embedding
    of q and k, store_kvcache (nanovllm/models/qwen3.py:74-80, nanovllm/layers/attention.py:29-31)."""
    d = q_weight.numel()
    q, k, v = qkv.split([num_heads * d, num_kv_heads * d, num_kv_heads * d], dim=-1)
    q = rms_forward(q.reshape(-1, num_heads, d), q_weight, eps)
    k = rms_forward(k.reshape(-1, num_kv_heads, d), k_weight, eps)
    v = v.reshape(-1, num_kv_heads, d)
    q = apply_rotary_emb(q, cos, sin)
    k = apply_rotary_emb(k, cos, sin)
    store_kvcache(k, v, k_cache, v_cache, slot_mapping)
    return q, (k if need_k else None), v
