"""Seeded synthetic inputs for the benchmark configurations (shapes of Qwen3-0.6B / Qwen3-8B attention).

Everything is drawn on the CPU from one torch.Generator in fp32 and cast to bf16, so a CPU checker and
the GPU kernels see identical bits; metadata is int32.  Builders return plain dicts of CPU tensors;
`to_device` moves a dict to the GPU.
"""
from __future__ import annotations

import torch

BLOCK_SIZE = 256
HEAD_DIM = 128


def _gen(seed: int) -> torch.Generator:
    return torch.Generator("cpu").manual_seed(seed)


def _normal(g, shape, std=1.0, mean=0.0):
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std + mean).to(torch.bfloat16)


def to_device(d: dict, device="cuda") -> dict:
    return {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in d.items()}


def rms_inputs(rows: int, hidden: int, seed: int = 0, with_residual: bool = False) -> dict:
    g = _gen(seed)
    d = {"x": _normal(g, (rows, hidden)), "weight": _normal(g, (hidden,), std=0.1, mean=1.0), "eps": 1e-6}
    if with_residual:
        d["residual"] = _normal(g, (rows, hidden))
    return d


def embedding_inputs(n_ids: int, vocab: int, hidden: int, seed: int = 0, id_dtype=torch.int32) -> dict:
    g = _gen(seed)
    weight = torch.empty((vocab, hidden), dtype=torch.bfloat16)
    step = 8192  # draw the table in slabs: fp32 staging of a 151936 x 4096 table would need 2.5 GB
    for r in range(0, vocab, step):
        weight[r:r + step] = _normal(g, (min(step, vocab - r), hidden), std=0.02)
    ids = torch.randint(0, vocab, (n_ids,), generator=g, dtype=torch.int64).to(id_dtype)
    return {"ids": ids, "weight": weight}


def store_inputs(n_tokens: int, hkv: int = 8, num_blocks: int | None = None, seed: int = 0,
                 v_row_stride: int | None = None) -> dict:
    """K/V rows plus a random-permutation slot_mapping into num_blocks x 256 slots.  With v_row_stride
    the V tensor is a strided view into a wider buffer (as nanovllm hands it: a slice of the qkv
    projection output)."""
    g = _gen(seed)
    if num_blocks is None:
        num_blocks = (n_tokens + BLOCK_SIZE - 1) // BLOCK_SIZE + 2
    key = _normal(g, (n_tokens, hkv, HEAD_DIM))
    if v_row_stride is None:
        value = _normal(g, (n_tokens, hkv, HEAD_DIM))
    else:
        wide = _normal(g, (n_tokens, v_row_stride))
        value = wide[:, v_row_stride - hkv * HEAD_DIM:].view(n_tokens, hkv, HEAD_DIM)
    slots = torch.randperm(num_blocks * BLOCK_SIZE, generator=g)[:n_tokens].to(torch.int32)
    return {"key": key, "value": value, "slot_mapping": slots, "num_blocks": num_blocks, "hkv": hkv}


def prefill_inputs(seq_lens, hq: int = 16, hkv: int = 8, seed: int = 0) -> dict:
    g = _gen(seed)
    lens = torch.as_tensor(seq_lens, dtype=torch.int64)
    total = int(lens.sum())
    cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0).to(torch.int32)
    return {
        "q": _normal(g, (total, hq, HEAD_DIM)),
        "k": _normal(g, (total, hkv, HEAD_DIM)),
        "v": _normal(g, (total, hkv, HEAD_DIM)),
        "cu_seqlens": cu,
        "max_seqlen": int(lens.max()) if len(lens) else 0,
        "scale": HEAD_DIM ** -0.5,
        "seq_lens": [int(x) for x in lens],
    }


def prefix_prefill_inputs(new_lens, prefix_lens, hq: int = 16, hkv: int = 8, seed: int = 0, poison_unused: bool = True) -> dict:
    """Prefill with a cached prefix (the prefix-cache hit path): sequence s has prefix_lens[s] tokens already
    in the paged cache followed by new_lens[s] new ones whose K/V have just been stored there too; q holds
    only the new tokens.  Returns the paged caches, block_table, cu_seqlens_q/k and, for checking, the
    packed K/V of every sequence."""
    g = _gen(seed)
    new = torch.as_tensor(new_lens, dtype=torch.int64)
    tot = new + torch.as_tensor(prefix_lens, dtype=torch.int64)
    bsz = len(new)
    blocks_per_seq = (tot + BLOCK_SIZE - 1) // BLOCK_SIZE
    nblk = int(blocks_per_seq.sum()) + 2
    max_blocks = max(int(blocks_per_seq.max()), 1)
    perm = torch.randperm(nblk, generator=g).to(torch.int32)
    table = torch.full((bsz, max_blocks), -1, dtype=torch.int32)
    fill = float("nan") if poison_unused else 0.0
    k_cache = torch.full((nblk, BLOCK_SIZE, hkv, HEAD_DIM), fill, dtype=torch.bfloat16)
    v_cache = torch.full((nblk, BLOCK_SIZE, hkv, HEAD_DIM), fill, dtype=torch.bfloat16)
    k_all = _normal(g, (int(tot.sum()), hkv, HEAD_DIM))
    v_all = _normal(g, (int(tot.sum()), hkv, HEAD_DIM))
    cu_q = torch.zeros(bsz + 1, dtype=torch.int32)
    cu_k = torch.zeros(bsz + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(new, 0).to(torch.int32)
    cu_k[1:] = torch.cumsum(tot, 0).to(torch.int32)
    pos = 0
    for b in range(bsz):
        nb = int(blocks_per_seq[b])
        table[b, :nb] = perm[pos:pos + nb]
        pos += nb
        lo = int(cu_k[b])
        for i in range(nb):
            n = min(BLOCK_SIZE, int(tot[b]) - i * BLOCK_SIZE)
            k_cache[int(table[b, i]), :n] = k_all[lo + i * BLOCK_SIZE: lo + i * BLOCK_SIZE + n]
            v_cache[int(table[b, i]), :n] = v_all[lo + i * BLOCK_SIZE: lo + i * BLOCK_SIZE + n]
    return {"q": _normal(g, (int(new.sum()), hq, HEAD_DIM)), "k_cache": k_cache, "v_cache": v_cache, "k_all": k_all, "v_all": v_all,
            "cu_seqlens_q": cu_q, "cu_seqlens_k": cu_k, "block_table": table, "max_seqlen_q": int(new.max()),
            "max_seqlen_k": int(tot.max()), "scale": HEAD_DIM ** -0.5}


def prefill_flops(seq_lens, hq: int = 16) -> float:
    """Causal attention flops: two products of 2*D flops per (query, visible key, head)."""
    return float(sum(4 * HEAD_DIM * hq * l * (l + 1) // 2 for l in seq_lens))


def random_seq_lens(n: int, lo: int, hi: int, seed: int = 0):
    g = _gen(seed)
    return [int(x) for x in torch.randint(lo, hi + 1, (n,), generator=g)]


def decode_inputs(ctx_lens, hq: int = 16, hkv: int = 8, seed: int = 0, poison_tail: bool = False,
                  extra_blocks: int = 0, cache_std: float = 1.0) -> dict:
    """Paged decode: one query per sequence; block_table rows are consecutive slices of one random
    block permutation, padded with -1.  With poison_tail the cache rows beyond each context (inside
    its last block) and all unused blocks are NaN."""
    g = _gen(seed)
    lens = torch.as_tensor(ctx_lens, dtype=torch.int64)
    bsz = len(lens)
    blocks_per_seq = (lens + BLOCK_SIZE - 1) // BLOCK_SIZE
    nblk = int(blocks_per_seq.sum()) + extra_blocks
    max_blocks = max(int(blocks_per_seq.max()) if bsz else 0, 1)
    perm = torch.randperm(max(nblk, 1), generator=g).to(torch.int32)
    table = torch.full((bsz, max_blocks), -1, dtype=torch.int32)
    pos = 0
    for b in range(bsz):
        nb = int(blocks_per_seq[b])
        table[b, :nb] = perm[pos:pos + nb]
        pos += nb
    k_cache = torch.empty((max(nblk, 1), BLOCK_SIZE, hkv, HEAD_DIM), dtype=torch.bfloat16)
    v_cache = torch.empty_like(k_cache)
    step = 64
    for r in range(0, k_cache.shape[0], step):
        k_cache[r:r + step] = _normal(g, (min(step, k_cache.shape[0] - r), BLOCK_SIZE, hkv, HEAD_DIM), std=cache_std)
        v_cache[r:r + step] = _normal(g, (min(step, k_cache.shape[0] - r), BLOCK_SIZE, hkv, HEAD_DIM), std=cache_std)
    if poison_tail:
        used = torch.zeros(k_cache.shape[0], dtype=torch.bool)
        for b in range(bsz):
            nb = int(blocks_per_seq[b])
            used[table[b, :nb].long()] = True
            tail = int(lens[b]) % BLOCK_SIZE
            if nb and tail:
                last = int(table[b, nb - 1])
                k_cache[last, tail:] = float("nan")
                v_cache[last, tail:] = float("nan")
        k_cache[~used] = float("nan")
        v_cache[~used] = float("nan")
    return {
        "q": _normal(g, (bsz, 1, hq, HEAD_DIM)),
        "k_cache": k_cache,
        "v_cache": v_cache,
        "cache_seqlens": lens.to(torch.int32),
        "block_table": table,
        "scale": HEAD_DIM ** -0.5,
        "ctx_lens": [int(x) for x in lens],
    }


def decode_bytes(ctx_lens, hq: int = 16, hkv: int = 8, max_blocks: int | None = None) -> float:
    """Algorithmic HBM bytes of one paged-decode call: K+V of every context token once
    (2 * hkv * 128 * 2 B = 4096 B per token at hkv = 8), Q read + O write, metadata."""
    bsz = len(ctx_lens)
    if max_blocks is None:
        max_blocks = max((l + BLOCK_SIZE - 1) // BLOCK_SIZE for l in ctx_lens)
    kv = sum(ctx_lens) * 2 * hkv * HEAD_DIM * 2
    qo = 2 * bsz * hq * HEAD_DIM * 2
    meta = 4 * (bsz * max_blocks + bsz)
    return float(kv + qo + meta)
