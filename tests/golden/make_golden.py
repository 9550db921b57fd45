"""Writes tests/golden/cfg1_small.npz: inputs and oracle outputs of one Qwen3-0.6B-shaped decoder-layer
op sequence at reduced size (the CPU plumbing configuration: RMSNorm -> store_kvcache -> varlen causal
prefill, plus one paged decode step and an embedding lookup over the same data).

The reference ships no fixtures for these ops (it has no tests), and its torch backend cannot run
without a GPU, flash-attn and Triton.  The vectors here are therefore produced by the build's own
CPU oracle (oracle/mops_torch.py), which tests/test_oracle.py pins against fp64 brute force, library
routines and invariants; this file freezes them so that a change to the oracle, to the workload
generators or to torch's CPU kernels shows up as a diff.  bf16 tensors are stored as uint16 bit patterns.

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from nano_vllm_ninetoothed_amd import workloads as W  # noqa: E402
import oracle.mops_torch as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cfg1_small.npz")


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def build():
    torch.set_num_threads(1)
    lens = [24, 40]                       # two sequences, 64 tokens (cfg1 uses 2 x 256)
    T = sum(lens)
    r = W.rms_inputs(T, 1024, seed=0, with_residual=True)
    y = O.rms_forward(r["x"], r["weight"], r["eps"])
    ya, ra = O.add_rms_forward(r["x"], r["residual"], r["weight"], r["eps"])
    p = W.prefill_inputs(lens, hq=16, hkv=8, seed=0)
    s = W.store_inputs(T, hkv=8, num_blocks=2, seed=0)
    kc = torch.full((2, 256, 8, 128), -7.0, dtype=torch.bfloat16)
    vc = torch.full((2, 256, 8, 128), -7.0, dtype=torch.bfloat16)
    O.store_kvcache(p["k"], p["v"], kc, vc, s["slot_mapping"])
    o = O.flash_attn_varlen_func(p["q"], p["k"], p["v"], max_seqlen_q=max(lens), cu_seqlens_q=p["cu_seqlens"],
                                 max_seqlen_k=max(lens), cu_seqlens_k=p["cu_seqlens"], softmax_scale=p["scale"], causal=True)
    d = W.decode_inputs([40, 17], hq=4, hkv=2, seed=1)   # small heads keep the cache fixture small
    od = O.flash_attn_with_kvcache(d["q"], d["k_cache"], d["v_cache"], cache_seqlens=d["cache_seqlens"],
                                   block_table=d["block_table"], softmax_scale=d["scale"], causal=True)
    e = W.embedding_inputs(16, 64, 256, seed=2, id_dtype=torch.int64)
    oe = O.embedding(e["ids"], e["weight"])
    return dict(
        rms_x=bits(r["x"]), rms_res=bits(r["residual"]), rms_w=bits(r["weight"]), rms_eps=np.float32(r["eps"]),
        rms_y=bits(y), addrms_y=bits(ya), addrms_res=bits(ra),
        q=bits(p["q"]), k=bits(p["k"]), v=bits(p["v"]), cu_seqlens=p["cu_seqlens"].numpy(), scale=np.float32(p["scale"]),
        slot_mapping=s["slot_mapping"].numpy(),
        k_cache_rows=bits(kc.view(-1, 1024)[s["slot_mapping"].long()]), k_cache_sentinel_count=np.int64((kc.float() == -7.0).sum()),
        prefill_out=bits(o),
        dec_q=bits(d["q"]), dec_k_cache=bits(d["k_cache"]), dec_v_cache=bits(d["v_cache"]),
        dec_seqlens=d["cache_seqlens"].numpy(), dec_table=d["block_table"].numpy(), dec_out=bits(od),
        emb_ids=e["ids"].numpy(), emb_w=bits(e["weight"]), emb_out=bits(oe),
    )


if __name__ == "__main__":
    np.savez_compressed(OUT, **build())
    print(OUT, os.path.getsize(OUT), "bytes")
