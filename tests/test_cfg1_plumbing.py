"""CPU plumbing (the benchmark's first configuration): one Qwen3-0.6B-shaped decoder-layer op sequence
through the registry on the oracle ("torch") backend — RMSNorm (eps 1e-6, w ~ 1+0.1N) over 512 tokens of
hidden 1024, store_kvcache of K/V [512,8,128] into a 4 x 256 cache through a shuffled slot_mapping, varlen
causal prefill over 2 x 256 tokens with 16/8 heads — plus the committed golden vectors at reduced size."""
import os

import numpy as np
import pytest
import torch

from helpers import assert_bit_exact
from nano_vllm_ninetoothed_amd import workloads as W

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cfg1_small.npz")


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


@pytest.fixture(scope="module")
def torch_ops():
    from nano_vllm_ninetoothed_amd import mops
    import oracle.mops_torch  # noqa: F401
    return lambda name: mops.get_op(name, "torch")


def test_cfg1_sequence_runs_through_the_registry(torch_ops):
    T = 512
    r = W.rms_inputs(T, 1024, seed=0)
    y = torch_ops("rms_forward")(r["x"], r["weight"], r["eps"])
    assert y.shape == (T, 1024) and y.dtype == torch.bfloat16 and torch.isfinite(y.float()).all()
    # unit RMS before the weight: mean(y/w)^2 ~ 1
    assert abs(((y.float() / r["weight"].float()) ** 2).mean().item() - 1.0) < 2e-2

    p = W.prefill_inputs([256, 256], hq=16, hkv=8, seed=0)
    g = torch.Generator().manual_seed(0)
    slots = torch.randperm(4 * 256, generator=g)[:T].to(torch.int32)
    kc = torch.full((4, 256, 8, 128), 123.0, dtype=torch.bfloat16)
    vc = torch.full_like(kc, 123.0)
    assert torch_ops("store_kvcache")(p["k"], p["v"], kc, vc, slots) is None
    assert_bit_exact(kc.view(-1, 8, 128)[slots.long()], p["k"], "stored K rows")
    assert_bit_exact(vc.view(-1, 8, 128)[slots.long()], p["v"], "stored V rows")
    assert int((kc.view(-1, 1024)[:, 0] == 123.0).sum()) == 512       # the other half of the cache is untouched

    o = torch_ops("flash_attn_varlen_func")(p["q"], p["k"], p["v"], max_seqlen_q=256, cu_seqlens_q=p["cu_seqlens"],
                                            max_seqlen_k=256, cu_seqlens_k=p["cu_seqlens"], softmax_scale=128 ** -0.5,
                                            causal=True, block_table=None)
    assert o.shape == (T, 16, 128) and o.dtype == torch.bfloat16 and torch.isfinite(o.float()).all()
    assert_bit_exact(o[0], p["v"][0].repeat_interleave(2, 0), "token 0 of sequence 0")
    assert_bit_exact(o[256], p["v"][256].repeat_interleave(2, 0), "token 0 of sequence 1")

    # decode one step over the cache just written: equals the last prefill row of each sequence
    table = torch.full((2, 1), -1, dtype=torch.int32)
    kc2 = torch.zeros((2, 256, 8, 128), dtype=torch.bfloat16)
    vc2 = torch.zeros_like(kc2)
    for s in range(2):
        kc2[s] = p["k"][256 * s:256 * (s + 1)]
        vc2[s] = p["v"][256 * s:256 * (s + 1)]
        table[s, 0] = s
    od = torch_ops("flash_attn_with_kvcache")(p["q"][[255, 511]].unsqueeze(1), kc2, vc2,
                                              cache_seqlens=torch.tensor([256, 256], dtype=torch.int32), block_table=table,
                                              softmax_scale=128 ** -0.5, causal=True)
    assert (od[:, 0].float() - o[[255, 511]].float()).abs().max() <= 2 ** -6


def test_oracle_reproduces_committed_golden_vectors(torch_ops):
    z = np.load(GOLDEN, allow_pickle=False)
    x, res, w, eps = from_bits(z["rms_x"]), from_bits(z["rms_res"]), from_bits(z["rms_w"]), float(z["rms_eps"])
    assert_bit_exact(torch_ops("rms_forward")(x, w, eps), from_bits(z["rms_y"]), "rms_forward")
    ya, ra = torch_ops("add_rms_forward")(x, res, w, eps)
    assert_bit_exact(ya, from_bits(z["addrms_y"]), "add_rms_forward y")
    assert_bit_exact(ra, from_bits(z["addrms_res"]), "add_rms_forward residual")

    q, k, v = from_bits(z["q"]), from_bits(z["k"]), from_bits(z["v"])
    cu = torch.from_numpy(z["cu_seqlens"])
    kc = torch.full((2, 256, 8, 128), -7.0, dtype=torch.bfloat16)
    vc = torch.full_like(kc, -7.0)
    slots = torch.from_numpy(z["slot_mapping"])
    torch_ops("store_kvcache")(k, v, kc, vc, slots)
    assert_bit_exact(kc.view(-1, 1024)[slots.long()], from_bits(z["k_cache_rows"]), "stored K rows")
    assert int((kc.float() == -7.0).sum()) == int(z["k_cache_sentinel_count"])
    o = torch_ops("flash_attn_varlen_func")(q, k, v, max_seqlen_q=40, cu_seqlens_q=cu, max_seqlen_k=40, cu_seqlens_k=cu,
                                            softmax_scale=float(z["scale"]), causal=True)
    want = from_bits(z["prefill_out"])
    assert (o.float() - want.float()).abs().max() <= 2 ** -7, "prefill vs golden (fp32 matmul blocking may differ by an ulp)"

    od = torch_ops("flash_attn_with_kvcache")(from_bits(z["dec_q"]), from_bits(z["dec_k_cache"]), from_bits(z["dec_v_cache"]),
                                              cache_seqlens=torch.from_numpy(z["dec_seqlens"]),
                                              block_table=torch.from_numpy(z["dec_table"]), softmax_scale=float(z["scale"]))
    assert (od.float() - from_bits(z["dec_out"]).float()).abs().max() <= 2 ** -7
    assert_bit_exact(torch_ops("embedding")(torch.from_numpy(z["emb_ids"]), from_bits(z["emb_w"])), from_bits(z["emb_out"]), "embedding")
