"""GPU parity against the committed golden vectors (tests/golden/cfg1_small.npz): the hip backend on
exactly the stored inputs vs the stored oracle outputs.  Copies bit-exact, norms by the two-rounding
rule, attention within max-abs 2e-2 / mean-abs 2e-3."""
import os

import numpy as np
import pytest
import torch

from helpers import assert_attention_close, assert_bit_exact, assert_rms_parity

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cfg1_small.npz")


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_hip_backend_on_golden_vectors(gpu):
    from nano_vllm_ninetoothed_amd import mops
    hip = lambda n: mops.get_op(n, "hip")  # noqa: E731
    z = np.load(GOLDEN, allow_pickle=False)
    x, res, w, eps = from_bits(z["rms_x"]), from_bits(z["rms_res"]), from_bits(z["rms_w"]), float(z["rms_eps"])

    def normed(s):
        return (s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps)).to(torch.bfloat16)

    y = hip("rms_forward")(x.to(gpu), w.to(gpu), eps)
    assert_rms_parity(y, normed(x.float()), w, from_bits(z["rms_y"]), "rms_forward")
    ya, ra = hip("add_rms_forward")(x.to(gpu), res.to(gpu), w.to(gpu), eps)
    assert_bit_exact(ra, from_bits(z["addrms_res"]), "add_rms residual")
    assert_rms_parity(ya, normed(x.float() + res.float()), w, from_bits(z["addrms_y"]), "add_rms_forward")

    q, k, v = from_bits(z["q"]), from_bits(z["k"]), from_bits(z["v"])
    cu = torch.from_numpy(z["cu_seqlens"]).to(gpu)
    slots = torch.from_numpy(z["slot_mapping"])
    kc = torch.full((2, 256, 8, 128), -7.0, dtype=torch.bfloat16, device=gpu)
    vc = torch.full_like(kc, -7.0)
    hip("store_kvcache")(k.to(gpu), v.to(gpu), kc, vc, slots.to(gpu))
    assert_bit_exact(kc.view(-1, 1024)[slots.long().to(gpu)], from_bits(z["k_cache_rows"]), "stored K rows")
    assert int((kc.float() == -7.0).sum()) == int(z["k_cache_sentinel_count"])
    assert_bit_exact(vc.view(-1, 8, 128)[slots.long().to(gpu)], v, "stored V rows")

    o = hip("flash_attn_varlen_func")(q.to(gpu), k.to(gpu), v.to(gpu), max_seqlen_q=40, cu_seqlens_q=cu, max_seqlen_k=40,
                                      cu_seqlens_k=cu, softmax_scale=float(z["scale"]), causal=True, block_table=None)
    assert_attention_close(o, from_bits(z["prefill_out"]), "prefill")
    od = hip("flash_attn_with_kvcache")(from_bits(z["dec_q"]).to(gpu), from_bits(z["dec_k_cache"]).to(gpu),
                                        from_bits(z["dec_v_cache"]).to(gpu),
                                        cache_seqlens=torch.from_numpy(z["dec_seqlens"]).to(gpu),
                                        block_table=torch.from_numpy(z["dec_table"]).to(gpu), softmax_scale=float(z["scale"]), causal=True)
    assert_attention_close(od, from_bits(z["dec_out"]), "decode")
    oe = hip("embedding")(torch.from_numpy(z["emb_ids"]).to(gpu), from_bits(z["emb_w"]).to(gpu))
    assert_bit_exact(oe, from_bits(z["emb_out"]), "embedding")
