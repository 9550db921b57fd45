"""GPU parity, bit-exact ops: store_kvcache and embedding through the hip backend (C ABI) vs the oracle."""
import pytest
import torch

from helpers import assert_bit_exact
from nano_vllm_ninetoothed_amd import workloads as W

pytestmark = pytest.mark.gpu


def _caches(num_blocks, hkv, sentinel=-7.0):
    shape = (num_blocks, W.BLOCK_SIZE, hkv, W.HEAD_DIM)
    return torch.full(shape, sentinel, dtype=torch.bfloat16), torch.full(shape, sentinel * 2, dtype=torch.bfloat16)


@pytest.mark.parametrize("n_tokens,v_stride", [(512, None), (1, None), (3, 4096), (777, 4096), (17437, 4096)])
def test_store_kvcache_matches_oracle(gpu, ops, n_tokens, v_stride):
    hip, ref = ops("store_kvcache")
    d = W.store_inputs(n_tokens, seed=n_tokens, v_row_stride=v_stride)
    kc, vc = _caches(d["num_blocks"], d["hkv"])
    ref(d["key"], d["value"], kc, vc, d["slot_mapping"])
    kc_g, vc_g = (t.to(gpu) for t in _caches(d["num_blocks"], d["hkv"]))
    value_g = d["value"].to(gpu) if v_stride is None else None
    if v_stride is not None:  # rebuild the strided view on the GPU
        wide = d["value"]._base.to(gpu)
        value_g = wide[:, v_stride - d["hkv"] * W.HEAD_DIM:].view(n_tokens, d["hkv"], W.HEAD_DIM)
        assert value_g.stride(0) == v_stride
    out = hip(d["key"].to(gpu), value_g, kc_g, vc_g, d["slot_mapping"].to(gpu))
    assert out is None
    assert_bit_exact(kc_g, kc, "k_cache")
    assert_bit_exact(vc_g, vc, "v_cache")


def test_store_kvcache_benchmark_token_count(gpu, ops):
    """The store of the prefill benchmark exactly as it is drawn: T = the sum of the 16 seeded sequence lengths
    (uniform in [128, 2048], seed 0) = 20514 tokens, V a view with row stride 4096, random-permutation slots; bit-exact
    against the scatter of mops/triton/attention.py:30-38."""
    hip, ref = ops("store_kvcache")
    T = sum(W.random_seq_lens(16, 128, 2048, seed=0))
    assert T == 20514
    d = W.store_inputs(T, seed=0, v_row_stride=4096)
    kc, vc = _caches(d["num_blocks"], d["hkv"])
    ref(d["key"], d["value"], kc, vc, d["slot_mapping"])
    kc_g, vc_g = (t.to(gpu) for t in _caches(d["num_blocks"], d["hkv"]))
    wide = d["value"]._base.to(gpu)
    value_g = wide[:, 4096 - d["hkv"] * W.HEAD_DIM:].view(T, d["hkv"], W.HEAD_DIM)
    assert value_g.stride(0) == 4096
    hip(d["key"].to(gpu), value_g, kc_g, vc_g, d["slot_mapping"].to(gpu))
    assert_bit_exact(kc_g, kc, "k_cache")
    assert_bit_exact(vc_g, vc, "v_cache")


def test_store_kvcache_skips_minus_one_and_keeps_other_slots(gpu, ops):
    hip, ref = ops("store_kvcache")
    d = W.store_inputs(300, seed=5)
    slots = d["slot_mapping"].clone()
    slots[::3] = -1
    kc, vc = _caches(d["num_blocks"], d["hkv"])
    ref(d["key"], d["value"], kc, vc, slots)
    kc_g, vc_g = (t.to(gpu) for t in _caches(d["num_blocks"], d["hkv"]))
    hip(d["key"].to(gpu), d["value"].to(gpu), kc_g, vc_g, slots.to(gpu))
    assert_bit_exact(kc_g, kc, "k_cache")
    assert_bit_exact(vc_g, vc, "v_cache")
    untouched = torch.ones(d["num_blocks"] * W.BLOCK_SIZE, dtype=torch.bool)
    untouched[slots[slots >= 0].long()] = False
    assert (kc_g.view(-1, 1024).cpu()[untouched] == -7.0).all()


def test_store_kvcache_empty_and_bad_layout(gpu, ops):
    hip, _ = ops("store_kvcache")
    kc_g, vc_g = (t.to(gpu) for t in _caches(2, 8))
    empty = torch.empty((0, 8, 128), dtype=torch.bfloat16, device=gpu)
    hip(empty, empty, kc_g, vc_g, torch.empty(0, dtype=torch.int32, device=gpu))
    k = torch.zeros((4, 8, 128), dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError):
        hip(k, k, kc_g, vc_g, torch.zeros(3, dtype=torch.int32, device=gpu))       # wrong slot count
    with pytest.raises(ValueError):
        hip(k.transpose(1, 2), k.transpose(1, 2), kc_g, vc_g, torch.zeros(4, dtype=torch.int32, device=gpu))


@pytest.mark.parametrize("n_ids,vocab,hidden,dtype", [
    (512, 151936, 1024, torch.int64), (512, 4096, 4096, torch.int32), (1, 1000, 1024, torch.int64),
    (37, 5000, 2048, torch.int32), (300, 777, 128, torch.int64), (64, 2000, 5120, torch.int32)])
def test_embedding_matches_oracle(gpu, ops, n_ids, vocab, hidden, dtype):
    hip, ref = ops("embedding")
    d = W.embedding_inputs(n_ids, vocab, hidden, seed=hidden + n_ids, id_dtype=dtype)
    want = ref(d["ids"], d["weight"])
    got = hip(d["ids"].to(gpu), d["weight"].to(gpu))
    assert_bit_exact(got, want, "embedding")
    assert_bit_exact(got, torch.nn.functional.embedding(d["ids"].long(), d["weight"]), "embedding vs F.embedding")


def test_embedding_full_size_8b_table(gpu, ops):
    """The Qwen3-8B-shaped case at its exact size: 512 int32 ids uniform over a bf16 [151936, 4096] table ~N(0, 0.02)
    (1.24 GB), bit-exact against weight[ids] (nanovllm/layers/embed_head.py:41)."""
    hip, ref = ops("embedding")
    d = W.embedding_inputs(512, 151936, 4096, seed=0, id_dtype=torch.int32)
    assert d["ids"].dtype == torch.int32 and d["weight"].shape == (151936, 4096)
    got = hip(d["ids"].to(gpu), d["weight"].to(gpu))
    assert got.shape == (512, 4096)
    assert_bit_exact(got, d["weight"][d["ids"].long()], "embedding, 151936 x 4096 table")
    assert_bit_exact(got, ref(d["ids"], d["weight"]), "embedding vs oracle")


def test_embedding_2d_ids_and_empty(gpu, ops):
    hip, ref = ops("embedding")
    d = W.embedding_inputs(48, 3000, 1024, seed=9, id_dtype=torch.int64)
    ids2 = d["ids"].view(4, 12)
    got = hip(ids2.to(gpu), d["weight"].to(gpu))
    assert got.shape == (4, 12, 1024)
    assert_bit_exact(got, ref(ids2, d["weight"]), "embedding 2-D")
    none = hip(torch.empty(0, dtype=torch.int64, device=gpu), d["weight"].to(gpu))
    assert none.shape == (0, 1024)
