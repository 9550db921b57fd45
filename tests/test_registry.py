"""Host logic: the op registry and facade behave like the reference's (mops/registry.py:1-39,
mops/__init__.py:1-26): fixed backend names plus "hip", ValueError / RuntimeError / print-and-None."""
import importlib

import pytest


def test_backend_names_and_selection():
    from nano_vllm_ninetoothed_amd.mops import registry
    assert set(registry._BACKEND_REGISTRY) == {"triton", "ninetoothed", "torch", "hip"}
    prev = registry.get_current_backend()
    with pytest.raises(ValueError):
        registry.set_current_backend("cuda")
    registry.set_current_backend("hip")
    assert registry.get_current_backend() == "hip"
    registry.set_current_backend(prev)


def test_register_duplicate_raises_and_missing_returns_none(capsys):
    from nano_vllm_ninetoothed_amd.mops import registry

    @registry.register_op("triton")
    def _probe_op():
        return 1

    try:
        with pytest.raises(RuntimeError):
            registry.register_op("triton")(_probe_op)
        assert registry.get_op("_probe_op", "triton") is _probe_op
        assert registry.get_op("no_such_op", "triton") is None
        assert "no_such_op" in capsys.readouterr().out
    finally:
        registry._BACKEND_REGISTRY["triton"].pop("_probe_op", None)


def test_hip_backend_registers_all_eleven_names():
    from nano_vllm_ninetoothed_amd import mops
    for name in ("linear", "rms_forward", "add_rms_forward", "softmax", "siluAndMul", "sampler_forward",
                 "apply_rotary_emb", "embedding", "store_kvcache", "flash_attn_varlen_func", "flash_attn_with_kvcache"):
        op = mops.get_op(name, "hip")
        assert callable(op) and op.__name__ == name
        assert getattr(mops, name) is op or mops.registry.get_current_backend() != "hip"


def test_facade_reads_backend_env(monkeypatch):
    import nano_vllm_ninetoothed_amd.mops as mops
    from nano_vllm_ninetoothed_amd.mops import registry
    prev = registry.get_current_backend()
    try:
        monkeypatch.setenv("BACKEND", "bogus")
        with pytest.raises(ValueError):
            importlib.reload(mops)
    finally:
        monkeypatch.setenv("BACKEND", prev or "hip")
        # reload re-executes `from . import hip`, which is already imported: ops stay registered once
        importlib.reload(mops)
    assert mops.store_kvcache is mops.get_op("store_kvcache", "hip")


def test_signatures_accept_the_layer_call_forms():
    """Keyword names used by nanovllm/layers/attention.py:34-42 must bind."""
    import inspect
    from nano_vllm_ninetoothed_amd import mops
    inspect.signature(mops.get_op("flash_attn_varlen_func", "hip")).bind(
        1, 2, 3, max_seqlen_q=1, cu_seqlens_q=2, max_seqlen_k=3, cu_seqlens_k=4, softmax_scale=1.0, causal=True, block_table=None)
    inspect.signature(mops.get_op("flash_attn_with_kvcache", "hip")).bind(
        1, 2, 3, cache_seqlens=1, block_table=2, softmax_scale=1.0, causal=True)
    inspect.signature(mops.get_op("store_kvcache", "hip")).bind(1, 2, 3, 4, 5)
    inspect.signature(mops.get_op("rms_forward", "hip")).bind(1, 2, 1e-6)
    inspect.signature(mops.get_op("add_rms_forward", "hip")).bind(1, 2, 3, 1e-6)
    inspect.signature(mops.get_op("embedding", "hip")).bind(1, 2)


def test_hot_ops_refuse_cpu_tensors_instead_of_falling_back():
    import torch
    from nano_vllm_ninetoothed_amd import mops
    x = torch.zeros((2, 128), dtype=torch.bfloat16)
    w = torch.ones(128, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        mops.get_op("rms_forward", "hip")(x, w, 1e-6)
    with pytest.raises(ValueError):
        mops.get_op("embedding", "hip")(torch.zeros(2, dtype=torch.int64), torch.zeros((4, 128), dtype=torch.bfloat16))
