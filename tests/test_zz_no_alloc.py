"""The allocation-free paged decode entry point (fixed device scratch inside the library) gives the bits of the
entry point that takes a caller workspace: same kernels, same plan.  Called straight through the C ABI, twice in a
row on the same GPU, the second time with a smaller problem (the scratch keeps the first call's contents)."""
import pytest
import torch

from helpers import assert_attention_close, assert_bit_exact
from nano_vllm_ninetoothed_amd import _capi
from nano_vllm_ninetoothed_amd import workloads as W

pytestmark = pytest.mark.gpu


def _args(g, out):
    q = g["q"]
    batch, _, hq, d = q.shape
    kc = g["k_cache"]
    num_blocks, block_size, hkv, _ = kc.shape
    bt = g["block_table"]
    return [q.data_ptr(), q.stride(0) if batch > 1 else hq * d, kc.data_ptr(), g["v_cache"].data_ptr(),
            g["cache_seqlens"].data_ptr(), bt.data_ptr(), bt.stride(0) if batch > 1 else bt.shape[1], out.data_ptr(),
            batch, hq, hkv, d, block_size, num_blocks, bt.shape[1]]


def _with_workspace(lib, g, scale, stream):
    q = g["q"]
    out = torch.full_like(q, float("nan"))
    a = _args(g, out)
    nbytes = lib.mops_hip_paged_decode_workspace_bytes(a[8], a[9], a[10], a[14], a[12])
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    _capi.check("mops_hip_attn_paged_decode_bf16",
                lib.mops_hip_attn_paged_decode_bf16(*a, scale, ws.data_ptr(), ws.numel(), stream))
    torch.cuda.synchronize()
    return out


def _no_alloc(lib, g, scale, stream):
    out = torch.full_like(g["q"], float("nan"))
    _capi.check("mops_hip_attn_paged_decode_noalloc_bf16",
                lib.mops_hip_attn_paged_decode_noalloc_bf16(*_args(g, out), scale, stream))
    torch.cuda.synchronize()
    return out


def test_no_alloc_decode_matches_workspace_decode_twice(gpu, ops):
    lib = _capi.load()
    _, ref = ops("flash_attn_with_kvcache")
    stream = torch.cuda.current_stream(gpu).cuda_stream
    # first call: 96 ragged sequences (many split over several columns), then a smaller one with other lengths:
    # whatever the first call left in the scratch must not leak into the second
    for ctx, seed in ((W.random_seq_lens(96, 1, 4096, seed=21), 21), ([700, 1, 33, 2049, 256], 22)):
        d = W.decode_inputs(ctx, seed=seed, poison_tail=True)
        g = W.to_device(d, gpu)
        want = _with_workspace(lib, g, d["scale"], stream)
        got = _no_alloc(lib, g, d["scale"], stream)
        assert_bit_exact(got, want, f"no-alloc decode vs workspace decode, {len(ctx)} sequences")
        oracle = ref(d["q"], torch.nan_to_num(d["k_cache"]), torch.nan_to_num(d["v_cache"]), cache_seqlens=d["cache_seqlens"],
                     block_table=d["block_table"], softmax_scale=d["scale"], causal=True)
        assert_attention_close(got, oracle, f"no-alloc decode vs oracle, {len(ctx)} sequences")


def test_no_alloc_decode_allocates_nothing_and_can_be_captured(gpu):
    """What the entry point exists for: a call after the first one on a device takes no device memory (neither from the
    driver nor from torch's allocator), and it can be recorded into a HIP graph (the first call, which looks up the
    scratch's address, has happened before); every replay gives the eager call's bits."""
    lib = _capi.load()
    d = W.decode_inputs([700, 1, 33, 2049, 256, 4000], seed=23)
    g = W.to_device(d, gpu)
    out = torch.full_like(g["q"], float("nan"))
    args = _args(g, out)
    stream = torch.cuda.current_stream(gpu).cuda_stream
    _capi.check("warm-up", lib.mops_hip_attn_paged_decode_noalloc_bf16(*args, d["scale"], stream))
    torch.cuda.synchronize()
    eager = out.clone()
    free0, _ = torch.cuda.mem_get_info(gpu)
    alloc0, reserved0 = torch.cuda.memory_allocated(gpu), torch.cuda.memory_reserved(gpu)
    for _ in range(3):
        _capi.check("call", lib.mops_hip_attn_paged_decode_noalloc_bf16(*args, d["scale"], stream))
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(gpu)
    assert (torch.cuda.memory_allocated(gpu), torch.cuda.memory_reserved(gpu)) == (alloc0, reserved0)
    assert free1 == free0, f"device memory in use changed by {free0 - free1} bytes across allocation-free calls"
    assert_bit_exact(out, eager, "repeated allocation-free call")
    side = torch.cuda.Stream(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _capi.check("captured call", lib.mops_hip_attn_paged_decode_noalloc_bf16(*args, d["scale"], side.cuda_stream))
    for i in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_bit_exact(out, eager, f"replay {i} of the captured allocation-free call")


def test_no_alloc_decode_rejects_what_does_not_fit(gpu):
    lib = _capi.load()
    A = 0x1000   # never dereferenced: the size check comes before any launch
    # 4 kv heads -> 512 columns x 2 slots x 64 query heads x 128 floats = 33.5 MB: beyond the fixed scratch
    st = lib.mops_hip_attn_paged_decode_noalloc_bf16(A, 64 * 128, A, A, A, A, 16, A, 4, 64, 4, 128, 256, 64, 16, 0.088, None)
    assert st == -6
    assert b"scratch" in lib.mops_hip_status_string(st)
    # the shared validation still applies
    assert lib.mops_hip_attn_paged_decode_noalloc_bf16(A, 2048, A, A, A, A, 16, A, 4, 16, 8, 64, 256, 64, 16, 0.088, None) == -2
    assert lib.mops_hip_attn_paged_decode_noalloc_bf16(None, 2048, A, A, A, A, 16, A, 0, 16, 8, 128, 256, 64, 16, 0.088, None) == 0
