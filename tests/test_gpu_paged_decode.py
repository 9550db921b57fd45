"""GPU parity for paged decode attention (flash_attn_with_kvcache) through the hip backend.

Tolerance: max-abs 2e-2, mean-abs 2e-3 against the fp32 oracle (bf16 inputs/outputs, fp32 accumulate)."""
import pytest
import torch

from helpers import assert_attention_close, assert_bit_exact
from nano_vllm_ninetoothed_amd import workloads as W

pytestmark = pytest.mark.gpu


def _run(hip, d, gpu):
    g = W.to_device(d, gpu)
    return hip(g["q"], g["k_cache"], g["v_cache"], cache_seqlens=g["cache_seqlens"], block_table=g["block_table"],
               softmax_scale=d["scale"], causal=True)


def _ref(ref, d):
    clean = dict(d)
    return ref(d["q"], torch.nan_to_num(d["k_cache"]), torch.nan_to_num(d["v_cache"]), cache_seqlens=d["cache_seqlens"],
               block_table=d["block_table"], softmax_scale=d["scale"], causal=True)


@pytest.mark.parametrize("ctx,hq,hkv", [
    ([1], 16, 8), ([31], 16, 8), ([32], 16, 8), ([33], 16, 8), ([255], 16, 8), ([256], 16, 8), ([257], 16, 8),
    ([512, 513, 1, 1024, 300], 16, 8), ([700, 64, 2048, 257], 32, 8), ([4096, 3, 1000], 16, 8),
    ([100, 200], 8, 8), ([640, 1300], 8, 1), ([900], 64, 4)])
def test_decode_matches_oracle(gpu, ops, ctx, hq, hkv):
    hip, ref = ops("flash_attn_with_kvcache")
    d = W.decode_inputs(ctx, hq=hq, hkv=hkv, seed=sum(ctx) + hq, poison_tail=True, extra_blocks=2)
    got = _run(hip, d, gpu)
    assert got.shape == (len(ctx), 1, hq, 128) and got.dtype == torch.bfloat16
    assert_attention_close(got, _ref(ref, d), f"decode ctx={ctx} {hq}:{hkv}")


def test_decode_batch_of_ragged_contexts(gpu, ops):
    hip, ref = ops("flash_attn_with_kvcache")
    ctx = W.random_seq_lens(48, 1, 4096, seed=2)
    d = W.decode_inputs(ctx, seed=2, poison_tail=True)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), "ragged batch")


@pytest.mark.parametrize("ctx", [[16384], [9000, 5], [70] * 3 + [12000]])
def test_decode_short_batch_of_long_contexts(gpu, ops, ctx):
    """Few sequences with long contexts: one sequence is spread over hundreds of columns of the flat split,
    so its partial results outnumber the lanes of the combining wave."""
    hip, ref = ops("flash_attn_with_kvcache")
    d = W.decode_inputs(ctx, seed=sum(ctx), poison_tail=True)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), f"decode ctx={ctx}")


def test_decode_plan_shared_between_calls(gpu, ops):
    """reuse_plan: a second call with other q and other caches but the same lengths and tables (the next layer
    of a decode step) skips the planning kernel and gives the bits of a call that plans for itself."""
    hip, _ = ops("flash_attn_with_kvcache")
    ctx = W.random_seq_lens(40, 1, 3000, seed=8)
    d1 = W.to_device(W.decode_inputs(ctx, seed=8), gpu)
    d2 = W.to_device(W.decode_inputs(ctx, seed=9), gpu)   # same geometry, different data
    kw = dict(cache_seqlens=d1["cache_seqlens"], block_table=d1["block_table"], softmax_scale=d1["scale"], causal=True)
    want2 = hip(d2["q"], d2["k_cache"], d2["v_cache"], **kw).clone()
    hip(d1["q"], d1["k_cache"], d1["v_cache"], **kw)                       # layer 1 plans
    got2 = hip(d2["q"], d2["k_cache"], d2["v_cache"], reuse_plan=True, **kw)   # layer 2 reuses
    assert_bit_exact(got2, want2, "decode with a reused plan")


def test_decode_is_bitwise_reproducible(gpu, ops):
    """The same launch repeated gives the same bits: the split of the KV stream over workgroups and the
    order in which partial results are combined do not depend on timing."""
    hip, _ = ops("flash_attn_with_kvcache")
    d = W.decode_inputs(W.random_seq_lens(64, 1, 4096, seed=5), seed=5)
    first = _run(hip, d, gpu).clone()
    for _ in range(30):
        assert_bit_exact(_run(hip, d, gpu), first, "decode, repeated launch")


def test_decode_zero_length_rows_are_zero_and_finite(gpu, ops):
    """Graph-replay padding hands cache_seqlens == 0 rows (model_runner.py:202 of the reference)."""
    hip, ref = ops("flash_attn_with_kvcache")
    d = W.decode_inputs([300, 1, 700], seed=4, poison_tail=True)
    d["cache_seqlens"] = torch.tensor([300, 0, 700], dtype=torch.int32)
    d["block_table"][1] = -1
    got = _run(hip, d, gpu)
    assert torch.isfinite(got.float()).all()
    assert (got[1].float() == 0).all()
    want = _ref(ref, d)
    assert_attention_close(got[[0, 2]], want[[0, 2]], "non-empty rows")


def test_decode_invariant_under_block_permutation(gpu, ops):
    hip, _ = ops("flash_attn_with_kvcache")
    d = W.decode_inputs([1000, 257, 513], seed=6)
    base = _run(hip, d, gpu)
    nb = d["k_cache"].shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nb)
    d2 = dict(d)
    d2["k_cache"] = d["k_cache"][perm]
    d2["v_cache"] = d["v_cache"][perm]
    tbl = d["block_table"].clone()
    mask = tbl >= 0
    tbl[mask] = inv[tbl[mask].long()].to(torch.int32)
    d2["block_table"] = tbl
    assert_bit_exact(_run(hip, d2, gpu), base, "permuting blocks + table")


def test_decode_equals_last_row_of_prefill(gpu, ops):
    dec, _ = ops("flash_attn_with_kvcache")
    pre, _ = ops("flash_attn_varlen_func")
    L = 777
    p = W.prefill_inputs([L], seed=8)
    nb = (L + 255) // 256
    kc = torch.zeros((nb, 256, 8, 128), dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    kc.view(-1, 8, 128)[:L] = p["k"]
    vc.view(-1, 8, 128)[:L] = p["v"]
    o_pre = pre(p["q"].to(gpu), p["k"].to(gpu), p["v"].to(gpu), max_seqlen_q=L, cu_seqlens_q=p["cu_seqlens"].to(gpu),
                max_seqlen_k=L, cu_seqlens_k=p["cu_seqlens"].to(gpu), softmax_scale=p["scale"], causal=True, block_table=None)
    o_dec = dec(p["q"][L - 1:L].unsqueeze(1).to(gpu), kc.to(gpu), vc.to(gpu),
                cache_seqlens=torch.tensor([L], dtype=torch.int32, device=gpu),
                block_table=torch.arange(nb, dtype=torch.int32, device=gpu).view(1, nb), softmax_scale=p["scale"], causal=True)
    assert_attention_close(o_dec[0, 0], o_pre[L - 1], "decode vs last prefill row")


def test_decode_single_token_returns_v_and_constant_v(gpu, ops):
    hip, _ = ops("flash_attn_with_kvcache")
    d = W.decode_inputs([1, 600], seed=10)
    d["v_cache"][d["block_table"][1, :3].long()] = 0.5      # constant V for sequence 1
    got = _run(hip, d, gpu).cpu()
    v0 = d["v_cache"][d["block_table"][0, 0].long(), 0]     # [8, 128]
    assert_bit_exact(got[0, 0], v0.repeat_interleave(2, dim=0), "L=1 -> o = v")
    assert (got[1].float() == 0.5).all(), "constant V -> o = V"


def test_decode_wide_padded_table_and_strided_q(gpu, ops):
    """block_table wider than needed (padded with -1) and q taken as a view of a [B, Hq*D + extra] buffer."""
    hip, ref = ops("flash_attn_with_kvcache")
    d = W.decode_inputs([300, 900], seed=12, poison_tail=True)
    wide = torch.full((2, 40), -1, dtype=torch.int32)
    wide[:, :d["block_table"].shape[1]] = d["block_table"]
    d["block_table"] = wide
    want = _ref(ref, d)
    g = W.to_device(d, gpu)
    buf = torch.zeros((2, 16 * 128 + 2048), dtype=torch.bfloat16, device=gpu)
    buf[:, :2048] = g["q"].view(2, -1)
    qv = buf[:, :2048].view(2, 16, 128).unsqueeze(1)
    got = hip(qv, g["k_cache"], g["v_cache"], cache_seqlens=g["cache_seqlens"], block_table=g["block_table"],
              softmax_scale=d["scale"], causal=True)
    assert_attention_close(got, want, "wide table / strided q")


def test_decode_large_scores_stay_finite(gpu, ops):
    hip, ref = ops("flash_attn_with_kvcache")
    d = W.decode_inputs([1500], seed=14, cache_std=6.0)
    d["q"] = d["q"] * 4
    got = _run(hip, d, gpu)
    assert torch.isfinite(got.float()).all()
    assert_attention_close(got, _ref(ref, d), "peaky softmax")


@pytest.mark.parametrize("hq,hkv,lo,hi,bsz", [(16, 8, 512, 4096, 256)])
def test_decode_full_size_properties(gpu, ops, hq, hkv, lo, hi, bsz):
    """Benchmark-size run (256 sequences, 512..4096 context): checked on a sample of sequences against the
    oracle, plus finiteness of everything and the convex-hull bound |o| <= max|v| of its context."""
    hip, ref = ops("flash_attn_with_kvcache")
    ctx = W.random_seq_lens(bsz, lo, hi, seed=0)
    d = W.decode_inputs(ctx, hq=hq, hkv=hkv, seed=0)
    got = _run(hip, d, gpu).cpu()
    assert torch.isfinite(got.float()).all()
    assert got.float().abs().max() <= d["v_cache"].float().abs().max()
    pick = [0, 1, 17, 100, 255, int(torch.tensor(ctx).argmax()), int(torch.tensor(ctx).argmin())]
    sub = {"q": d["q"][pick], "k_cache": d["k_cache"], "v_cache": d["v_cache"], "cache_seqlens": d["cache_seqlens"][pick],
           "block_table": d["block_table"][pick], "scale": d["scale"]}
    assert_attention_close(got[pick], _ref(ref, sub), "sampled sequences of the full-size batch")


def test_decode_8b_shape_full_size_properties(gpu, ops):
    """The 8B-shaped benchmark configuration at full size (512 sequences, 32 query / 8 kv heads, contexts
    1024..8192, ~9.7 GB of cache) with the cache filled on the device: finiteness, the convex-hull bound
    |o| <= max|v|, and a sample of sequences checked against the oracle on a cache cut down to their blocks."""
    hip, ref = ops("flash_attn_with_kvcache")
    bsz, hq, hkv, bs = 512, 32, 8, 256
    ctx = torch.tensor(W.random_seq_lens(bsz, 1024, 8192, seed=0), dtype=torch.int64)
    nblocks = (ctx + bs - 1) // bs
    total = int(nblocks.sum())
    g = torch.Generator().manual_seed(4)
    perm = torch.randperm(total, generator=g).to(torch.int32)
    table = torch.full((bsz, int(nblocks.max())), -1, dtype=torch.int32)
    pos = 0
    for b in range(bsz):
        table[b, :int(nblocks[b])] = perm[pos:pos + int(nblocks[b])]
        pos += int(nblocks[b])
    gd = torch.Generator(device=gpu).manual_seed(4)
    k_cache = torch.empty((total, bs, hkv, 128), dtype=torch.bfloat16, device=gpu)
    v_cache = torch.empty_like(k_cache)
    for r in range(0, total, 512):      # filled in slabs: the fp32 draw of the whole cache would not fit beside it
        n = min(512, total - r)
        k_cache[r:r + n] = torch.randn((n, bs, hkv, 128), generator=gd, device=gpu, dtype=torch.float32).to(torch.bfloat16)
        v_cache[r:r + n] = torch.randn((n, bs, hkv, 128), generator=gd, device=gpu, dtype=torch.float32).to(torch.bfloat16)
    q = torch.randn((bsz, 1, hq, 128), generator=g).to(torch.bfloat16)
    scale = 128 ** -0.5
    got = hip(q.to(gpu), k_cache, v_cache, cache_seqlens=ctx.to(torch.int32).to(gpu), block_table=table.to(gpu),
              softmax_scale=scale, causal=True)
    assert got.shape == (bsz, 1, hq, 128)
    assert torch.isfinite(got.float()).all()
    assert got.float().abs().max() <= v_cache.float().abs().max()
    pick = [0, 7, 255, 511, int(ctx.argmax()), int(ctx.argmin())]
    blocks = torch.cat([table[b, :int(nblocks[b])] for b in pick]).long()
    sub_table = torch.full((len(pick), table.shape[1]), -1, dtype=torch.int32)
    pos = 0
    for i, b in enumerate(pick):
        sub_table[i, :int(nblocks[b])] = torch.arange(pos, pos + int(nblocks[b]), dtype=torch.int32)
        pos += int(nblocks[b])
    want = ref(q[pick], k_cache[blocks.to(gpu)].cpu(), v_cache[blocks.to(gpu)].cpu(), cache_seqlens=ctx[pick].to(torch.int32),
               block_table=sub_table, softmax_scale=scale, causal=True)
    assert_attention_close(got[pick].cpu(), want, "sampled sequences of the 8B-shaped full-size batch")


@pytest.mark.parametrize("ctx,hq,hkv", [([300, 900, 31], 8, 4), ([700, 5], 4, 2), ([513, 1025], 16, 1), ([2000], 12, 6)])
def test_decode_other_head_counts(gpu, ops, ctx, hq, hkv):
    hip, ref = ops("flash_attn_with_kvcache")
    d = W.decode_inputs(ctx, hq=hq, hkv=hkv, seed=sum(ctx) + hkv, poison_tail=True)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), f"decode {hq}:{hkv}")


def test_decode_many_short_sequences_uses_the_large_batch_plan(gpu, ops):
    """More sequences than the plan kernel keeps in LDS (4096): prefix sums are searched in global memory;
    a quarter of the rows are empty."""
    hip, ref = ops("flash_attn_with_kvcache")
    g = torch.Generator().manual_seed(3)
    ctx = torch.randint(0, 80, (5000,), generator=g)
    ctx[ctx < 20] = 0
    lens = [int(x) for x in ctx]
    d = W.decode_inputs([max(l, 1) for l in lens], hq=4, hkv=2, seed=3)
    d["cache_seqlens"] = torch.tensor(lens, dtype=torch.int32)
    got = _run(hip, d, gpu).cpu()
    want = _ref(ref, d)
    assert (got[ctx == 0].float() == 0).all()
    assert_attention_close(got, want, "5000 short sequences")


@pytest.mark.parametrize("block_size", [64, 512])
def test_decode_other_block_sizes(gpu, ops, block_size):
    """The kernels only need the block size to be a multiple of 32; the reference uses multiples of 256."""
    hip, ref = ops("flash_attn_with_kvcache")
    d = W.decode_inputs([1000, 300, 64], seed=block_size)
    # re-block the same tokens: [nblk, 256, h, d] -> [nblk * 256 / bs, bs, h, d] with the table expanded / merged
    nblk = d["k_cache"].shape[0]
    if block_size < 256:
        f = 256 // block_size
        kc = d["k_cache"].view(nblk * f, block_size, 8, 128)
        vc = d["v_cache"].view(nblk * f, block_size, 8, 128)
        t = d["block_table"]
        tbl = torch.where(t.unsqueeze(-1) >= 0, t.unsqueeze(-1) * f + torch.arange(f, dtype=torch.int32), torch.full((1,), -1, dtype=torch.int32))
        tbl = tbl.reshape(t.shape[0], -1).contiguous()
        g = {"q": d["q"].to(gpu), "k": kc.to(gpu), "v": vc.to(gpu), "t": tbl.to(gpu)}
        got = hip(g["q"], g["k"], g["v"], cache_seqlens=d["cache_seqlens"].to(gpu), block_table=g["t"], softmax_scale=d["scale"], causal=True)
        assert_attention_close(got, _ref(ref, d), f"block size {block_size}")
    else:
        d2 = W.decode_inputs([1000, 300, 64], seed=block_size)
        # build a 512-token-block cache by pairing up 256-token blocks of a fresh layout
        from nano_vllm_ninetoothed_amd import workloads as W2
        lens = d2["ctx_lens"]
        bps = [(l + 511) // 512 for l in lens]
        nb = sum(bps)
        gen = torch.Generator().manual_seed(9)
        kc = torch.randn((nb, 512, 8, 128), generator=gen).to(torch.bfloat16)
        vc = torch.randn((nb, 512, 8, 128), generator=gen).to(torch.bfloat16)
        tbl = torch.full((3, max(bps)), -1, dtype=torch.int32)
        perm = torch.randperm(nb, generator=gen).to(torch.int32)
        pos = 0
        for b, n in enumerate(bps):
            tbl[b, :n] = perm[pos:pos + n]
            pos += n
        want = ref(d2["q"], kc, vc, cache_seqlens=d2["cache_seqlens"], block_table=tbl, softmax_scale=d2["scale"], causal=True)
        got = hip(d2["q"].to(gpu), kc.to(gpu), vc.to(gpu), cache_seqlens=d2["cache_seqlens"].to(gpu), block_table=tbl.to(gpu),
                  softmax_scale=d2["scale"], causal=True)
        assert_attention_close(got, want, "block size 512")


def test_reuse_plan_without_a_matching_plan_is_refused(gpu, ops):
    """reuse_plan=True is only legal right after a planning call with the same metadata tensors and head
    geometry on the same stream; the wrapper raises instead of launching on a plan made for something else."""
    hip, _ = ops("flash_attn_with_kvcache")
    d1 = W.to_device(W.decode_inputs([700, 300, 64], seed=31), gpu)
    d2 = W.to_device(W.decode_inputs([700, 300, 64, 90], seed=32), gpu)
    kw1 = dict(cache_seqlens=d1["cache_seqlens"], block_table=d1["block_table"], softmax_scale=d1["scale"], causal=True)
    kw2 = dict(cache_seqlens=d2["cache_seqlens"], block_table=d2["block_table"], softmax_scale=d2["scale"], causal=True)
    hip(d1["q"], d1["k_cache"], d1["v_cache"], **kw1)
    with pytest.raises(ValueError, match="reuse_plan"):
        hip(d2["q"], d2["k_cache"], d2["v_cache"], reuse_plan=True, **kw2)        # other batch, other tensors
    with pytest.raises(ValueError, match="reuse_plan"):
        hip(d1["q"], d1["k_cache"], d1["v_cache"], reuse_plan=True, **dict(kw1, cache_seqlens=d1["cache_seqlens"].clone()))
    hip(d1["q"], d1["k_cache"], d1["v_cache"], reuse_plan=True, **kw1)            # the matching one is accepted


def test_lengths_rewritten_in_place_need_a_new_plan(gpu, ops):
    """The static-buffer pattern of a serving loop: cache_seqlens and block_table keep their addresses and are rewritten
    in place between decode steps.  The reuse_plan check compares addresses, so it cannot see that; the contract is that
    the first layer of every step plans again.  Doing so gives the oracle's answer for the new lengths, and the layers
    that then reuse the plan give the bits of calls that plan for themselves.  (Reusing the OLD plan after the rewrite is
    the caller's error: it would cut the new lengths by the old split; it is documented, not detected.)"""
    hip, ref = ops("flash_attn_with_kvcache")
    ctx_a, ctx_b = [900, 2100, 64, 3000, 1], [901, 2101, 65, 3001, 2]        # the next step: every sequence one longer
    da, db = W.decode_inputs(ctx_a, seed=41), W.decode_inputs(ctx_b, seed=41)
    g = W.to_device(da, gpu)
    kw = dict(cache_seqlens=g["cache_seqlens"], block_table=g["block_table"], softmax_scale=da["scale"], causal=True)
    hip(g["q"], g["k_cache"], g["v_cache"], **kw)                                     # step t, layer 0: plans
    hip(g["q"], g["k_cache"], g["v_cache"], reuse_plan=True, **kw)                    # step t, layer 1
    gb = W.to_device(db, gpu)
    assert gb["block_table"].shape == g["block_table"].shape
    g["cache_seqlens"].copy_(gb["cache_seqlens"])                                     # in place: same addresses
    g["block_table"].copy_(gb["block_table"])
    got0 = hip(gb["q"], gb["k_cache"], gb["v_cache"], **kw)                           # step t+1, layer 0: plans again
    got1 = hip(gb["q"], gb["k_cache"], gb["v_cache"], reuse_plan=True, **kw)          # step t+1, layer 1: reuses
    want = ref(db["q"], db["k_cache"], db["v_cache"], cache_seqlens=db["cache_seqlens"], block_table=db["block_table"],
               softmax_scale=db["scale"], causal=True)
    assert_attention_close(got0, want, "decode after an in-place rewrite of the lengths, planned again")
    assert_bit_exact(got1, got0, "the next layer on the renewed plan")


def test_kernels_refuse_a_plan_made_for_another_launch(gpu):
    """Through the C ABI, where nothing tracks the plan: MOPS_HIP_DECODE_REUSE_PLAN on a workspace that was never
    planned, or was planned for a larger batch, must not follow the stale sequence indices.  The kernels compare the
    plan's recorded batch and head geometry with their own launch and write zero rows instead."""
    from nano_vllm_ninetoothed_amd import _capi
    lib = _capi.load()
    stream = torch.cuda.current_stream(gpu).cuda_stream
    big = W.to_device(W.decode_inputs(W.random_seq_lens(64, 1, 2000, seed=33), seed=33), gpu)
    small = W.to_device(W.decode_inputs([500, 900, 40], seed=34), gpu)

    def call(g, ws, mode):
        q, kc, bt = g["q"], g["k_cache"], g["block_table"]
        out = torch.full_like(q, float("nan"))
        st = lib.mops_hip_attn_paged_decode_planned_bf16(
            q.data_ptr(), q.stride(0), kc.data_ptr(), g["v_cache"].data_ptr(), g["cache_seqlens"].data_ptr(), bt.data_ptr(),
            bt.stride(0), out.data_ptr(), q.shape[0], q.shape[2], kc.shape[2], 128, kc.shape[1], kc.shape[0], bt.shape[1],
            g["scale"], ws.data_ptr(), ws.numel(), mode, stream)
        _capi.check("mops_hip_attn_paged_decode_planned_bf16", st)
        torch.cuda.synchronize()
        return out

    nbytes = lib.mops_hip_paged_decode_workspace_bytes(64, 16, 8, 16, 256)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=gpu)
    assert (call(small, ws, 1).float() == 0).all(), "never planned"
    want_small = call(small, ws.clone(), 0)
    call(big, ws, 0)                                                   # plan for 64 sequences
    assert (call(small, ws, 1).float() == 0).all(), "planned for a larger batch"
    assert_bit_exact(call(small, ws, 0), want_small, "planning afresh on the used workspace")
