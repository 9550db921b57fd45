"""GPU parity for varlen causal prefill attention (flash_attn_varlen_func) through the hip backend.

Tolerance: max-abs 2e-2, mean-abs 2e-3 against the fp32 oracle (bf16 inputs/outputs, fp32 accumulate)."""
import pytest
import torch

from helpers import assert_attention_close, assert_bit_exact
from nano_vllm_ninetoothed_amd import workloads as W

pytestmark = pytest.mark.gpu


def _run(hip, d, gpu, **over):
    g = W.to_device(d, gpu)
    kw = dict(max_seqlen_q=d["max_seqlen"], cu_seqlens_q=g["cu_seqlens"], max_seqlen_k=d["max_seqlen"],
              cu_seqlens_k=g["cu_seqlens"], softmax_scale=d["scale"], causal=True, block_table=None)
    kw.update(over)
    return hip(g["q"], g["k"], g["v"], **kw)


def _ref(ref, d):
    return ref(d["q"], d["k"], d["v"], max_seqlen_q=d["max_seqlen"], cu_seqlens_q=d["cu_seqlens"],
               max_seqlen_k=d["max_seqlen"], cu_seqlens_k=d["cu_seqlens"], softmax_scale=d["scale"], causal=True)


@pytest.mark.parametrize("lens,hq,hkv", [
    ([256, 256], 16, 8), ([1], 16, 8), ([1, 1, 1], 16, 8), ([5], 16, 8), ([63, 64, 65], 16, 8),
    ([127, 128, 129], 16, 8), ([300, 1, 77, 513], 16, 8), ([1000], 32, 8), ([200, 345], 8, 8),
    ([130, 70], 8, 1), ([2048], 16, 8)])
def test_prefill_matches_oracle(gpu, ops, lens, hq, hkv):
    hip, ref = ops("flash_attn_varlen_func")
    d = W.prefill_inputs(lens, hq=hq, hkv=hkv, seed=sum(lens) + hq)
    got = _run(hip, d, gpu)
    assert got.shape == d["q"].shape and got.dtype == torch.bfloat16
    assert_attention_close(got, _ref(ref, d), f"prefill lens={lens} {hq}:{hkv}")


@pytest.mark.parametrize("scale,qmul", [(0.25, 1.0), (0.0, 1.0), (0.02, 30.0), (-0.0884, 1.0), (0.0884, 4.0), (1.0, 1.0)])
def test_prefill_other_scales_and_large_scores(gpu, ops, scale, qmul):
    """The scale is applied in fp32 to the fp32 scores, as the reference does (mops/triton/attention.py:83), so the error
    does not grow with the size of the scores; the softmax reference is folded into the accumulator the score MFMAs start
    from and moves only when a row maximum outgrows it by 2^8.  Scale 1 on N(0,1) data gives scores of +-40 in the
    exponent's units (the reference moves again and again, probabilities collapse onto a few keys, outputs reach 4 and
    their bf16 ulp 0.031), scale 0 a uniform softmax, a negative scale turns the order of the scores around."""
    hip, ref = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([333, 64, 700], seed=17)
    d["q"] = (d["q"].float() * qmul).to(torch.bfloat16)
    d["scale"] = scale
    got = _run(hip, d, gpu).float().cpu()
    want = _ref(ref, d).float()
    assert torch.isfinite(got).all()
    diff = (got - want).abs()
    assert diff.max().item() <= (4e-2 if scale == 1.0 else 2e-2), f"scale {scale}, q x {qmul}: max-abs {diff.max().item():.4g}"
    assert diff.mean().item() <= 2e-3, f"scale {scale}, q x {qmul}: mean-abs {diff.mean().item():.4g}"


def test_prefill_prescaled_q_form_meets_the_benchmark_tolerance(gpu):
    """MOPS_HIP_PREFILL_PRESCALE=1 (read once per process, hence the child process) selects the form that multiplies Q by
    scale * log2(e) once and rounds it back to bf16: faster, and within the benchmark's tolerance on the benchmark's
    inputs, but its error grows with the size of the scores (the figures at four times the benchmark's Q are printed)."""
    import os, subprocess, sys
    code = r'''
import sys, torch
sys.path.insert(0, ".")
from nano_vllm_ninetoothed_amd import mops, workloads as W
import oracle.mops_torch
dev = torch.device("cuda:%d")
hip = mops.get_op("flash_attn_varlen_func", "hip"); ref = mops.get_op("flash_attn_varlen_func", "torch")
for qmul in (1.0, 4.0):
    d = W.prefill_inputs([333, 64, 700], seed=17)
    d["q"] = (d["q"].float() * qmul).to(torch.bfloat16)
    g = W.to_device(d, dev)
    o = hip(g["q"], g["k"], g["v"], max_seqlen_q=d["max_seqlen"], cu_seqlens_q=g["cu_seqlens"], max_seqlen_k=d["max_seqlen"],
            cu_seqlens_k=g["cu_seqlens"], softmax_scale=d["scale"], causal=True).cpu().float()
    w = ref(d["q"], d["k"], d["v"], max_seqlen_q=d["max_seqlen"], cu_seqlens_q=d["cu_seqlens"], softmax_scale=d["scale"]).float()
    e = (o - w).abs()
    print(qmul, float(e.max()), float(e.mean()))
''' % (gpu.index or 0)
    env = dict(os.environ, MOPS_HIP_PREFILL_PRESCALE="1")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, capture_output=True, text=True, timeout=150)
    assert out.returncode == 0, out.stderr[-2000:]
    rows = [l.split() for l in out.stdout.strip().splitlines()[-2:]]
    (q1, max1, mean1), (q4, max4, mean4) = [(float(a), float(b), float(c)) for a, b, c in rows]
    assert (q1, q4) == (1.0, 4.0)
    assert max1 <= 2e-2 and mean1 <= 2e-3, (max1, mean1)
    print(f"pre-scaled Q form: mean-abs {mean1:.3g} at the benchmark's Q, {mean4:.3g} at four times it (max-abs {max4:.3g})")


def test_prefill_row_form_still_matches_oracle(gpu):
    """Causal prefill over grouped heads takes the two-heads-per-wave form (varlen_prefill_pair.hip); the 128-row form
    stays the path of odd group sizes, very large batches and block tables too large for LDS.  MOPS_HIP_PREFILL_FORM=rows
    (read once per process, hence the child process) forces it for every input, so that its ragged and rectangular
    launches and its paged and packed cached-prefix paths stay covered against the oracle."""
    import os, subprocess, sys
    code = r'''
import sys, torch
sys.path.insert(0, ".")
from nano_vllm_ninetoothed_amd import mops, workloads as W
import oracle.mops_torch
dev = torch.device("cuda:%d")
hip = mops.get_op("flash_attn_varlen_func", "hip"); ref = mops.get_op("flash_attn_varlen_func", "torch")
for lens in ([300, 1, 77, 513], [256, 256], [2048], [0, 31, 700, 64, 65, 1, 129] * 3):
    d = W.prefill_inputs(lens, seed=sum(lens))
    g = W.to_device(d, dev)
    o = hip(g["q"], g["k"], g["v"], max_seqlen_q=d["max_seqlen"], cu_seqlens_q=g["cu_seqlens"], max_seqlen_k=d["max_seqlen"],
            cu_seqlens_k=g["cu_seqlens"], softmax_scale=d["scale"], causal=True).cpu().float()
    w = ref(d["q"], d["k"], d["v"], max_seqlen_q=d["max_seqlen"], cu_seqlens_q=d["cu_seqlens"], softmax_scale=d["scale"]).float()
    e = (o - w).abs()
    print(len(lens), float(e.max()), float(e.mean()))
for new, prefix in (([100, 200], [256, 512]), ([300, 17, 129], [0, 256, 768]), ([1, 1, 1], [256, 1, 1023]), ([200], [17000])):
    d = W.prefix_prefill_inputs(new, prefix, seed=sum(new) + sum(prefix))
    g = W.to_device(d, dev)
    w = ref(d["q"], torch.nan_to_num(d["k_cache"]), torch.nan_to_num(d["v_cache"]), max_seqlen_q=d["max_seqlen_q"],
            cu_seqlens_q=d["cu_seqlens_q"], max_seqlen_k=d["max_seqlen_k"], cu_seqlens_k=d["cu_seqlens_k"],
            softmax_scale=d["scale"], causal=True, block_table=d["block_table"]).float()
    for paged in (True, False):
        k, v = (g["k_cache"], g["v_cache"]) if paged else (g["k_all"], g["v_all"])
        o = hip(g["q"], k, v, max_seqlen_q=d["max_seqlen_q"], cu_seqlens_q=g["cu_seqlens_q"], max_seqlen_k=d["max_seqlen_k"],
                cu_seqlens_k=g["cu_seqlens_k"], softmax_scale=d["scale"], causal=True, block_table=g["block_table"] if paged else None).cpu().float()
        e = (o - w).abs()
        print(len(new), float(e.max()), float(e.mean()))
''' % (gpu.index or 0)
    env = dict(os.environ, MOPS_HIP_PREFILL_FORM="rows")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, capture_output=True, text=True, timeout=150)
    assert out.returncode == 0, out.stderr[-2000:]
    rows = [l.split() for l in out.stdout.strip().splitlines()[-12:]]
    assert len(rows) == 12
    for n, mx, mean in rows:
        assert float(mx) <= 2e-2 and float(mean) <= 2e-3, (n, mx, mean)


@pytest.mark.parametrize("nseq", [70, 200, 300])
def test_prefill_many_ragged_sequences(gpu, ops, nseq):
    """Ragged batches launch workgroups for existing q tiles only (up to 256 sequences; sequence index found
    inside the kernel from per-lane tile counts, one 64-sequence chunk per register), larger batches use the
    plain tile x sequence rectangle.  Lengths include empty sequences and one long straggler."""
    hip, ref = ops("flash_attn_varlen_func")
    gen = torch.Generator().manual_seed(nseq)
    lens = torch.randint(0, 260, (nseq,), generator=gen).tolist()
    lens[nseq // 2] = 700
    lens[3] = 0
    d = W.prefill_inputs(lens, seed=nseq)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), f"prefill {nseq} ragged sequences")


def test_prefill_more_sequences_than_the_resident_form_holds(gpu, ops):
    """Beyond 512 sequences the launch falls back to the 128-row form and its tile x sequence rectangle."""
    hip, ref = ops("flash_attn_varlen_func")
    gen = torch.Generator().manual_seed(600)
    lens = torch.randint(0, 70, (600,), generator=gen).tolist()
    lens[17] = 300
    d = W.prefill_inputs(lens, hq=4, hkv=2, seed=600)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), "prefill 600 short sequences")


def test_prefill_items_of_a_single_tile(gpu, ops):
    """Sequences shorter than 64 tokens only: every work item of the resident form is a single K/V tile, so every draw of
    the next item is waited for inside the item (the path with one more barrier), and every first tile is a partial one."""
    hip, ref = ops("flash_attn_varlen_func")
    gen = torch.Generator().manual_seed(5)
    lens = torch.randint(1, 64, (400,), generator=gen).tolist()
    d = W.prefill_inputs(lens, seed=5)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), "400 sequences of fewer than 64 tokens")


def test_prefill_counter_rows_wrap_and_streams_overlap(gpu, ops):
    """The resident form hands out work items through counters in device memory, one row of counters per launch, rows used
    round robin (128 of them) and cleared by the last workgroup of a launch.  More launches than rows, then launches that
    overlap on two streams: every result has the bits of the first launch."""
    hip, _ = ops("flash_attn_varlen_func")
    a = W.prefill_inputs([200, 64, 1, 333], seed=3)
    b = W.prefill_inputs([129, 700], seed=4)
    first_a, first_b = _run(hip, a, gpu).clone(), _run(hip, b, gpu).clone()
    for i in range(300):
        assert_bit_exact(_run(hip, a, gpu), first_a, f"launch {i}")
    s1, s2 = torch.cuda.Stream(gpu), torch.cuda.Stream(gpu)
    torch.cuda.synchronize()
    outs = []
    for _ in range(20):
        with torch.cuda.stream(s1):
            outs.append((_run(hip, a, gpu), first_a))
        with torch.cuda.stream(s2):
            outs.append((_run(hip, b, gpu), first_b))
    torch.cuda.synchronize()
    for i, (got, want) in enumerate(outs):
        assert_bit_exact(got, want, f"overlapping launch {i}")


def test_prefill_ragged_batch_with_a_very_long_sequence(gpu, ops):
    """More than 64 q tiles in the longest sequence: the rank -> (tile, sequence) mapping of the compact
    launch takes its search form instead of the one-ballot form.  Two query heads keep the oracle quick."""
    hip, ref = ops("flash_attn_varlen_func")
    lens = [150, 8400, 0, 64, 129, 1]
    d = W.prefill_inputs(lens, hq=2, hkv=1, seed=84)
    want = _ref(ref, d)
    assert_attention_close(_run(hip, d, gpu), want, "ragged batch with an 8400-token sequence")
    # and the same lengths when max_seqlen_q is a loose bound (more tile indices than any sequence has)
    assert_attention_close(_run(hip, d, gpu, max_seqlen_q=16384), want, "same, max_seqlen_q = 16384")


def test_prefill_v_is_strided_view_and_max_seqlen_is_only_a_bound(gpu, ops):
    """q, k, v as nanovllm hands them: slices of one [T, 4096] qkv buffer (row stride 4096)."""
    hip, ref = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([190, 333], seed=21)
    T = 523
    qkv = torch.cat([d["q"].view(T, -1), d["k"].view(T, -1), d["v"].view(T, -1)], dim=1).to(gpu)
    q, k, v = qkv.split([2048, 1024, 1024], dim=-1)
    cu = d["cu_seqlens"].to(gpu)
    got = hip(q.view(T, 16, 128), k.view(T, 8, 128), v.view(T, 8, 128), max_seqlen_q=4096, cu_seqlens_q=cu,
              max_seqlen_k=4096, cu_seqlens_k=cu, softmax_scale=d["scale"], causal=True, block_table=None)
    assert got.is_contiguous()
    assert_attention_close(got, _ref(ref, d), "strided qkv views")


def test_prefill_sequences_do_not_leak_into_each_other(gpu, ops):
    """Changing sequence 1 must not change sequence 0's output bits; NaN in a later sequence stays there."""
    hip, _ = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([100, 150, 60], seed=23)
    base = _run(hip, d, gpu).cpu()
    d2 = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in d.items()}
    d2["k"][100:250] = float("nan")
    d2["v"][100:250] = float("nan")
    got = _run(hip, d2, gpu).cpu()
    assert_bit_exact(got[:100], base[:100], "sequence 0")
    assert_bit_exact(got[250:], base[250:], "sequence 2")


def test_prefill_first_token_returns_v_and_constant_v(gpu, ops):
    hip, _ = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([40, 300], seed=25)
    d["v"][40:] = -1.25
    got = _run(hip, d, gpu).cpu()
    assert_bit_exact(got[0], d["v"][0].repeat_interleave(2, dim=0), "row 0 sees only key 0")
    assert (got[40:].float() == -1.25).all()


def test_prefill_empty_sequence_in_batch_and_no_tokens(gpu, ops):
    hip, ref = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([70, 0, 130], seed=27)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), "batch with an empty sequence")
    e = torch.empty((0, 16, 128), dtype=torch.bfloat16, device=gpu)
    ek = torch.empty((0, 8, 128), dtype=torch.bfloat16, device=gpu)
    cu = torch.zeros(1, dtype=torch.int32, device=gpu)
    out = hip(e, ek, ek, max_seqlen_q=0, cu_seqlens_q=cu, max_seqlen_k=0, cu_seqlens_k=cu, softmax_scale=1.0, causal=True)
    assert out.shape == (0, 16, 128)


def test_prefill_rejects_non_causal(gpu, ops):
    hip, _ = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([32], seed=29)
    with pytest.raises(ValueError):
        _run(hip, d, gpu, causal=False)


def _run_prefix(op, d, dev, paged=True):
    g = W.to_device(d, dev) if dev is not None else d
    k, v = (g["k_cache"], g["v_cache"]) if paged else (g["k_all"], g["v_all"])
    return op(g["q"], k, v, max_seqlen_q=d["max_seqlen_q"], cu_seqlens_q=g["cu_seqlens_q"], max_seqlen_k=d["max_seqlen_k"],
              cu_seqlens_k=g["cu_seqlens_k"], softmax_scale=d["scale"], causal=True, block_table=g["block_table"] if paged else None)


@pytest.mark.parametrize("new,prefix,hq,hkv", [
    ([100, 200], [256, 512], 16, 8), ([1, 1, 1], [256, 1, 1023], 16, 8), ([300, 17, 129], [0, 256, 768], 16, 8),
    ([64, 65], [63, 700], 32, 8), ([513], [1024], 8, 8), ([250, 5], [300, 2000], 8, 1)])
def test_prefill_with_cached_prefix_matches_oracle(gpu, ops, new, prefix, hq, hkv):
    """Prefix-cache hit (nanovllm/layers/attention.py:32-33 of the reference): k/v are the paged caches, keys
    are addressed through block_table, causal mask aligned bottom-right; unused cache rows are NaN."""
    hip, ref = ops("flash_attn_varlen_func")
    d = W.prefix_prefill_inputs(new, prefix, hq=hq, hkv=hkv, seed=sum(new) + sum(prefix))
    want = ref(d["q"], torch.nan_to_num(d["k_cache"]), torch.nan_to_num(d["v_cache"]), max_seqlen_q=d["max_seqlen_q"],
               cu_seqlens_q=d["cu_seqlens_q"], max_seqlen_k=d["max_seqlen_k"], cu_seqlens_k=d["cu_seqlens_k"],
               softmax_scale=d["scale"], causal=True, block_table=d["block_table"])
    got = _run_prefix(hip, d, gpu, paged=True)
    assert_attention_close(got, want, f"paged prefix prefill new={new} prefix={prefix}")
    got_packed = _run_prefix(hip, d, gpu, paged=False)       # same keys handed over packed, with cu_seqlens_k
    assert_bit_exact(got_packed, got, "packed keys with cu_seqlens_k vs paged keys")


@pytest.mark.parametrize("block_size,new,prefix", [
    (64, [300, 70], [200, 1000]), (128, [129, 640], [127, 900]), (512, [700], [1500]),
    (64, [200], [4300]),     # 71 cache blocks: more than the 64 table entries a wave keeps in registers
    (256, [500, 300], [16500, 100])])
def test_prefill_with_cached_prefix_other_block_sizes_and_long_tables(gpu, ops, monkeypatch, block_size, new, prefix):
    """The steady part of the tile loop steps through a cache block tile by tile and takes the next block's table entry
    from a register (up to 64 blocks per sequence); other block sizes change how many tiles a block holds, and
    sequences with more blocks take the general loop for every tile."""
    hip, ref = ops("flash_attn_varlen_func")
    monkeypatch.setattr(W, "BLOCK_SIZE", block_size)
    d = W.prefix_prefill_inputs(new, prefix, hq=4, hkv=2, seed=block_size + sum(new))
    assert d["k_cache"].shape[1] == block_size
    want = ref(d["q"], torch.nan_to_num(d["k_cache"]), torch.nan_to_num(d["v_cache"]), max_seqlen_q=d["max_seqlen_q"],
               cu_seqlens_q=d["cu_seqlens_q"], max_seqlen_k=d["max_seqlen_k"], cu_seqlens_k=d["cu_seqlens_k"],
               softmax_scale=d["scale"], causal=True, block_table=d["block_table"])
    got = _run_prefix(hip, d, gpu, paged=True)
    assert_attention_close(got, want, f"paged prefix prefill, block size {block_size}, new={new} prefix={prefix}")
    assert_bit_exact(_run_prefix(hip, d, gpu, paged=False), got, "packed keys with cu_seqlens_k vs paged keys")


def test_prefix_prefill_with_a_block_table_too_large_for_the_resident_form(gpu, ops):
    """The two-heads-per-wave form keeps the block table in LDS (768 entries); 40 sequences x 24 blocks do not fit and go
    to the 128-row form, as do more than 64 sequences with a prefix."""
    hip, ref = ops("flash_attn_varlen_func")
    for new, prefix in (([20, 70] * 20, [6000, 300] * 20), ([5] * 70, [300] * 70)):
        d = W.prefix_prefill_inputs(new, prefix, hq=4, hkv=2, seed=len(new))
        assert len(new) > 64 or d["block_table"].numel() > 768
        want = ref(d["q"], torch.nan_to_num(d["k_cache"]), torch.nan_to_num(d["v_cache"]), max_seqlen_q=d["max_seqlen_q"],
                   cu_seqlens_q=d["cu_seqlens_q"], max_seqlen_k=d["max_seqlen_k"], cu_seqlens_k=d["cu_seqlens_k"],
                   softmax_scale=d["scale"], causal=True, block_table=d["block_table"])
        assert_attention_close(_run_prefix(hip, d, gpu, paged=True), want, f"paged prefix prefill, {len(new)} sequences")


def test_prefix_prefill_sequence_without_keys_gives_zeros(gpu, ops):
    """cu_seqlens_k may give a sequence no keys at all, or fewer keys than queries (rows whose horizon lies before key 0
    see nothing): such rows come out as zeros, the other sequences are not disturbed."""
    hip, ref = ops("flash_attn_varlen_func")
    d = W.prefix_prefill_inputs([50, 100, 70], [0, 200, 0], seed=77)
    g = W.to_device(d, gpu)
    # sequence 0 keeps no keys; sequence 2 keeps 30 keys for its 70 queries: rows 0..39 see nothing, row 40 + i sees keys 0..i
    cu_k = torch.tensor([0, 0, 300, 330], dtype=torch.int32)
    got = hip(g["q"], g["k_all"][50:], g["v_all"][50:], max_seqlen_q=100, cu_seqlens_q=g["cu_seqlens_q"], max_seqlen_k=300,
              cu_seqlens_k=cu_k.to(gpu), softmax_scale=d["scale"], causal=True).cpu()
    assert torch.isfinite(got.float()).all()
    assert (got[:50] == 0).all() and (got[150:190] == 0).all()
    want1 = ref(d["q"][50:150], d["k_all"][50:350], d["v_all"][50:350], max_seqlen_q=100, cu_seqlens_q=torch.tensor([0, 100], dtype=torch.int32),
                max_seqlen_k=300, cu_seqlens_k=torch.tensor([0, 300], dtype=torch.int32), softmax_scale=d["scale"], causal=True)
    assert_attention_close(got[50:150], want1, "sequence between two sequences without visible keys")
    want2 = ref(d["q"][190:220], d["k_all"][350:380], d["v_all"][350:380], max_seqlen_q=30, cu_seqlens_q=torch.tensor([0, 30], dtype=torch.int32),
                max_seqlen_k=30, cu_seqlens_k=torch.tensor([0, 30], dtype=torch.int32), softmax_scale=d["scale"], causal=True)
    assert_attention_close(got[190:220], want2, "the rows of a sequence with fewer keys than queries that do see keys")


def test_prefix_prefill_treats_a_missing_block_as_empty(gpu, ops):
    """A block_table entry outside [0, num_blocks) inside the used range: the keys of that block get no weight (the
    rule paged decode follows for the same metadata), instead of entering the softmax with score 0."""
    hip, _ = ops("flash_attn_varlen_func")
    d = W.prefix_prefill_inputs([100, 300], [512, 300], seed=12)
    table = d["block_table"].clone()
    table[0, 1] = -1                      # keys 256..511 of sequence 0 (inside its cached prefix)
    table[1, 0] = d["k_cache"].shape[0]   # keys 0..255 of sequence 1: one past the last block
    g = W.to_device(d, gpu)
    got = hip(g["q"], g["k_cache"], g["v_cache"], max_seqlen_q=d["max_seqlen_q"], cu_seqlens_q=g["cu_seqlens_q"],
              max_seqlen_k=d["max_seqlen_k"], cu_seqlens_k=g["cu_seqlens_k"], softmax_scale=d["scale"], causal=True,
              block_table=table.to(gpu))
    cq, ck = d["cu_seqlens_q"].tolist(), d["cu_seqlens_k"].tolist()
    want = torch.zeros_like(d["q"])
    for s, dead in ((0, range(256, 512)), (1, range(0, 256))):
        q = d["q"][cq[s]:cq[s + 1]].float().transpose(0, 1)                                    # [Hq, Lq, D]
        k = d["k_all"][ck[s]:ck[s + 1]].float().transpose(0, 1).repeat_interleave(2, dim=0)  # [Hq, Lk, D]
        v = d["v_all"][ck[s]:ck[s + 1]].float().transpose(0, 1).repeat_interleave(2, dim=0)
        lq, lk = q.shape[1], k.shape[1]
        scores = q @ k.transpose(1, 2) * d["scale"]
        i, j = torch.arange(lq).unsqueeze(1), torch.arange(lk).unsqueeze(0)
        hidden = (j > i + (lk - lq)) | torch.isin(j, torch.tensor(list(dead)))
        want[cq[s]:cq[s + 1]] = (torch.softmax(scores.masked_fill(hidden, float("-inf")), -1) @ v).transpose(0, 1).to(torch.bfloat16)
    assert_attention_close(got, want, "prefix prefill with two missing blocks")


def test_prefill_is_bitwise_reproducible(gpu, ops):
    """The same launch repeated gives the same bits (plain, packed-with-prefix and paged inputs).  Guards the
    kernel's hand-placed instruction order: a VALU read of an MFMA result that comes too early returns
    a mix of old and new register contents, which shows up as run-to-run differences of an ulp."""
    hip, _ = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([700, 130, 1025], seed=91)
    first = _run(hip, d, gpu).clone()
    for _ in range(30):
        assert_bit_exact(_run(hip, d, gpu), first, "plain prefill, repeated launch")
    dp = W.prefix_prefill_inputs([513, 100], [1024, 256], hq=16, hkv=8, seed=92)
    for paged in (True, False):
        first = _run_prefix(hip, dp, gpu, paged=paged).clone()
        for _ in range(30):
            assert_bit_exact(_run_prefix(hip, dp, gpu, paged=paged), first, f"prefix prefill paged={paged}, repeated launch")


def test_prefix_prefill_last_row_equals_decode(gpu, ops):
    pre, _ = ops("flash_attn_varlen_func")
    dec, _ = ops("flash_attn_with_kvcache")
    d = W.prefix_prefill_inputs([40, 7], [512, 300], seed=33, poison_unused=False)
    g = W.to_device(d, gpu)
    o = _run_prefix(pre, d, gpu)
    last = (d["cu_seqlens_q"][1:] - 1).long()
    lens = (d["cu_seqlens_k"][1:] - d["cu_seqlens_k"][:-1]).to(torch.int32)
    od = dec(g["q"][last.to(gpu)].unsqueeze(1), g["k_cache"], g["v_cache"], cache_seqlens=lens.to(gpu), block_table=g["block_table"],
             softmax_scale=d["scale"], causal=True)
    assert_attention_close(od[:, 0], o[last.to(gpu)], "last new token vs a decode step over the same cache")


def test_prefill_warmup_shape(gpu, ops):
    """The engine's warm-up batch: 4 sequences of 4096 tokens (model_runner.py:94-97 of the reference);
    checked on sampled rows against the oracle."""
    hip, ref = ops("flash_attn_varlen_func")
    d = W.prefill_inputs([4096] * 4, seed=31)
    got = _run(hip, d, gpu).cpu()
    assert torch.isfinite(got.float()).all()
    rows = [0, 1, 127, 128, 4095, 4096, 4096 + 2047, 3 * 4096 + 4095]
    from oracle.bruteforce import attention_row  # fp64 definition, row by row
    import numpy as np
    for r in rows:
        s, i = divmod(r, 4096)
        lo = s * 4096
        for h in (0, 15):
            want = attention_row(d["q"][r, h].float().numpy(), d["k"][lo:lo + i + 1, h // 2].float().numpy(),
                                 d["v"][lo:lo + i + 1, h // 2].float().numpy(), d["scale"]) if i < 300 else None
            if want is not None:
                assert np.abs(got[r, h].float().numpy() - want).max() <= 2e-2
    one = {"q": d["q"][:4096], "k": d["k"][:4096], "v": d["v"][:4096], "cu_seqlens": torch.tensor([0, 4096], dtype=torch.int32),
           "max_seqlen": 4096, "scale": d["scale"]}
    assert_attention_close(got[:4096], _ref(ref, one), "first warm-up sequence")


def test_prefill_full_size_config(gpu, ops):
    """Benchmark-size batch: 16 sequences, lengths uniform in [128, 2048]; whole output vs the oracle."""
    hip, ref = ops("flash_attn_varlen_func")
    lens = W.random_seq_lens(16, 128, 2048, seed=0)
    d = W.prefill_inputs(lens, seed=0)
    assert_attention_close(_run(hip, d, gpu), _ref(ref, d), "cfg2")
