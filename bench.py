#!/usr/bin/env python3
"""Benchmark of the mops `hip` backend on one MI355X.

Default run = the headline workload: paged decode attention at Qwen3-0.6B shape (256 sequences, one
query token each, 16 q heads / 8 kv heads, head_dim 128, context uniform in [512, 4096], block 256).
A step is one flash_attn_with_kvcache call over the whole batch, KV cache resident in HBM.
`--op` selects another operator of the hot path (same JSON format, its own metric):
  decode (default) | decode8b | prefill | store | add_rms | rms | embedding
  e2e  = end-to-end generation on a randomly initialised Qwen3-0.6B-shaped model through the engine
         counterpart (256 random-token prompts of 100..1024 tokens, 100..1024 output tokens each,
         temperature 0.6, no EOS): output tokens per second; --steps/--warmup are ignored.
  copy = a plain 1 GiB device-to-device tensor copy (not a mops op): the known-size kernel against which
         the FETCH_SIZE / WRITE_SIZE counters of a profile are calibrated.
  launch_floor = an empty kernel: the floor under the durations of the small operators (value 0, read the time).

The default line also carries an `e2e` block: the cfg5 workload's output tok/s in three modes (eager with per-step
readback, which is the reference's own setting; the decode step replayed from HIP graphs with per-step readback; the
same pipelined) and the same engine on the torch-restated backend on a reduced run (--no-e2e skips the block).

Prints ONE JSON line on stdout.  `roofline` is computed from HIP-event time of the op on its launch
stream; `cpu_baseline` times the CPU restatement of the reference's torch backend (oracle/) on a
bounded sample of the same workload on this machine's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
TRAFFIC_PROFILE = "profiles/hbm_traffic_decode_prefill.txt"


def profiled_traffic(section):
    """HBM-side bytes per launch of a workload ("decode", "prefill", "prefill_long") as the committed rocprofv3 --pmc
    summary states them (FETCH_SIZE + WRITE_SIZE, calibrated against a 1 GiB copy): the "total per launch" line of that
    section.  Returns (bytes, source) or (None, reason): the figure is read, never re-typed, and it is a figure of that
    profile, not of this run."""
    import re
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), TRAFFIC_PROFILE)
    try:
        text = open(path).read()
    except OSError:
        return None, f"{TRAFFIC_PROFILE} not found"
    m = re.search(r"^%s:\n(?:  .*\n)*?  total per launch: ([0-9.]+) MB" % re.escape(section), text, re.M)
    if not m:
        return None, f"no section '{section}' with a 'total per launch' line in {TRAFFIC_PROFILE}"
    return float(m.group(1)) * 1e6, f"{TRAFFIC_PROFILE}, section '{section}' (rocprofv3 --pmc, not measured by this run)"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 50; 500 for the prefill ops)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed warm-up steps (default 10; 300 for the prefill ops)")
    ap.add_argument("--op", default="decode",
                    choices=["decode", "decode8b", "prefill", "prefill_long", "prefix_prefill", "prefix_prefill_short", "store", "silu", "sampler", "qk_rope_store", "add_rms", "rms", "embedding", "copy", "launch_floor", "e2e"])
    ap.add_argument("--e2e-seqs", type=int, default=256, help="number of prompts of the e2e workload")
    ap.add_argument("--e2e-eager", action="store_true", help="e2e: no HIP-graph replay of the decode step")
    ap.add_argument("--e2e-stepwise", action="store_true", help="e2e: read every step's tokens back before the next step, as the reference does")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-e2e", action="store_true", help="default op only: skip the end-to-end block of the line (profiling runs)")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()
    # The prefill kernels keep the matrix pipes of all CUs busy, and the chip's power management answers the step from idle
    # to that load with a transient: launches 10..150 of a back-to-back series run up to 40 % slower than the first ten
    # and than everything after launch 250.  The warm-up of these ops is long enough to sit the transient out, and the
    # timed series long enough not to be dominated by what is left of it.
    matrix_bound = args.op in ("prefill", "prefill_long", "prefix_prefill", "prefix_prefill_short")
    if args.steps is None:
        args.steps = 500 if matrix_bound else 50
    if args.warmup is None:
        args.warmup = 300 if matrix_bound else 10
    return args


def e2e_workload(n):
    """Prompts and output lengths of the reference's bench.py:9-28 (random.seed(0), token ids 0..10000)."""
    import random
    random.seed(0)
    prompts = [[random.randint(0, 10000) for _ in range(random.randint(100, 1024))] for _ in range(n)]
    max_tokens = [random.randint(100, 1024) for _ in range(n)]
    return prompts, max_tokens


def e2e_modes(args, torch, modes):
    """Runs the e2e workload once per mode on one engine (random-init Qwen3-0.6B architecture, hip backend).
    Modes: "pipelined" (decode step replayed from HIP graphs, sampled tokens kept on the device and read back once
    at the end), "stepwise" (graphs, every step's tokens read back before the next step is scheduled, as
    nanovllm/engine/model_runner.py:212 does), "eager" (no graphs, per-step readback: the reference's
    enforce_eager=True setting, bench.py:15).  Returns {mode: {...}} in the order given."""
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    n = args.e2e_seqs
    prompts, max_tokens = e2e_workload(n)
    total = sum(max_tokens)
    eng = Engine(Qwen3Shape(), backend="hip", num_blocks=max(64, n * 10), seed=args.seed)
    eng.generate([[1, 2, 3, 4, 5, 6, 7, 8]], 8)                 # warm-up, as the reference does
    res = {}
    for mode in sorted(modes, key=lambda m: m != "eager"):       # eager first: it must run before graphs exist
        if mode != "eager" and not eng.graphs:
            eng.capture_decode_graphs(max_bs=min(512, max(16, (n + 15) // 16 * 16)), max_model_len=4096)
        eng.pipelined = mode == "pipelined"
        _, st = eng.generate(prompts, max_tokens, temperature=0.6)
        assert not eng.running and not eng.waiting and len(eng.free_blocks) == eng.num_blocks
        res[mode] = {"mode": mode, "tok_per_s": round(total / st["total_s"], 1), "output_tokens": total,
                     "seconds": round(st["total_s"], 3), "prompt_tokens": sum(len(p) for p in prompts),
                     "prefill_steps": st["prefill_steps"], "decode_steps": st["decode_steps"],
                     "prefill_tok_per_s": round(st["prefill_tokens"] / max(st["prefill_s"], 1e-9), 1),
                     "decode_tok_per_s": round(st["decode_tokens"] / max(st["decode_s"], 1e-9), 1)}
    del eng
    torch.cuda.empty_cache()
    return {m: res[m] for m in modes}


def e2e_comparison(args, torch, prompts, m=32, outlen=32):
    """The same engine on the same GPU with the mops ops of the pure-torch restatement of the reference's torch backend,
    next to the hip backend, on a reduced run (first m prompts, outlen output tokens each, no graphs).  It stands in for
    the comparison the reference cannot offer: its triton backend has no decode attention (mops/triton/attention.py:150-168)."""
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    import oracle.mops_torch  # noqa: F401  comparison backend only
    res = {}
    for backend in ("hip", "torch"):
        e = Engine(Qwen3Shape(), backend=backend, num_blocks=m * 6, seed=args.seed)
        e.generate([[1, 2, 3, 4, 5, 6, 7, 8]], 4)
        _, s2 = e.generate(prompts[:m], outlen, temperature=0.6)
        res[backend] = m * outlen / s2["total_s"]
        del e
        torch.cuda.empty_cache()
    return {"what": "same engine, same GPU, no graphs, mops ops from the pure-torch restatement of the reference's torch backend "
                    "(per-sequence attention loops) against the hip backend",
            "sample": f"first {m} prompts, {outlen} output tokens each",
            "hip_tok_per_s": round(res["hip"], 1), "torch_tok_per_s": round(res["torch"], 1),
            "speedup": round(res["hip"] / res["torch"], 2)}


E2E_WORKLOAD_TEXT = ("cfg5 end-to-end generate, random-init Qwen3-0.6B architecture (28 layers, hidden 1024, 16/8 heads, "
                     "vocab 151936, tied embeddings), mops hip backend, engine counterpart of the reference's bench.py:9-28")


def run_e2e(args, torch, dev, mops):
    """`--op e2e`: the cfg5 workload as the line's own metric, plus a reduced run of the same engine on the
    CPU-restated torch backend (on the GPU) as the comparison baseline."""
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    mode = "eager" if args.e2e_eager else ("stepwise" if args.e2e_stepwise else "pipelined")
    r = e2e_modes(args, torch, [mode])[mode]
    n = args.e2e_seqs
    prompts, _ = e2e_workload(n)
    steps = r["prefill_steps"] + r["decode_steps"]
    out = {
        "metric": "e2e_output_tok_per_s", "value": r["tok_per_s"], "unit": "tok/s", "n_gpus": 1,
        "steps": steps, "warmup": 1, "ms_per_step": round(r["seconds"] * 1e3 / steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": E2E_WORKLOAD_TEXT + ", mode " + mode,
                   "prompts": n, "prompt_len": "uniform[100,1024]", "max_tokens": "uniform[100,1024]", "temperature": 0.6,
                   "output_tokens": r["output_tokens"], "prompt_tokens": r["prompt_tokens"]},
        "breakdown": r,
    }
    if not args.no_cpu_baseline:
        out["comparison_baseline"] = e2e_comparison(args, torch, prompts)
    print(json.dumps(out))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); the hot path has no "
              "cross-GPU exchange: each GPU would run the same kernels on its own kv heads or sequences.", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from nano_vllm_ninetoothed_amd import _capi, mops
    from nano_vllm_ninetoothed_amd import workloads as W
    _capi.load()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    g = torch.Generator(device=dev).manual_seed(args.seed)

    def randn_bf16(shape, std=1.0):
        return (torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std).to(torch.bfloat16) \
            if torch.Size(shape).numel() < (1 << 28) else _big_randn(shape, std)

    def _big_randn(shape, std):
        out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
        flat = out.view(-1)
        step = 1 << 27
        for i in range(0, flat.numel(), step):
            n = min(step, flat.numel() - i)
            flat[i:i + n] = (torch.randn(n, generator=g, device=dev, dtype=torch.float32) * std).to(torch.bfloat16)
        return out

    cpu_fn = None      # () -> (seconds, description, units_done)  on a bounded sample
    measured_traffic = None
    traffic_source = None

    if args.op == "e2e":
        run_e2e(args, torch, dev, mops)
        return
    bound = "hbm"
    dtype = "bf16"

    # ------------------------------------------------------------------ workloads
    if args.op in ("decode", "decode8b"):
        if args.op == "decode":
            bsz, hq, hkv, lo, hi, name = 256, 16, 8, 512, 4096, "cfg3 paged decode, Qwen3-0.6B shape"
        else:
            bsz, hq, hkv, lo, hi, name = 512, 32, 8, 1024, 8192, "cfg4 paged decode, Qwen3-8B shape"
        ctx = W.random_seq_lens(bsz, lo, hi, seed=args.seed)
        blocks_per_seq = [(c + W.BLOCK_SIZE - 1) // W.BLOCK_SIZE for c in ctx]
        nblk = sum(blocks_per_seq)
        max_blocks = max(blocks_per_seq)
        perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(args.seed)).to(torch.int32)
        table = torch.full((bsz, max_blocks), -1, dtype=torch.int32)
        pos = 0
        for b, nb in enumerate(blocks_per_seq):
            table[b, :nb] = perm[pos:pos + nb]
            pos += nb
        n_copies = 2 if args.op == "decode" else 1   # rotate KV buffers so no step re-reads warm lines
        caches = [(randn_bf16((nblk, W.BLOCK_SIZE, hkv, W.HEAD_DIM)), randn_bf16((nblk, W.BLOCK_SIZE, hkv, W.HEAD_DIM)))
                  for _ in range(n_copies)]
        q = randn_bf16((bsz, 1, hq, W.HEAD_DIM))
        lens_g = torch.tensor(ctx, dtype=torch.int32, device=dev)
        table_g = table.to(dev)
        scale = W.HEAD_DIM ** -0.5
        op = mops.flash_attn_with_kvcache

        def step(i):
            kc, vc = caches[i % n_copies]
            return op(q, kc, vc, cache_seqlens=lens_g, block_table=table_g, softmax_scale=scale, causal=True)

        work = W.decode_bytes(ctx, hq, hkv, max_blocks)      # algorithmic bytes per step
        metric, unit = "paged_decode_attn_GBps", "GB/s"
        config = {"workload": name, "batch": bsz, "q_heads": hq, "kv_heads": hkv, "head_dim": W.HEAD_DIM,
                  "block_size": W.BLOCK_SIZE, "context": f"uniform[{lo},{hi}] seed {args.seed}",
                  "context_tokens": sum(ctx), "kv_buffers_rotated": n_copies}
        kernel_name = "paged_decode_kernel (+ paged_decode_plan_kernel, paged_decode_combine_kernel)"
        # HBM-side bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this exact workload;
        # a figure copied from that profile, not measured by this run: only given for the default seed and
        # launch shape, with its source next to it
        tuned = any(os.environ.get(v) for v in ("MOPS_HIP_DECODE_HPW", "MOPS_HIP_DECODE_NCOLS", "MOPS_HIP_DECODE_MIN_PER_COL"))
        if args.op == "decode" and args.seed == 0 and not tuned:
            measured_traffic, traffic_source = profiled_traffic("decode")

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("flash_attn_with_kvcache", "torch")
            n = 64
            sub_tbl = table[:n]
            used = sub_tbl[sub_tbl >= 0].long()
            remap = torch.full((nblk,), -1, dtype=torch.int32)
            remap[used] = torch.arange(len(used), dtype=torch.int32)
            tbl = torch.where(sub_tbl >= 0, remap[sub_tbl.clamp(min=0).long()], sub_tbl)
            kc = caches[0][0][used.to(dev)].cpu()
            vc = caches[0][1][used.to(dev)].cpu()
            qc = q[:n].cpu()
            lens = torch.tensor(ctx[:n], dtype=torch.int32)
            ref(qc, kc, vc, cache_seqlens=lens, block_table=tbl, softmax_scale=scale)
            ts, t_start = [], time.perf_counter()
            while len(ts) < 5 or (time.perf_counter() - t_start < 12.0 and len(ts) < 400):
                t0 = time.perf_counter()
                ref(qc, kc, vc, cache_seqlens=lens, block_table=tbl, softmax_scale=scale)
                ts.append(time.perf_counter() - t0)
            return (sorted(ts)[len(ts) // 2], f"first {n} of {bsz} sequences, median of {len(ts)} passes (~12 s of CPU work)",
                    W.decode_bytes(ctx[:n], hq, hkv, max_blocks))

    elif args.op in ("prefill", "prefill_long"):
        # prefill_long: four 8192-token sequences, where the fixed cost per 128-row item no longer shows
        long_case = args.op == "prefill_long"
        lens = [8192] * 4 if long_case else W.random_seq_lens(16, 128, 2048, seed=args.seed)
        d = W.to_device(W.prefill_inputs(lens, seed=args.seed), dev)
        op = mops.flash_attn_varlen_func

        def step(i):
            return op(d["q"], d["k"], d["v"], max_seqlen_q=d["max_seqlen"], cu_seqlens_q=d["cu_seqlens"],
                      max_seqlen_k=d["max_seqlen"], cu_seqlens_k=d["cu_seqlens"], softmax_scale=d["scale"], causal=True)

        work = W.prefill_flops(lens, 16)
        bound = "mfma"
        metric, unit = "varlen_prefill_attn_TFLOPs", "TFLOP/s"
        config = {"workload": ("varlen causal prefill, four 8192-token sequences, Qwen3-0.6B shape" if long_case
                               else "cfg2 varlen causal prefill, Qwen3-0.6B shape"), "batch": len(lens), "q_heads": 16, "kv_heads": 8,
                  "head_dim": 128, "seq_lens": "4 x 8192" if long_case else f"uniform[128,2048] seed {args.seed}",
                  "total_tokens": sum(lens)}
        kernel_name = "varlen_prefill_pair_kernel<false>"
        if args.seed == 0:
            measured_traffic, traffic_source = profiled_traffic(args.op)

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("flash_attn_varlen_func", "torch")
            c = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in d.items()}
            ts = []
            if long_case:   # one 8192-token sequence is ~10 s of CPU work; the batch is four of them
                one = {"q": c["q"][:8192], "k": c["k"][:8192], "v": c["v"][:8192], "cu": c["cu_seqlens"][:2]}
                t0 = time.perf_counter()
                ref(one["q"], one["k"], one["v"], max_seqlen_q=8192, cu_seqlens_q=one["cu"], softmax_scale=c["scale"])
                return time.perf_counter() - t0, "first of the four sequences, one run", work / 4
            for _ in range(3):
                t0 = time.perf_counter()
                ref(c["q"], c["k"], c["v"], max_seqlen_q=c["max_seqlen"], cu_seqlens_q=c["cu_seqlens"], softmax_scale=c["scale"])
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[1], "whole batch, median of 3", work

    elif args.op in ("prefix_prefill", "prefix_prefill_short"):
        # prefix-cache hit (nanovllm/layers/attention.py:32-33 of the reference): 16 sequences with 1024 tokens already in
        # the paged cache and 1024 new ones; keys are read through block_table.  The short case is the shape of a shared
        # prompt followed by a few new tokens: 32 sequences, 2048 cached and 64 new tokens each.
        short_case = args.op == "prefix_prefill_short"
        new, prefix = ([64] * 32, [2048] * 32) if short_case else ([1024] * 16, [1024] * 16)
        d = W.to_device(W.prefix_prefill_inputs(new, prefix, seed=args.seed, poison_unused=False), dev)
        op = mops.flash_attn_varlen_func

        def step(i):
            return op(d["q"], d["k_cache"], d["v_cache"], max_seqlen_q=d["max_seqlen_q"], cu_seqlens_q=d["cu_seqlens_q"],
                      max_seqlen_k=d["max_seqlen_k"], cu_seqlens_k=d["cu_seqlens_k"], softmax_scale=d["scale"], causal=True,
                      block_table=d["block_table"])

        work = float(sum(4 * 128 * 16 * (n * pl + n * (n + 1) // 2) for n, pl in zip(new, prefix)))
        bound = "mfma"
        metric, unit = "varlen_prefill_attn_TFLOPs", "TFLOP/s"
        config = {"workload": "varlen causal prefill behind a cached prefix, keys in the paged cache, Qwen3-0.6B shape", "batch": len(new),
                  "q_heads": 16, "kv_heads": 8, "head_dim": 128, "new_tokens": f"{len(new)} x {new[0]}",
                  "cached_prefix": f"{len(new)} x {prefix[0]}", "block_size": W.BLOCK_SIZE}
        # long runs of new tokens stay on the 128-row kernel, few new tokens per sequence take the two-heads-per-wave form
        kernel_name = "varlen_prefill_pair_kernel<true>" if short_case else "varlen_prefill_kernel<false>"

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("flash_attn_varlen_func", "torch")
            c = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in d.items()}
            t0 = time.perf_counter()
            ref(c["q"][:new[0]], c["k_cache"], c["v_cache"], max_seqlen_q=new[0], cu_seqlens_q=c["cu_seqlens_q"][:2], max_seqlen_k=new[0] + prefix[0],
                cu_seqlens_k=c["cu_seqlens_k"][:2], softmax_scale=c["scale"], causal=True, block_table=c["block_table"][:1])
            return time.perf_counter() - t0, f"first of the {len(new)} sequences, one run", work / len(new)

    elif args.op == "store":
        lens = W.random_seq_lens(16, 128, 2048, seed=args.seed)
        T = sum(lens)
        n_copies = 4
        sets = []
        for i in range(n_copies):
            s = W.to_device(W.store_inputs(T, seed=args.seed + i, v_row_stride=4096), dev)
            wide = s["value"]
            s["value"] = wide
            s["kc"] = torch.zeros((s["num_blocks"], 256, 8, 128), dtype=torch.bfloat16, device=dev)
            s["vc"] = torch.zeros_like(s["kc"])
            sets.append(s)
        op = mops.store_kvcache

        def step(i):
            s = sets[i % n_copies]
            return op(s["key"], s["value"], s["kc"], s["vc"], s["slot_mapping"])

        work = float(2 * T * 1024 * 2 * 2 + 4 * T)
        metric, unit = "store_kvcache_GBps", "GB/s"
        config = {"workload": "cfg2 store_kvcache", "tokens": T, "row_bytes": 2048, "buffers_rotated": n_copies}
        kernel_name = "store_kvcache_kernel"

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("store_kvcache", "torch")
            s = sets[0]
            k, v, kc, vc, sl = (s[x].cpu() for x in ("key", "value", "kc", "vc", "slot_mapping"))
            ts = []
            for _ in range(5):
                t0 = time.perf_counter()
                ref(k, v, kc, vc, sl)
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[2], "whole batch, median of 5", work

    elif args.op in ("add_rms", "rms"):
        rows, hidden = 512, 4096
        n_copies = 24   # 24 x 16.8 MB > 256 MB of last-level cache
        sets = [W.to_device(W.rms_inputs(rows, hidden, seed=args.seed + i, with_residual=True), dev) for i in range(n_copies)]
        if args.op == "add_rms":
            op = mops.add_rms_forward

            def step(i):
                s = sets[i % n_copies]
                return op(s["x"], s["residual"], s["weight"], s["eps"])
            work = float(4 * rows * hidden * 2 + hidden * 2)
        else:
            op = mops.rms_forward

            def step(i):
                s = sets[i % n_copies]
                return op(s["x"], s["weight"], s["eps"])
            work = float(2 * rows * hidden * 2 + hidden * 2)
        metric, unit = f"{args.op}_forward_GBps", "GB/s"
        config = {"workload": f"cfg4 {args.op}_forward", "rows": rows, "hidden": hidden, "buffers_rotated": n_copies}
        kernel_name = "rmsnorm_kernel"

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op(f"{args.op}_forward", "torch")
            s = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in sets[0].items()}
            a = (s["x"], s["residual"], s["weight"], s["eps"]) if args.op == "add_rms" else (s["x"], s["weight"], s["eps"])
            ts = []
            for _ in range(7):
                t0 = time.perf_counter()
                ref(*a)
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[3], "whole batch, median of 7", work

    elif args.op == "silu":
        # siluAndMul on the gate_up buffer of a 16384-token prefill step (intermediate 3072); x and y are its two halves
        rows, inter, n_copies = 16384, 3072, 4
        bufs = [torch.randn((rows, 2 * inter), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(n_copies)]
        op = mops.get_op("siluAndMul", "hip")

        def step(i):
            x, y = bufs[i % n_copies].chunk(2, dim=-1)
            return op(x, y)

        work = float(rows * 3 * inter * 2)
        metric, unit = "silu_and_mul_GBps", "GB/s"
        config = {"workload": "siluAndMul, 16384 tokens x intermediate 3072 (Qwen3-0.6B), halves of one gate_up buffer", "rows": rows,
                  "intermediate": inter, "buffers_rotated": n_copies}
        kernel_name = "silu_and_mul_kernel"

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("siluAndMul", "torch")
            x, y = bufs[0].cpu().chunk(2, dim=-1)
            ts = []
            for _ in range(5):
                t0 = time.perf_counter()
                ref(x, y)
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[2], "whole batch, median of 5", work

    elif args.op == "sampler":
        # sampler_forward on the logits of a 256-sequence decode step (vocab 151936)
        rows, vocab, n_copies = 256, 151936, 4
        logit_sets = [torch.randn((rows, vocab), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(n_copies)]
        temps = torch.full((rows,), 0.6, device=dev)
        op = mops.get_op("sampler_forward", "hip")

        def step(i):
            return op(logit_sets[i % n_copies], temps)

        work = float(rows * vocab * 2 + rows * 8)
        metric, unit = "sampler_GBps", "GB/s"
        config = {"workload": "sampler_forward (greedy: row argmax), 256 rows x vocab 151936 bf16 logits", "rows": rows, "vocab": vocab,
                  "buffers_rotated": n_copies}
        kernel_name = "row_argmax_kernel"

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("sampler_forward", "torch")
            lg, tp = logit_sets[0].cpu(), temps.cpu()
            ts = []
            for _ in range(3):
                t0 = time.perf_counter()
                ref(lg, tp)
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[1], "whole batch, median of 3", work

    elif args.op == "qk_rope_store":
        # the fused q_norm + k_norm + rotary + store_kvcache launch on the qkv buffer of the cfg2 token count
        lens = W.random_seq_lens(16, 128, 2048, seed=args.seed)
        T, hq, hkv, hd, n_copies = sum(lens), 16, 8, 128, 4
        nblk = (T + 255) // 256 + 2
        sets = []
        for i in range(n_copies):
            qkv = torch.randn((T, (hq + 2 * hkv) * hd), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
            sets.append({"qkv": qkv, "kc": torch.zeros((nblk, 256, hkv, hd), dtype=torch.bfloat16, device=dev),
                         "vc": torch.zeros((nblk, 256, hkv, hd), dtype=torch.bfloat16, device=dev),
                         "slots": torch.randperm(nblk * 256, generator=g, device=dev)[:T].to(torch.int32)})
        qw = (1 + 0.1 * torch.randn(hd, generator=g, device=dev)).to(torch.bfloat16)
        kw = (1 + 0.1 * torch.randn(hd, generator=g, device=dev)).to(torch.bfloat16)
        ang = torch.rand((T, 1, hd // 2), generator=g, device=dev) * 6.28
        cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
        op = mops.get_op("qk_norm_rope_store", "hip")

        def step(i):
            st = sets[i % n_copies]
            return op(st["qkv"], qw, kw, 1e-6, cos, sin, st["kc"], st["vc"], st["slots"], hq, hkv, need_k=False)

        # read q, k, v rows, cos, sin and the slot; write q, the rotated k and v into the caches
        work = float(T * ((hq + 2 * hkv) * hd * 2 + 2 * (hd // 2) * 4 + 4 + hq * hd * 2 + 2 * hkv * hd * 2))
        metric, unit = "qk_norm_rope_store_GBps", "GB/s"
        config = {"workload": "fused q_norm + k_norm + rotary + store_kvcache, cfg2 token count, Qwen3-0.6B heads", "tokens": T,
                  "q_heads": hq, "kv_heads": hkv, "head_dim": hd, "buffers_rotated": n_copies}
        kernel_name = "qk_norm_rope_store_kernel"

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("qk_norm_rope_store", "torch")
            st = {k: v.cpu() for k, v in sets[0].items()}
            t0 = time.perf_counter()
            ref(st["qkv"], qw.cpu(), kw.cpu(), 1e-6, cos.cpu(), sin.cpu(), st["kc"], st["vc"], st["slots"], hq, hkv, need_k=False)
            return time.perf_counter() - t0, "whole batch, one run", work

    elif args.op == "launch_floor":
        # an empty kernel: the floor under the durations of the small operators
        lib = _capi.load()

        def step(i):
            return lib.mops_hip_launch_floor(torch.cuda.current_stream(dev).cuda_stream)

        work = 0.0
        metric, unit = "launch_floor_GBps", "GB/s"
        config = {"workload": "an empty kernel (64 lanes), launches back to back: what a launch costs with nothing to do"}
        kernel_name = "launch_floor_kernel"
        cpu_fn = None

    elif args.op == "copy":
        nbytes = 1 << 30
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)

        def step(i):
            return dst.copy_(src)

        work = float(2 * nbytes)
        metric, unit = "device_copy_GBps", "GB/s"
        config = {"workload": "calibration: 1 GiB device-to-device copy (reads 1 GiB, writes 1 GiB)", "bytes": nbytes}
        kernel_name = "torch elementwise copy"
        cpu_fn = None

    else:  # embedding
        vocab, hidden, n_ids = 151936, 4096, 512
        weight = _big_randn((vocab, hidden), 0.02)
        ids = [torch.randint(0, vocab, (n_ids,), generator=g, device=dev, dtype=torch.int32) for _ in range(64)]
        op = mops.embedding

        def step(i):
            return op(ids[i % len(ids)], weight)

        work = float(2 * n_ids * hidden * 2 + n_ids * 4)
        metric, unit = "embedding_GBps", "GB/s"
        config = {"workload": "cfg4 embedding", "vocab": vocab, "hidden": hidden, "ids": n_ids, "id_sets_rotated": len(ids)}
        kernel_name = "embedding_kernel"

        def cpu_fn():
            import oracle.mops_torch  # noqa: F401
            ref = mops.get_op("embedding", "torch")
            w, x = weight.cpu(), ids[0].cpu()
            ts = []
            for _ in range(7):
                t0 = time.perf_counter()
                ref(x, w)
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[3], "whole batch, median of 7", work

    # ------------------------------------------------------------------ timed region
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    ev_start, ev_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev_start.record()
    for i in range(args.steps):
        step(i)
    ev_end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    # one event pair over the whole timed region: launches run back to back, as they do in the kernel trace
    ev_ms = ev_start.elapsed_time(ev_end) / args.steps
    ms_per_step = wall * 1e3 / args.steps
    # shortest single launch, from a few individually bracketed launches after the timed region
    per_step_ms = []
    for i in range(min(args.steps, 10)):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        step(i)
        b.record()
        b.synchronize()
        per_step_ms.append(a.elapsed_time(b))

    if bound == "hbm":
        value = work / (ms_per_step * 1e-3) / 1e9
        achieved = work / (ev_ms * 1e-3) / 1e9
        peak, runit = HBM_PEAK_GBPS, "GB/s"
    else:
        value = work / (ms_per_step * 1e-3) / 1e12
        achieved = work / (ev_ms * 1e-3) / 1e12
        peak, runit = MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"

    out = {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic", "config": config,
        "roofline": {"bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": runit,
                     "frac": round(achieved / peak, 4), "traffic": measured_traffic, "traffic_source": traffic_source,
                     "kernel": kernel_name,
                     "algorithmic_work_per_launch": work, "event_ms_per_launch": round(ev_ms, 5),
                     "event_ms_min": round(min(per_step_ms), 5)},
    }
    if not args.no_cpu_baseline and cpu_fn is not None:
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        secs, sample, units = cpu_fn()
        cval = units / secs / (1e9 if bound == "hbm" else 1e12)
        out["cpu_baseline"] = {"value": round(cval, 4), "unit": unit, "cores": torch.get_num_threads(), "kind": "port",
                               "sample": sample, "seconds": round(secs, 4)}
    if args.op in ("prefill", "prefill_long", "prefix_prefill", "prefix_prefill_short"):
        # what a library bf16 GEMM sustains on this chip in this run: the 2.5 PFLOP/s peak assumes 2.4 GHz, which the
        # part does not hold under matrix load, so this is the practical MFMA ceiling to read the fraction against
        n = 8192
        ga = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
        gb = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
        for _ in range(3):
            ga @ gb
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            ga @ gb
        e1.record()
        torch.cuda.synchronize()
        gemm_tf = 2.0 * n ** 3 * 20 / (e0.elapsed_time(e1) * 1e-3) / 1e12
        out["roofline"]["library_gemm"] = {"what": "torch.matmul (hipBLASLt) bf16 8192^3, 20 launches back to back, same run",
                                           "TFLOP/s": round(gemm_tf, 1), "kernel_vs_library_gemm": round(achieved / gemm_tf, 4)}
    if args.op == "decode" and not args.no_e2e:
        # second half of the headline metric: end-to-end output tok/s of the cfg5 workload.  "eager" is the reference's own
        # setting (enforce_eager=True, bench.py:15 of the reference; every step's tokens read back,
        # nanovllm/engine/model_runner.py:212); the two graph modes replay the decode step from HIP graphs.
        step = op = caches = q = None
        torch.cuda.empty_cache()
        r = e2e_modes(args, torch, ["eager", "stepwise", "pipelined"])
        out["e2e"] = {"metric": "e2e_output_tok_per_s", "unit": "tok/s", "workload": E2E_WORKLOAD_TEXT,
                      "prompts": args.e2e_seqs, "prompt_len": "uniform[100,1024]", "max_tokens": "uniform[100,1024]",
                      "temperature": 0.6, "runs": [r["eager"], r["stepwise"], r["pipelined"]]}
        if not args.no_cpu_baseline:
            out["e2e"]["comparison_baseline"] = e2e_comparison(args, torch, e2e_workload(args.e2e_seqs)[0])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
