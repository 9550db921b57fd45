"""GPU: the engine counterpart drives the hip backend through a whole prefill + decode loop; a small
Qwen3-shaped model must produce the same logits (to bf16 GEMM tolerance) as the same engine running on the
oracle backend, and generation must respect max_tokens and free its cache blocks."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _engines(gpu):
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    import oracle.mops_torch  # noqa: F401
    shape = Qwen3Shape(num_layers=2, vocab=2048)
    return (Engine(shape, backend="hip", num_blocks=24, seed=3, device=str(gpu)),
            Engine(shape, backend="torch", num_blocks=24, seed=3, device=str(gpu)))


def test_prefill_and_decode_logits_match_oracle_backend(gpu):
    hip, ref = _engines(gpu)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, 2048, (n,), generator=g).tolist() for n in (300, 17, 256, 1)]
    outs = []
    for eng in (hip, ref):
        for p in prompts:
            eng.add_request(p, 4)
        seqs, is_prefill = eng._schedule()
        assert is_prefill and len(seqs) == 4
        ids, pos, ctx = eng._prepare_prefill(seqs)
        logits_p = eng.forward(ids, pos, ctx).float()
        for q in seqs:                      # same next token for both engines so the decode inputs agree
            q.token_ids.append(7)
        seqs2, is_prefill2 = eng._schedule()
        assert not is_prefill2
        ids, pos, ctx = eng._prepare_decode(seqs2)
        logits_d = eng.forward(ids, pos, ctx).float()
        outs.append((logits_p.cpu(), logits_d.cpu()))
    for a, b, what in ((outs[0][0], outs[1][0], "prefill"), (outs[0][1], outs[1][1], "decode")):
        assert a.shape == b.shape == (4, 2048)
        assert torch.isfinite(a).all()
        err = (a - b).abs().max().item()
        assert err <= 0.05 * b.abs().max().item() + 1e-3, f"{what} logits differ by {err}"


def test_fused_qk_step_gives_the_same_logits_and_cache_as_the_separate_ops(gpu):
    """The engine with the fused q_norm/k_norm/rotary/store launch and one decode plan per step, and the same
    engine with the separate ops and a plan per layer, produce bit-identical prefill and decode logits and
    KV caches."""
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    shape = Qwen3Shape(num_layers=2, vocab=2048)
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, 2048, (n,), generator=g).tolist() for n in (129, 3, 256)]
    res = []
    for fused in (True, False):
        eng = Engine(shape, backend="hip", num_blocks=24, seed=3, device=str(gpu))
        assert eng.op_qk_norm_rope_store is not None
        eng.use_fused_qk = fused
        eng.share_decode_plan = fused   # and the decode plan shared between the layers, or made per layer
        for p in prompts:
            eng.add_request(p, 4)
        seqs, _ = eng._schedule()
        ids, pos, ctx = eng._prepare_prefill(seqs)
        lp = eng.forward(ids, pos, ctx)
        for q in seqs:
            q.token_ids.append(11)
        seqs2, _ = eng._schedule()
        ids, pos, ctx = eng._prepare_decode(seqs2)
        ld = eng.forward(ids, pos, ctx)
        res.append((lp.cpu(), ld.cpu(), eng.kv_cache.cpu()))
    for a, b, what in zip(res[0], res[1], ("prefill logits", "decode logits", "kv cache")):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), what


def test_generate_respects_max_tokens_and_frees_blocks(gpu):
    hip, _ = _engines(gpu)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 2048, (n,), generator=g).tolist() for n in (250, 255, 256, 5, 511)]
    max_tokens = [3, 10, 1, 7, 4]
    outs, stats = hip.generate(prompts, max_tokens)
    assert [len(o) for o in outs] == max_tokens
    assert all(0 <= t < 2048 for o in outs for t in o)
    assert len(hip.free_blocks) == 24 and not hip.running and not hip.waiting
    assert stats["prefill_steps"] == 1 and stats["decode_steps"] == 9


@pytest.mark.parametrize("smallest_first", [False, True])
def test_graph_replay_matches_eager_decode(gpu, smallest_first):
    """The captured decode forward is replayed several times with eager work and synchronisation in
    between; every replay must reproduce the eager logits bit for bit, including with padded rows.  With
    smallest_first the small buckets are captured before the large ones: the attention scratch the graphs point
    at is sized before the first capture, so a later, larger capture must not move it."""
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    shape = Qwen3Shape(num_layers=2, vocab=2048)
    eng = Engine(shape, backend="hip", num_blocks=40, seed=5, device=str(gpu))
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 2048, (n,), generator=g).tolist() for n in (40, 300, 255, 256, 7)]
    for p in prompts:
        eng.add_request(p, 64)
    eng.step()                                    # prefill
    eng.capture_decode_graphs(max_bs=16, max_model_len=1024, smallest_first=smallest_first)
    for it in range(4):
        seqs, is_prefill = eng._schedule()
        assert not is_prefill
        ids, pos, ctx = eng._prepare_decode(seqs)
        # eager run on the same padded batch the graph sees (the GEMM library picks its kernels by row count)
        bs, bucket = len(seqs), 8
        pad = bucket - bs
        ids_p = torch.cat((ids, ids.new_zeros(pad)))
        pos_p = torch.cat((pos, pos.new_zeros(pad)))
        ctx_p = dict(is_prefill=False, slot_mapping=torch.cat((ctx["slot_mapping"], ctx["slot_mapping"].new_full((pad,), -1))),
                     context_lens=torch.cat((ctx["context_lens"], ctx["context_lens"].new_zeros(pad))),
                     block_tables=torch.cat((ctx["block_tables"], ctx["block_tables"].new_full((pad, ctx["block_tables"].size(1)), -1))))
        eager = eng.forward(ids_p, pos_p, ctx_p)[:bs]
        torch.cuda.synchronize()
        replay = eng._decode_replay(ids, pos, ctx)
        torch.cuda.synchronize()
        assert torch.equal(eager, replay), f"replay {it} differs from eager"
        for q in seqs:
            q.token_ids.append(int(eager[0].argmax()) % 2048)


def test_pipelined_generate_gives_the_tokens_of_stepwise_generate(gpu):
    """generate() with graphs captured keeps the sampled tokens on the device and reads them back at the
    end; the tokens, the step counts and the freed state must equal those of the stepwise loop, which reads
    every step's tokens back before it schedules the next.  Run twice on the same engine: the second call
    starts from the rows and blocks the first one freed."""
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    shape = Qwen3Shape(num_layers=2, vocab=2048)
    g = torch.Generator().manual_seed(9)
    res = []
    for pipelined in (True, False):
        eng = Engine(shape, backend="hip", num_blocks=64, seed=4, device=str(gpu), max_num_seqs=8, max_num_batched_tokens=1024)
        eng.capture_decode_graphs(max_bs=16, max_model_len=1024)
        eng.pipelined = pipelined
        runs = []
        for rnd in range(2):
            gg = torch.Generator().manual_seed(20 + rnd)
            lens = (40, 300, 255, 256, 7, 130, 1, 90, 64, 200, 33)          # more prompts than max_num_seqs
            prompts = [torch.randint(0, 2048, (n,), generator=gg).tolist() for n in lens]
            max_tokens = [5, 12, 1, 7, 30, 2, 9, 16, 3, 21, 8]
            outs, stats = eng.generate(prompts, max_tokens)
            assert [len(o) for o in outs] == max_tokens
            assert all(0 <= t < 2048 for o in outs for t in o)
            assert len(eng.free_blocks) == 64 and not eng.running and not eng.waiting
            runs.append((outs, stats["prefill_steps"], stats["decode_steps"], stats["decode_tokens"]))
        res.append(runs)
    assert res[0] == res[1]


def test_shipped_gemm_solution_table_is_applied(gpu):
    """The table of hipBLASLt solutions shipped in the package was measured for this GPU and this library
    version; if either differs the loader pins nothing and the engine silently runs on the heuristic's picks."""
    from nano_vllm_ninetoothed_amd.mops.hip.ops import load_linear_solutions
    assert load_linear_solutions() > 0


def test_full_size_engine_pipelined_equals_stepwise(gpu):
    """The end-to-end configuration at its real shape: random-init Qwen3-0.6B architecture (28 layers, vocab
    151936), 64 prompts of 100..1024 random tokens, graph buckets up to 256 sequences.  Pipelined generation must
    give the stepwise loop's tokens; every sequence gets exactly its max_tokens and all cache blocks come back."""
    import random
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    shape = Qwen3Shape()
    assert (shape.num_layers, shape.vocab, shape.hidden, shape.num_heads, shape.num_kv_heads) == (28, 151936, 1024, 16, 8)
    random.seed(0)
    prompts = [[random.randint(0, 10000) for _ in range(random.randint(100, 1024))] for _ in range(64)]
    max_tokens = [random.randint(8, 48) for _ in range(64)]
    eng = Engine(shape, backend="hip", num_blocks=64 * 5, seed=0, device=str(gpu))
    eng.capture_decode_graphs(max_bs=256, max_model_len=4096)
    assert eng.graph_bs[-1] == 256
    runs = []
    for pipelined in (True, False):
        eng.pipelined = pipelined
        outs, stats = eng.generate(prompts, max_tokens)
        assert [len(o) for o in outs] == max_tokens
        assert all(0 <= t < shape.vocab for o in outs for t in o)
        assert len(eng.free_blocks) == eng.num_blocks and not eng.running and not eng.waiting
        assert stats["decode_tokens"] + 64 == sum(max_tokens)       # the first token of a sequence comes from its prefill
        runs.append(outs)
    assert runs[0] == runs[1], "pipelined and stepwise generation disagree"


def test_end_to_end_workload_exactly_as_the_reference_words_it(gpu):
    """The end-to-end configuration at its full size (bench.py:9-28 of the reference): random.seed(0), 256 prompts of
    100..1024 random token ids, 100..1024 output tokens each, temperature 0.6, no EOS, on the random-init Qwen3-0.6B
    architecture.  One engine runs it pipelined and then stepwise: the tokens must be equal, every sequence gets exactly
    its max_tokens, every cache block comes back."""
    import random
    from nano_vllm_ninetoothed_amd.engine import Engine, Qwen3Shape
    random.seed(0)
    prompts = [[random.randint(0, 10000) for _ in range(random.randint(100, 1024))] for _ in range(256)]
    max_tokens = [random.randint(100, 1024) for _ in range(256)]
    eng = Engine(Qwen3Shape(), backend="hip", num_blocks=2560, seed=0, device=str(gpu))
    eng.generate([[1, 2, 3, 4, 5, 6, 7, 8]], 8)
    eng.capture_decode_graphs(max_bs=256, max_model_len=4096)
    runs = []
    for pipelined in (True, False):
        eng.pipelined = pipelined
        outs, stats = eng.generate(prompts, max_tokens, temperature=0.6)
        assert [len(o) for o in outs] == max_tokens
        assert len(eng.free_blocks) == eng.num_blocks and not eng.running and not eng.waiting
        assert stats["decode_tokens"] + 256 == sum(max_tokens)
        runs.append(outs)
    assert runs[0] == runs[1], "pipelined and stepwise generation disagree on the full workload"
