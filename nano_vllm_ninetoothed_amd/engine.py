"""Engine counterpart for the end-to-end generation benchmark: the smallest caller that drives the mops
operators the way the reference's engine does, so that generation throughput can be measured on a
Qwen3-shaped, randomly initialised model without tokenizer or checkpoint files.

What it mirrors (and nothing more):
  * op order of a decoder layer and of the model (nanovllm/models/qwen3.py:69-82, 140-153, 167-177,
    199-210): embedding -> [rms/add_rms -> qkv linear -> q_norm/k_norm on strided views -> rotary ->
    store_kvcache + varlen prefill | paged decode -> o_proj -> add_rms -> gate_up linear -> siluAndMul ->
    down linear] x L -> add_rms -> lm head (tied) on the last token of each sequence -> sampler;
  * the metadata the model runner hands to attention (nanovllm/engine/model_runner.py:120-180): int32
    cu_seqlens, slot_mapping, context_lens, block_tables padded with -1, one contiguous
    [2, L, blocks, 256, Hkv, D] cache whose per-layer slabs are the k/v caches (:100-118);
  * the scheduling policy (nanovllm/engine/scheduler.py:25-59): prefill first, limited by
    max_num_batched_tokens / max_num_seqs, otherwise one decode step for every running sequence.
  * optional HIP-graph replay of the decode forward for bucketed batch sizes with static input buffers,
    slot_mapping padded with -1 and context_lens with 0 (model_runner.py:189-206, 216-251).
Beyond the reference: with graphs captured, generate() does not wait for a step's tokens before it issues
the next step.  Which sequences run, their lengths, slots and block tables depend only on token counts, so
the host prepares step t+1 while the GPU works on step t; the sampled tokens stay on the device (one row
per sequence, gathered as the next step's input ids) and are read back once at the end.  The reference
reads them back every step (model_runner.py:212), which leaves the GPU idle while the host schedules.
Not mirrored: prefix caching, preemption (the cache is sized so it never triggers), tensor parallelism,
the tokenizer, weight loading.

Every tensor op goes through a mops backend looked up by name, so the same engine runs on the `hip`
backend and on any other registered one.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field

import torch

from . import mops

BLOCK_SIZE = 256


@dataclass
class Qwen3Shape:
    """Qwen3-0.6B architecture numbers."""
    num_layers: int = 28
    hidden: int = 1024
    num_heads: int = 16
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate: int = 3072
    vocab: int = 151936
    rms_eps: float = 1e-6
    rope_theta: float = 1000000.0
    max_position: int = 40960


@dataclass
class Sequence:
    token_ids: list
    max_tokens: int
    temperature: float
    num_prompt_tokens: int = 0
    block_table: list = field(default_factory=list)
    row: int = -1      # pipelined generation: this sequence's row in the device-side last-token table
    filled: int = 0    # pipelined generation: completion tokens whose values have been read back

    def __post_init__(self):
        self.num_prompt_tokens = len(self.token_ids)

    def __len__(self):
        return len(self.token_ids)

    @property
    def num_completion_tokens(self):
        return len(self.token_ids) - self.num_prompt_tokens


class Engine:
    def __init__(self, shape: Qwen3Shape | None = None, backend: str = "hip", num_blocks: int = 2560, seed: int = 0,
                 max_num_batched_tokens: int = 16384, max_num_seqs: int = 512, device="cuda:0"):
        self.shape = s = shape if shape is not None else Qwen3Shape()
        self.dev = torch.device(device)
        self.backend = backend
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_num_seqs = max_num_seqs
        for name in mops.OP_NAMES:
            op = mops.get_op(name, backend)
            if op is None and name != "softmax":
                raise RuntimeError(f"backend {backend} does not provide {name}")
            setattr(self, "op_" + name, op)
        # the fused q_norm + k_norm + rotary + store_kvcache launch, where the backend has it
        self.op_qk_norm_rope_store = mops.get_op("qk_norm_rope_store", backend) if mops.has_op("qk_norm_rope_store", backend) else None
        self.use_fused_qk = True
        self.share_decode_plan = True   # layers 2..N of a decode step reuse layer 1's split of the KV stream

        g = torch.Generator(device=self.dev).manual_seed(seed)

        def w(*shape_, std):
            return (torch.randn(shape_, generator=g, device=self.dev, dtype=torch.float32) * std).to(torch.bfloat16)

        def norm_w(n):
            return (1.0 + 0.05 * torch.randn(n, generator=g, device=self.dev, dtype=torch.float32)).to(torch.bfloat16)

        q_size, kv_size = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
        self.q_size, self.kv_size = q_size, kv_size
        self.embed = w(s.vocab, s.hidden, std=0.02)          # tied: also the lm head
        self.layers = []
        for _ in range(s.num_layers):
            self.layers.append(dict(
                input_norm=norm_w(s.hidden), post_norm=norm_w(s.hidden), q_norm=norm_w(s.head_dim), k_norm=norm_w(s.head_dim),
                qkv=w(q_size + 2 * kv_size, s.hidden, std=s.hidden ** -0.5), o=w(s.hidden, q_size, std=q_size ** -0.5),
                gate_up=w(2 * s.intermediate, s.hidden, std=s.hidden ** -0.5), down=w(s.hidden, s.intermediate, std=s.intermediate ** -0.5)))
        self.final_norm = norm_w(s.hidden)

        inv_freq = 1.0 / (s.rope_theta ** (torch.arange(0, s.head_dim, 2, dtype=torch.float32) / s.head_dim))
        freqs = torch.outer(torch.arange(s.max_position, dtype=torch.float32), inv_freq)
        self.cos_sin = torch.cat((freqs.cos(), freqs.sin()), dim=-1).unsqueeze(1).to(self.dev)   # [P, 1, D]

        self.num_blocks = num_blocks
        self.kv_cache = torch.zeros((2, s.num_layers, num_blocks, BLOCK_SIZE, s.num_kv_heads, s.head_dim),
                                    dtype=torch.bfloat16, device=self.dev)
        self.free_blocks = deque(range(num_blocks))
        self.waiting: deque = deque()
        self.running: deque = deque()
        self.scale = s.head_dim ** -0.5
        self.graphs = {}
        self.graph_bs = []
        # pipelined generation (see the module docstring): last sampled token per sequence row; row 0
        # takes the writes of padding rows
        self.pipelined = True
        self.last_tok = torch.zeros(max_num_seqs + 1, dtype=torch.int64, device=self.dev)
        self.free_rows = deque(range(1, max_num_seqs + 1))
        self.unit_temps = torch.ones(max_num_seqs, dtype=torch.float32, device=self.dev)
        self._sampler_checked = False
        self.capture_stream = None

    def _check_sampler_ignores_temperature(self):
        """Pipelined generation hands the sampler unit temperatures (the per-sequence ones would cost a gather per step).
        That is only right while the backend's sampler is greedy, as the reference's is (mops/torch/ops.py:37-43 with
        the sampling line commented out): checked once, on random logits, before the first pipelined run."""
        if self._sampler_checked:
            return
        g = torch.Generator(device=self.dev).manual_seed(1234)
        logits = torch.randn((8, 4096), generator=g, device=self.dev, dtype=torch.float32).to(torch.bfloat16)
        hot = torch.full((8,), 0.3, dtype=torch.float32, device=self.dev)
        a = self.op_sampler_forward(logits, self.unit_temps[:8])
        b = self.op_sampler_forward(logits, hot)
        if not torch.equal(a, b):
            raise RuntimeError(f"the {self.backend} backend's sampler depends on the temperature: pipelined generation "
                               "passes unit temperatures and would sample differently; set engine.pipelined = False")
        self._sampler_checked = True

    # ------------------------------------------------------------------ HIP graphs for decode
    @torch.inference_mode()
    def capture_decode_graphs(self, max_bs: int = 256, max_model_len: int = 4096, smallest_first: bool = False):
        """Captures the decode forward (embedding .. final norm) once per batch-size bucket.  Replays
        read their inputs from static buffers; rows beyond the live batch carry slot -1 / length 0,
        which store_kvcache skips and paged decode answers with zeros.  The order of the captures does not matter
        (smallest_first exists for the test of that)."""
        max_blocks = (max_model_len + BLOCK_SIZE - 1) // BLOCK_SIZE
        dev = self.dev
        self.g_ids = torch.zeros(max_bs, dtype=torch.int64, device=dev)
        self.g_i64 = torch.zeros((2, max_bs), dtype=torch.int64, device=dev)    # int64 copies of rows and positions
        self.g_rows64, self.g_pos = self.g_i64[0], self.g_i64[1]
        # the int32 inputs are views of one buffer, so that one host-to-device copy can fill them all:
        # [sequence rows | positions | slots | lengths | block tables]
        self.g_meta = torch.empty(max_bs * (4 + max_blocks), dtype=torch.int32, device=dev)
        self.g_rows, self.g_pos32 = self.g_meta[:max_bs], self.g_meta[max_bs:2 * max_bs]
        self.g_slots, self.g_lens = self.g_meta[2 * max_bs:3 * max_bs], self.g_meta[3 * max_bs:4 * max_bs]
        self.g_tables = self.g_meta[4 * max_bs:].view(max_bs, max_blocks)
        self.g_rows.zero_()
        self.g_pos32.zero_()
        self.g_slots.fill_(-1)
        self.g_lens.zero_()
        self.g_tables.fill_(-1)
        self.g_out = torch.zeros((max_bs, self.shape.hidden), dtype=torch.bfloat16, device=dev)
        self.graph_bs = [b for b in (1, 2, 4, 8) if b <= max_bs] + list(range(16, max_bs + 1, 16))
        # Every bucket is captured on one stream of our own.  The ops keep their scratch buffers per stream, and
        # the graphs hold those addresses: sizing the scratch for the largest bucket on that stream before the
        # first capture means no capture, in whatever order, allocates or moves it.
        # The stream stays alive with the engine: the scratch is keyed by the stream's handle, and a handle that went back
        # to torch's pool could be handed to unrelated eager work, which would then share the graphs' scratch.
        capture_stream = self.capture_stream = self.capture_stream or torch.cuda.Stream(dev)
        if self.backend == "hip":
            from .mops.hip.ops import reserve_decode_workspace
            with torch.cuda.stream(capture_stream):
                reserve_decode_workspace(max_bs, self.shape.num_heads, self.shape.num_kv_heads, max_blocks, BLOCK_SIZE, dev)
        pool = None
        for bs in (self.graph_bs if smallest_first else reversed(self.graph_bs)):
            ctx = dict(is_prefill=False, slot_mapping=self.g_slots[:bs], context_lens=self.g_lens[:bs],
                       block_tables=self.g_tables[:bs], hidden_only=True)
            graph = torch.cuda.CUDAGraph()
            self.g_out[:bs] = self.forward(self.g_ids[:bs], self.g_pos[:bs], ctx)      # warm-up outside capture
            torch.cuda.synchronize(dev)
            with torch.cuda.graph(graph, pool, stream=capture_stream):
                self.g_out[:bs] = self.forward(self.g_ids[:bs], self.g_pos[:bs], ctx)
            if pool is None:
                pool = graph.pool()
            self.graphs[bs] = graph
        torch.cuda.synchronize(dev)

    @torch.inference_mode()
    def _decode_replay(self, ids, pos, ctx):
        bs = ids.numel()
        bucket = next(b for b in self.graph_bs if b >= bs)
        self.g_ids[:bs] = ids
        self.g_pos[:bs] = pos
        self.g_slots.fill_(-1)
        self.g_slots[:bs] = ctx["slot_mapping"]
        self.g_lens.zero_()
        self.g_lens[:bs] = ctx["context_lens"]
        self.g_tables[:bs, : ctx["block_tables"].size(1)] = ctx["block_tables"]
        self.graphs[bucket].replay()
        # the lm head runs on the bucket's row count, like the captured layers: GEMM solutions are chosen per shape
        return self.op_linear(self.g_out[:bucket], self.embed)[:bs]

    # ------------------------------------------------------------------ model
    def _attention(self, layer_id, q, k, v, ctx, stored=False):
        k_cache, v_cache = self.kv_cache[0, layer_id], self.kv_cache[1, layer_id]
        if not stored:
            self.op_store_kvcache(k, v, k_cache, v_cache, ctx["slot_mapping"])
        if ctx["is_prefill"]:
            return self.op_flash_attn_varlen_func(q, k, v, max_seqlen_q=ctx["max_seqlen"], cu_seqlens_q=ctx["cu_seqlens"],
                                                  max_seqlen_k=ctx["max_seqlen"], cu_seqlens_k=ctx["cu_seqlens"],
                                                  softmax_scale=self.scale, causal=True, block_table=None)
        extra = {"reuse_plan": True} if (self.backend == "hip" and self.share_decode_plan and layer_id > 0) else {}
        return self.op_flash_attn_with_kvcache(q.unsqueeze(1), k_cache, v_cache, cache_seqlens=ctx["context_lens"],
                                               block_table=ctx["block_tables"], softmax_scale=self.scale, causal=True, **extra)

    @torch.inference_mode()
    def forward(self, input_ids, positions, ctx):
        s = self.shape
        h = self.op_embedding(input_ids, self.embed)
        residual = None
        cos, sin = self.cos_sin[positions].chunk(2, dim=-1)
        for i, L in enumerate(self.layers):
            if residual is None:
                h, residual = self.op_rms_forward(h, L["input_norm"], s.rms_eps), h
            else:
                h, residual = self.op_add_rms_forward(h, residual, L["input_norm"], s.rms_eps)
            qkv = self.op_linear(h, L["qkv"])
            if self.op_qk_norm_rope_store is not None and self.use_fused_qk:
                q, k, v = self.op_qk_norm_rope_store(qkv, L["q_norm"], L["k_norm"], s.rms_eps, cos, sin, self.kv_cache[0, i],
                                                     self.kv_cache[1, i], ctx["slot_mapping"], s.num_heads, s.num_kv_heads,
                                                     need_k=ctx["is_prefill"])
                o = self._attention(i, q, k, v, ctx, stored=True)
            else:
                q, k, v = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
                q = self.op_rms_forward(q.view(-1, s.num_heads, s.head_dim), L["q_norm"], s.rms_eps)
                k = self.op_rms_forward(k.view(-1, s.num_kv_heads, s.head_dim), L["k_norm"], s.rms_eps)
                v = v.view(-1, s.num_kv_heads, s.head_dim)
                q = self.op_apply_rotary_emb(q, cos, sin)
                k = self.op_apply_rotary_emb(k, cos, sin)
                o = self._attention(i, q, k, v, ctx)
            h = self.op_linear(o.flatten(1, -1), L["o"])
            h, residual = self.op_add_rms_forward(h, residual, L["post_norm"], s.rms_eps)
            gate, up = self.op_linear(h, L["gate_up"]).chunk(2, -1)
            h = self.op_linear(self.op_siluAndMul(gate, up), L["down"])
        h, _ = self.op_add_rms_forward(h, residual, self.final_norm, s.rms_eps)
        if ctx.get("hidden_only"):
            return h
        if ctx["is_prefill"]:
            h = h[ctx["cu_seqlens"][1:].long() - 1].contiguous()
        return self.op_linear(h, self.embed)

    # ------------------------------------------------------------------ metadata (model_runner.py:120-187)
    def _to_dev(self, data, dtype):
        return torch.tensor(data, dtype=dtype, pin_memory=True).to(self.dev, non_blocking=True)

    def _block_tables(self, seqs):
        width = max(len(q.block_table) for q in seqs)
        return self._to_dev([q.block_table + [-1] * (width - len(q.block_table)) for q in seqs], torch.int32)

    def _prepare_prefill(self, seqs):
        ids, pos, cu, slots, max_len = [], [], [0], [], 0
        for q in seqs:
            n = len(q)
            ids.extend(q.token_ids)
            pos.extend(range(n))
            cu.append(cu[-1] + n)
            max_len = max(max_len, n)
            for i, blk in enumerate(q.block_table):
                start = blk * BLOCK_SIZE
                slots.extend(range(start, start + min(BLOCK_SIZE, n - i * BLOCK_SIZE)))
        ctx = dict(is_prefill=True, cu_seqlens=self._to_dev(cu, torch.int32), max_seqlen=max_len,
                   slot_mapping=self._to_dev(slots, torch.int32))
        return self._to_dev(ids, torch.int64), self._to_dev(pos, torch.int64), ctx

    def _prepare_decode(self, seqs):
        ids = [q.token_ids[-1] for q in seqs]
        pos = [len(q) - 1 for q in seqs]
        slots = [q.block_table[-1] * BLOCK_SIZE + (len(q) - 1) % BLOCK_SIZE for q in seqs]
        ctx = dict(is_prefill=False, slot_mapping=self._to_dev(slots, torch.int32),
                   context_lens=self._to_dev([len(q) for q in seqs], torch.int32), block_tables=self._block_tables(seqs))
        return self._to_dev(ids, torch.int64), self._to_dev(pos, torch.int64), ctx

    # ------------------------------------------------------------------ scheduling (scheduler.py:25-72)
    def _blocks_needed(self, n_tokens):
        return (n_tokens + BLOCK_SIZE - 1) // BLOCK_SIZE

    def add_request(self, token_ids, max_tokens, temperature=0.6):
        self.waiting.append(Sequence(list(token_ids), max_tokens, temperature))

    def _schedule(self):
        batch, tokens = [], 0
        while self.waiting and len(batch) < self.max_num_seqs:
            q = self.waiting[0]
            need = self._blocks_needed(len(q))
            if tokens + len(q) > self.max_num_batched_tokens or need > len(self.free_blocks):
                break
            q.block_table = [self.free_blocks.popleft() for _ in range(need)]
            tokens += len(q)
            self.waiting.popleft()
            self.running.append(q)
            batch.append(q)
        if batch:
            return batch, True
        batch = list(self.running)[: self.max_num_seqs]
        for q in batch:   # the token about to be written may open a new block
            if len(q) % BLOCK_SIZE == 1 and len(q.block_table) < self._blocks_needed(len(q)):
                if not self.free_blocks:
                    raise RuntimeError("KV cache exhausted: this engine counterpart does not preempt; raise num_blocks")
                q.block_table.append(self.free_blocks.popleft())
        return batch, False

    @torch.inference_mode()
    def step(self):
        seqs, is_prefill = self._schedule()
        ids, pos, ctx = self._prepare_prefill(seqs) if is_prefill else self._prepare_decode(seqs)
        temps = self._to_dev([q.temperature for q in seqs], torch.float32)
        if not is_prefill and self.graphs and len(seqs) <= self.graph_bs[-1] and ctx["block_tables"].size(1) <= self.g_tables.size(1):
            logits = self._decode_replay(ids, pos, ctx)
        else:
            logits = self.forward(ids, pos, ctx)
        tokens = self.op_sampler_forward(logits, temps).tolist()     # the only device->host sync of a step
        finished = []
        for q, t in zip(seqs, tokens):
            q.token_ids.append(t)
            if q.num_completion_tokens >= q.max_tokens:
                finished.append(q)
        for q in finished:
            self.running.remove(q)
            self.free_blocks.extend(q.block_table)
            q.block_table = []
        return seqs, is_prefill, finished

    @torch.inference_mode()
    def _generate_pipelined(self, stats):
        """Runs until no sequence is waiting or running without reading a token back in between."""
        import numpy as np
        self._check_sampler_ignores_temperature()
        dev = self.dev
        n, max_blocks = self.g_ids.numel(), self.g_tables.size(1)
        depth = 8                                  # steps the host may be ahead of the GPU
        staging = [torch.empty(self.g_meta.numel(), dtype=torch.int32, pin_memory=True) for _ in range(depth)]
        staged = [None] * depth                    # event: the copy out of that staging buffer has run
        hist_rows = 2048
        hist = torch.empty((hist_rows, self.max_num_seqs), dtype=torch.int64, device=dev)
        steps = []                                 # (history row, sequences, is_prefill, end-of-step event)
        mark = torch.cuda.Event(enable_timing=True)
        mark.record()

        def drain():
            nonlocal mark
            if not steps:
                return
            torch.cuda.synchronize(dev)
            host = hist[:len(steps)].cpu()
            prev = mark
            for h, seqs, is_prefill, ev in steps:
                row = host[h].tolist()
                for j, q in enumerate(seqs):
                    q.token_ids[q.num_prompt_tokens + q.filled] = row[j]
                    q.filled += 1
                stats["prefill_s" if is_prefill else "decode_s"] += prev.elapsed_time(ev) * 1e-3
                prev = ev
            mark = prev
            steps.clear()

        it = 0
        while self.waiting or self.running:
            if len(steps) == hist_rows:
                drain()
            seqs, is_prefill = self._schedule()
            bs = len(seqs)
            graphable = (not is_prefill and bs <= self.graph_bs[-1]
                         and max(len(q.block_table) for q in seqs) <= max_blocks)
            if is_prefill:
                if len(self.free_rows) < bs:     # more sequences in flight than rows so far: grow the table
                    old = self.last_tok.numel()
                    self.last_tok = torch.cat((self.last_tok, torch.zeros(max(bs, old), dtype=torch.int64, device=dev)))
                    self.free_rows.extend(range(old, self.last_tok.numel()))
                for q in seqs:
                    q.row = self.free_rows.popleft()
                ids, pos, ctx = self._prepare_prefill(seqs)
                logits = self.forward(ids, pos, ctx)
                rows = self._to_dev([q.row for q in seqs], torch.int64)
            elif graphable:
                slot = it % depth
                it += 1
                if staged[slot] is not None:
                    staged[slot].synchronize()
                a = staging[slot].numpy()
                a[:2 * n] = 0
                a[2 * n:3 * n] = -1
                a[3 * n:4 * n] = 0
                a[4 * n:] = -1
                a[:bs] = [q.row for q in seqs]
                a[n:n + bs] = [len(q) - 1 for q in seqs]
                a[2 * n:2 * n + bs] = [q.block_table[-1] * BLOCK_SIZE + (len(q) - 1) % BLOCK_SIZE for q in seqs]
                a[3 * n:3 * n + bs] = [len(q) for q in seqs]
                tab = a[4 * n:].reshape(n, max_blocks)
                for j, q in enumerate(seqs):
                    tab[j, :len(q.block_table)] = q.block_table
                self.g_meta.copy_(staging[slot], non_blocking=True)
                staged[slot] = torch.cuda.Event()
                staged[slot].record()
                bucket = next(b for b in self.graph_bs if b >= bs)
                self.g_i64.copy_(self.g_meta[:2 * n].view(2, n))
                torch.index_select(self.last_tok, 0, self.g_rows64[:bucket], out=self.g_ids[:bucket])
                self.graphs[bucket].replay()
                logits = self.op_linear(self.g_out[:bucket], self.embed)[:bs]
                rows = self.g_rows64[:bs]
            else:                                   # a batch no graph covers: this step runs the stepwise way
                drain()
                ids, pos, ctx = self._prepare_decode(seqs)
                logits = self.forward(ids, pos, ctx)
                rows = self._to_dev([q.row for q in seqs], torch.int64)
            tok = self.op_sampler_forward(logits, self.unit_temps[:bs])   # greedy: the temperature does not move the argmax
            self.last_tok.index_copy_(0, rows, tok)
            hist[len(steps), :bs] = tok
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            steps.append((len(steps), list(seqs), is_prefill, ev))
            for q in seqs:
                q.token_ids.append(-1)              # value pending; only the count matters to the scheduler
                if q.num_completion_tokens >= q.max_tokens:
                    self.running.remove(q)
                    self.free_blocks.extend(q.block_table)
                    q.block_table = []
                    self.free_rows.append(q.row)
                    q.row = -1
            if is_prefill:
                stats["prefill_steps"] += 1
                stats["prefill_tokens"] += sum(len(q) - 1 for q in seqs)
            else:
                stats["decode_steps"] += 1
                stats["decode_tokens"] += bs
        drain()

    def generate(self, prompts, max_tokens, temperature=0.6):
        """prompts: list of token-id lists; max_tokens: int or list.  Returns (completions, stats)."""
        if isinstance(max_tokens, int):
            max_tokens = [max_tokens] * len(prompts)
        order = []
        for p, m in zip(prompts, max_tokens):
            self.add_request(p, m, temperature)
            order.append(self.waiting[-1])
        stats = dict(prefill_steps=0, decode_steps=0, prefill_tokens=0, decode_tokens=0, prefill_s=0.0, decode_s=0.0)
        torch.cuda.synchronize(self.dev)
        t_all = time.perf_counter()
        if self.graphs and self.pipelined:
            self._generate_pipelined(stats)
        while self.waiting or self.running:     # stepwise: every step's tokens are read back before the next
            t0 = time.perf_counter()
            seqs, is_prefill, _ = self.step()
            dt = time.perf_counter() - t0
            if is_prefill:
                stats["prefill_steps"] += 1
                stats["prefill_tokens"] += sum(len(q) - 1 for q in seqs)
                stats["prefill_s"] += dt
            else:
                stats["decode_steps"] += 1
                stats["decode_tokens"] += len(seqs)
                stats["decode_s"] += dt
        stats["total_s"] = time.perf_counter() - t_all
        return [q.token_ids[q.num_prompt_tokens:] for q in order], stats
