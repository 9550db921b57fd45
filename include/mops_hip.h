/*
 * mops_hip.h — C ABI of libmops_hip.so: hand-written gfx950 (MI355X) kernels for the hot operators of
 * the `mops` operator library of nano_vllm_ninetoothed.
 *
 * Conventions for every launcher below
 *   - all pointers are DEVICE pointers unless stated; activations/caches/weights are bf16 (raw 16-bit
 *     words), metadata is int32 unless a flag says otherwise;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); the launch is asynchronous,
 *     nothing synchronises, nothing is allocated, nothing is freed;
 *   - return value: MOPS_HIP_OK (0) or a negative MOPS_HIP_E* status; on a negative status no kernel was
 *     launched.  Argument validation (null pointers, unsupported sizes, misalignment) happens on the host
 *     before launch, mirroring the reference's wrapper-side `assert`s.
 *
 * The reference has no native code: each entry point replaces the GPU kernel(s) behind one op name of
 * the reference's registry (mops/__init__.py:15-26), cited per function.
 */
#ifndef MOPS_HIP_H
#define MOPS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOPS_HIP_OK 0
#define MOPS_HIP_EINVAL (-1)       /* null pointer, negative size, inconsistent arguments            */
#define MOPS_HIP_EUNSUPPORTED (-2) /* shape the kernels are not written for (head_dim, block size…)  */
#define MOPS_HIP_EALIGN (-3)       /* pointer or stride breaks the 16-byte alignment the kernels need */
#define MOPS_HIP_EWORKSPACE (-4)   /* workspace missing or smaller than mops_hip_*_workspace_bytes    */
#define MOPS_HIP_ELAUNCH (-5)      /* a HIP call or launch reported an error (see mops_hip_last_hip_error) */
#define MOPS_HIP_ETOOLARGE (-6)    /* problem exceeds the fixed scratch of an allocation-free entry point */

/* ABI version of this header; bumped on any signature change. */
int mops_hip_abi_version(void);

/* Static, human-readable text for a status returned by any function here. */
const char* mops_hip_status_string(int status);

/* hipError_t (as int) of the last failed launch on this host thread, 0 if none. */
int mops_hip_last_hip_error(void);

/*
 * store_kvcache — slot_mapping scatter of freshly computed K and V rows into the paged cache.
 * Replaces: mops/triton/attention.py:7-38 (store_kvcache_kernel + wrapper), reached from
 * mops/torch/ops.py:62-65 and called at nanovllm/layers/attention.py:29.
 *
 *   for i in [0, n_tokens): s = slot_mapping[i]; if s == -1 skip;
 *       k_cache[s*row_elems : (s+1)*row_elems] = key[i*key_row_stride : +row_elems]   (same for V)
 *
 * key/value: rows of row_elems (= num_kv_heads*head_dim) contiguous bf16, row i at element offset
 * i*{key,value}_row_stride (strides in ELEMENTS, may exceed row_elems: V is a view into the qkv buffer).
 * k_cache/v_cache: contiguous [num_slots, row_elems].  Slots outside [0, num_slots) other than -1 are
 * skipped as well (the reference would write out of bounds).  Bit-exact copy.
 * Needs row_elems % 8 == 0, strides % 8 == 0 and 16-byte aligned base pointers.
 */
int mops_hip_store_kvcache(const void* key, int64_t key_row_stride,
                           const void* value, int64_t value_row_stride,
                           void* k_cache, void* v_cache,
                           const int32_t* slot_mapping,
                           int64_t n_tokens, int64_t row_elems, int64_t num_slots,
                           void* stream);

/*
 * embedding — row gather out[i, :] = weight[ids[i], :].
 * Replaces: mops/torch/ops.py:57-59 (F.embedding), mops/triton/embedding.py:6-50; called at
 * nanovllm/layers/embed_head.py:41.
 * ids: n_ids indices, int64 when ids_are_int64 != 0 else int32.  weight: [vocab, hidden] bf16 with row
 * stride weight_row_stride (elements).  out: contiguous [n_ids, hidden].  An id outside [0, vocab)
 * produces a zero row instead of a fault.  Bit-exact copy.  hidden % 8 == 0, stride % 8 == 0.
 */
int mops_hip_embedding(const void* ids, int ids_are_int64,
                       const void* weight, int64_t weight_row_stride,
                       void* out,
                       int64_t n_ids, int64_t vocab, int64_t hidden,
                       void* stream);

/*
 * rms_forward — y = bf16(bf16(x * rsqrt(mean(x^2) + eps)) * w), fp32 statistics, two bf16 roundings.
 * Replaces: mops/torch/ops.py:9-16, mops/triton/rms_forward.py:7-36; called at
 * nanovllm/layers/layernorm.py:21 (2-D hidden states and the 3-D strided q/k views of
 * nanovllm/models/qwen3.py:76-77).
 * x is addressed as x[(o*stride_outer + i*stride_inner) + 0..n) for o < rows_outer, i < rows_inner
 * (strides in elements); y is contiguous [rows_outer*rows_inner, n]; x is never written.
 * n % 8 == 0, n <= 16384, strides % 8 == 0.
 */
int mops_hip_rms_forward(const void* x, const void* weight, void* y,
                         int64_t rows_outer, int64_t rows_inner, int64_t n,
                         int64_t stride_outer, int64_t stride_inner,
                         float eps, void* stream);

/*
 * add_rms_forward — s = float(x) + float(residual); residual_out = bf16(s);
 *                   y = bf16(bf16(s * rsqrt(mean(s^2) + eps)) * w)   (statistics on the unrounded s).
 * Replaces: mops/torch/ops.py:18-30, mops/triton/add_rms_forward.py:7-39; called at
 * nanovllm/layers/layernorm.py:29.
 * x, residual: [rows, n] with row strides x_row_stride / residual_row_stride (elements); y and
 * residual_out contiguous [rows, n].  residual_out may alias residual (in-place convention of the
 * triton/ninetoothed backends) when residual is contiguous; y must not alias an input.
 */
int mops_hip_add_rms_forward(const void* x, int64_t x_row_stride,
                             const void* residual, int64_t residual_row_stride,
                             const void* weight,
                             void* y, void* residual_out,
                             int64_t rows, int64_t n,
                             float eps, void* stream);

/*
 * Paged decode attention (one query token per sequence against the block-table-addressed KV cache).
 * Replaces: flash_attn.flash_attn_with_kvcache as reached from mops/torch/ops.py:74-76 (semantics
 * spelled out in the commented torch version at mops/torch/ops.py:78-125) and the NineToothed kernel
 * mops/ninetoothed/attention.py:157-348; called at nanovllm/layers/attention.py:40-42.
 *
 *   out[b,h,:] = softmax_t( scale * q[b,h,:] . K[b,t,h/(hq/hkv),:] ) @ V[b,t,h/(hq/hkv),:],
 *   t in [0, cache_seqlens[b]),  token t at cache[block_table[b, t/block_size], t%block_size, kvhead, :]
 *
 * q: [batch, hq, 128] bf16, batch stride q_batch_stride elements (head stride 128).
 * k_cache/v_cache: contiguous [num_blocks, block_size, hkv, 128] bf16.
 * block_table: int32 [batch, *] with row stride block_table_row_stride, at least
 * max_blocks_per_seq columns; columns at or beyond ceil(cache_seqlens[b]/block_size) are never read
 * (they hold -1); an entry outside [0, num_blocks) inside the used range is treated as an empty block.
 * cache_seqlens[b] is clamped to [0, max_blocks_per_seq*block_size]; 0 gives a zero output row.
 * out: contiguous [batch, hq, 128] bf16.
 * workspace: device scratch of at least mops_hip_paged_decode_workspace_bytes(...) bytes, 256-byte
 * aligned, private to this call until it completes on `stream`.
 * Supported: head_dim 128, block_size a multiple of 32, hq/hkv <= 16, num_blocks >= 1.
 */
int64_t mops_hip_paged_decode_workspace_bytes(int64_t batch, int64_t hq, int64_t hkv,
                                              int64_t max_blocks_per_seq, int64_t block_size);

int mops_hip_attn_paged_decode_bf16(const void* q, int64_t q_batch_stride,
                                    const void* k_cache, const void* v_cache,
                                    const int32_t* cache_seqlens,
                                    const int32_t* block_table, int64_t block_table_row_stride,
                                    void* out,
                                    int64_t batch, int64_t hq, int64_t hkv, int64_t head_dim,
                                    int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                    float softmax_scale,
                                    void* workspace, int64_t workspace_bytes,
                                    void* stream);

/*
 * The same with the planning step under the caller's control.  The plan (how the KV stream of the batch is
 * cut over the workgroups) depends only on cache_seqlens, the batch and head counts and the block size, not
 * on q or on the caches, so the layers of one decode step can share it: call the first layer with
 * MOPS_HIP_DECODE_PLAN_AND_ATTEND and the others, on the same stream with the same workspace and the same
 * metadata, with MOPS_HIP_DECODE_REUSE_PLAN.  "The same metadata" means the same CONTENTS: a plan records the batch and
 * the head geometry it was made for (a call whose batch or heads differ is refused: its output is zeros), but not the
 * lengths.  If cache_seqlens or block_table have been rewritten in place since the planning call (same pointers, new
 * values, as a serving loop's static buffers are), MOPS_HIP_DECODE_REUSE_PLAN follows the old split: rows come out
 * truncated or zero, and nothing reports it.  Plan again whenever the contents may have changed (once per decode
 * step).  No counterpart in the reference (its attention call is per layer, nanovllm/layers/attention.py:40-42).
 */
#define MOPS_HIP_DECODE_PLAN_AND_ATTEND 0
#define MOPS_HIP_DECODE_REUSE_PLAN 1
int mops_hip_attn_paged_decode_planned_bf16(const void* q, int64_t q_batch_stride,
                                            const void* k_cache, const void* v_cache,
                                            const int32_t* cache_seqlens,
                                            const int32_t* block_table, int64_t block_table_row_stride,
                                            void* out,
                                            int64_t batch, int64_t hq, int64_t hkv, int64_t head_dim,
                                            int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                            float softmax_scale,
                                            void* workspace, int64_t workspace_bytes,
                                            int plan_mode, void* stream);

/*
 * Paged decode attention for callers that cannot allocate: code under HIP-graph capture, tight serving loops
 * that hold no workspace, harnesses that forbid hipMalloc.  No counterpart in the reference.  Arguments and
 * results are those of mops_hip_attn_paged_decode_bf16 (same kernels, bit-identical output) without the
 * workspace pair: the split-context partials live in a fixed device array inside the library, one copy of
 * MOPS_HIP_DECODE_NOALLOC_SCRATCH_BYTES per GPU, held until the process ends.  The call allocates and frees
 * nothing and does not synchronise.  A problem whose workspace (mops_hip_paged_decode_workspace_bytes) exceeds
 * that size returns MOPS_HIP_ETOOLARGE and launches nothing; both benchmark shapes fit (4.3 MB at 256
 * sequences x 16/8 heads, 8.5 MB at 512 x 32/8).  All calls on one GPU share that GPU's array: calls that
 * overlap in time on one GPU (different streams, or threads) race; calls on one stream are ordered and safe.
 * The first call on a GPU looks the array's device address up (hipGetSymbolAddress); make it outside capture.
 */
#define MOPS_HIP_DECODE_NOALLOC_SCRATCH_BYTES (16ll << 20)
int mops_hip_attn_paged_decode_noalloc_bf16(const void* q, int64_t q_batch_stride,
                                            const void* k_cache, const void* v_cache,
                                            const int32_t* cache_seqlens,
                                            const int32_t* block_table, int64_t block_table_row_stride,
                                            void* out,
                                            int64_t batch, int64_t hq, int64_t hkv, int64_t head_dim,
                                            int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                            float softmax_scale, void* stream);

/*
 * Varlen (packed, THD) causal prefill attention with grouped-query heads, with or without a cached prefix.
 * Replaces: flash_attn.flash_attn_varlen_func as reached from mops/torch/ops.py:70-72 and the Triton
 * kernel mops/triton/attention.py:42-146; called at nanovllm/layers/attention.py:34-37 (with the paged
 * caches as k/v and block_table set when a prefix-cache hit occurred, attention.py:32-33).
 *
 *   for sequence s with query tokens [cu_q[s], cu_q[s+1]) and Lk = cu_k[s+1]-cu_k[s] keys (Lk >= Lq):
 *     out[i,h,:] = softmax_{j <= i + (Lk-Lq)}( scale * q[i,h,:] . K_s[j,h/(hq/hkv),:] ) @ V_s[j,h/(hq/hkv),:]
 *
 * q/out: [total_tokens, hq, 128] bf16, token strides in elements (multiples of 8), head stride 128.
 * block_table == NULL: k/v are packed [total_k_tokens, hkv, 128] with their own token strides (multiples of 8,
 *   at most 2^24 elements: MOPS_HIP_EUNSUPPORTED beyond) and key j of sequence s is row cu_k[s] + j;
 *   cu_seqlens_k may be NULL (then it equals cu_seqlens_q).
 * block_table != NULL: k/v are the contiguous paged caches [num_blocks, block_size, hkv, 128] and key j of
 *   sequence s is cache[block_table[s, j/block_size], j%block_size] (row stride block_table_row_stride,
 *   at least max_blocks_per_seq columns; entries beyond the sequence's keys are never read; an entry
 *   outside [0, num_blocks) inside the used range is treated as an empty block, i.e. its keys get no weight,
 *   the rule of the decode entry points; block_size must be a multiple of 64); k/v token strides are ignored.
 * cu_seqlens_*: int32 [batch+1], non-decreasing, starting at 0.  max_seqlen_q bounds every query length
 * and only sizes the launch.  Sequences of length 0 are allowed.  softmax_scale may be any finite value
 * (0: uniform weights over the visible keys).  The scale is applied to the fp32 scores in fp32; with
 * MOPS_HIP_PREFILL_PRESCALE=1 in the environment (read at the first call) Q is multiplied by
 * softmax_scale * log2(e) once and rounded back to bf16 instead: faster, less accurate for large scores.
 * Accuracy: max-abs 2e-2 and mean-abs 2e-3 against an fp32 reference for scores of the benchmark's size
 * (softmax_scale 128^-1/2 on N(0,1) data: outputs below 2, one bf16 ulp <= 0.0156).  The bound is one bf16 ulp of the
 * output, so it scales with the outputs: at softmax_scale 1 on the same data the outputs reach 4 (ulp 0.031) and the
 * tests allow max-abs 4e-2 there.
 * Launches with an even hq / hkv, up to 512 sequences and up to 65536 tokens per sequence whose keys are the sequences'
 * own tokens, and launches behind a cached prefix (cu_seqlens_k or block_table given) with at most 64 sequences, at
 * most 512 new tokens per sequence on average and, when paged, at most 768 block table entries
 * (batch * max_blocks_per_seq), keep two workgroups per CU resident and hand them work items through counters in a
 * device array inside the library (128 rows, one per launch, round robin, cleared by the launch): at most 128 such
 * launches may be in flight per device; a launch captured into a HIP graph keeps its row.  MOPS_HIP_PREFILL_FORM=rows
 * (read at the first call) keeps every launch on the one-workgroup-per-128-rows form the other inputs take.
 */
int mops_hip_attn_varlen_causal_bf16(const void* q, int64_t q_token_stride,
                                     const void* k, int64_t k_token_stride,
                                     const void* v, int64_t v_token_stride,
                                     void* out, int64_t out_token_stride,
                                     const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                     const int32_t* block_table, int64_t block_table_row_stride,
                                     int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                     int64_t batch, int64_t total_tokens, int64_t total_k_tokens,
                                     int64_t max_seqlen_q,
                                     int64_t hq, int64_t hkv, int64_t head_dim,
                                     float softmax_scale,
                                     void* stream);

/*
 * siluAndMul — out = bf16( bf16(silu(x)) * y ), elementwise over [rows, n].
 * Replaces: mops/torch/ops.py:32-34 (F.silu(x) * y), mops/ninetoothed/activation.py:10-32; called at
 * nanovllm/layers/activation.py:16 with x, y the two halves of the gate_up projection (row strides in
 * elements; out contiguous [rows, n]).  n % 8 == 0, strides % 8 == 0.
 */
int mops_hip_silu_and_mul(const void* x, int64_t x_row_stride, const void* y, int64_t y_row_stride,
                          void* out, int64_t rows, int64_t n, void* stream);

/*
 * apply_rotary_emb — neox-style half-split rotation of x [tokens, heads, head_dim] bf16 by per-token
 * fp32 cos/sin rows of head_dim/2 values: y1 = x1*cos - x2*sin, y2 = x2*cos + x1*sin (fp32, products
 * rounded separately), out contiguous [tokens, heads, head_dim] bf16.
 * Replaces: mops/torch/ops.py:45-54, mops/ninetoothed/rotary_emb.py:10-65; called at
 * nanovllm/layers/rotary_embedding.py:35-36.  head_dim % 16 == 0.
 */
int mops_hip_apply_rotary_emb(const void* x, int64_t x_token_stride, int64_t x_head_stride,
                              const float* cos, int64_t cos_token_stride,
                              const float* sin, int64_t sin_token_stride,
                              void* out, int64_t tokens, int64_t heads, int64_t head_dim, void* stream);

/*
 * sampler_forward — out[r] = argmax(softmax(logits[r, :] / temperature[r])) for positive temperatures, i.e.
 * the index of the row's largest logit (first index on ties).  The temperatures do not change the result
 * and are not passed.  A row holding a NaN or +inf logit, or only -inf, gives 0: the library softmax turns such a row
 * into NaNs and its argmax of an all-NaN row is 0.  Not reproduced: temperatures <= 0 (the library expression yields
 * inf/NaN garbage) and logits so close to zero that they collide after the fp32 division and exponential
 * (|logit| / T below ~1e-5, where every candidate is equally tiny).  Replaces: mops/torch/ops.py:37-43 (greedy: the Gumbel line is commented out),
 * mops/ninetoothed/sampler_forward.py:9-94; called at nanovllm/layers/sampler.py:12.
 * logits: [rows, n] bf16 with row stride in elements (% 8 == 0); out: int64 [rows].
 */
int mops_hip_sampler_argmax(const void* logits, int64_t row_stride, int64_t* out, int64_t rows, int64_t n,
                            void* stream);

/*
 * An empty kernel on `stream`: what one launch costs on this device with nothing to do.  No counterpart in the
 * reference; it exists so that the durations of the small operators (norms, embedding at decode sizes) can be read
 * against a measured floor (bench.py --op launch_floor).
 */
int mops_hip_launch_floor(void* stream);

/*
 * qk_norm_rope_store — the four small steps between the qkv projection and the attention call of a Qwen3
 * layer as one launch: per-head RMSNorm of q and k, rotary embedding of both, scatter of k and v into the
 * paged cache.  Replaces the sequence nanovllm/models/qwen3.py:74-80 (q_norm, k_norm, rotary_emb) +
 * nanovllm/layers/attention.py:29-31 (store_kvcache), i.e. mops rms_forward x2, apply_rotary_emb x2 and
 * store_kvcache, and is bit-identical to running those (same roundings in the same order).
 * qkv: [tokens, (hq + 2*hkv) * 128] bf16, q heads first, then k, then v, token stride in elements (% 8 == 0);
 * q_weight, k_weight: [128] bf16; cos, sin: fp32 [tokens, 64] with token strides; slot_mapping: int32 [tokens],
 * -1 or out of range = skip the cache rows of that token; q_out: [tokens, hq, 128] bf16; k_out: [tokens, hkv, 128]
 * bf16 or NULL when the rotated keys are only needed in the cache (decode); caches: [num_slots, hkv, 128] bf16.
 * v is not copied out: the attention call reads it from qkv as a strided view.
 */
int mops_hip_qk_norm_rope_store(const void* qkv, int64_t qkv_token_stride, const void* q_weight,
                                const void* k_weight, const float* cos, int64_t cos_token_stride,
                                const float* sin, int64_t sin_token_stride,
                                const int32_t* slot_mapping, void* q_out, void* k_out, void* k_cache,
                                void* v_cache, int64_t tokens, int64_t hq, int64_t hkv, int64_t head_dim,
                                int64_t num_slots, float eps, void* stream);

/*
 * linear — y = x . W^T (+ bias), bf16 in and out, fp32 accumulation, as a library GEMM (hipBLASLt).
 * Replaces: mops/torch/ops.py:5-7 (F.linear), called from nanovllm/layers/linear.py:53,75,152 and
 * nanovllm/layers/embed_head.py:64.
 * x: [m, k] bf16, w: [n, k] bf16 (nn.Linear layout), y: [m, n] bf16, row strides in elements (% 8 == 0, as
 * are n and k); bias: [n] bf16 or NULL.  workspace: device scratch for solutions that split k (may be NULL
 * with workspace_bytes 0; solutions that need more than is given are not chosen).
 * The solution is the one pinned for (m, n, k) with mops_hip_linear_pin_solution if it supports the
 * problem; without a pin for m, the one pinned for the next larger row count with the same n and k; else the
 * first the library's heuristic returns.  Unlike the kernels above this entry point keeps
 * host-side state (a library handle per device, one descriptor per distinct shape).
 */
int mops_hip_linear_bf16(const void* x, int64_t x_row_stride, const void* w, int64_t w_row_stride,
                         const void* bias, void* y, int64_t y_row_stride,
                         int64_t m, int64_t n, int64_t k,
                         void* workspace, int64_t workspace_bytes, void* stream);

/* Pins the library solution `solution_index` (as returned by mops_hip_linear_tune on the same library
 * version) for problems with these m, n, k; a negative index removes the pin.  Host-only, no GPU work. */
int mops_hip_linear_pin_solution(int64_t m, int64_t n, int64_t k, int solution_index);

/*
 * Times every solution the library offers for (m, n, k) on `distinct_weights` different weight matrices used
 * in turn (so that none is served from cache, as in a decode step that walks through the layers), `rounds`
 * passes per measurement, and returns the index of the fastest, its time per GEMM in microseconds, and the
 * time of the heuristic's choice.  A set-up utility: it allocates and frees its own buffers, creates a
 * stream and synchronises; not for use on a hot path or under stream capture.  No counterpart in the
 * reference.
 */
int mops_hip_linear_tune(int64_t m, int64_t n, int64_t k, int64_t distinct_weights, int rounds,
                         void* workspace, int64_t workspace_bytes,
                         int* best_solution_index, float* best_us, float* heuristic_us);

#ifdef __cplusplus
}
#endif
#endif /* MOPS_HIP_H */
