"""The `hip` backend: the six hot operators, plus siluAndMul, apply_rotary_emb and sampler_forward, run
hand-written gfx950 kernels through the C ABI of libmops_hip.so; linear is a library GEMM (hipBLASLt through
the same C ABI for the decode-sized problems, torch otherwise) and softmax a library-torch delegate.

Every function keeps the name and call form the reference's layers use (nanovllm/layers/attention.py:29-42,
layernorm.py:21,29, embed_head.py:41).  Wrappers validate layouts with exceptions before launching
(the reference asserts in its wrappers, mops/triton/attention.py:34-37), allocate outputs with the torch
allocator, launch on the current torch stream and never synchronise.
"""
from __future__ import annotations

import math

import torch

from ... import _capi
from .registry import register_hip_op


# The raw handle of the current stream of a device.  In the reference's own setting (eager, one Python call per op) the
# host side of a decode step costs as much as its kernels, so the wrappers keep their per-call work small: this
# lookup is 0.1 us where torch.cuda.current_stream(...).cuda_stream is 2 us, messages are only formatted on failure.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_of(device: torch.device) -> int:
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _stream(t: torch.Tensor) -> int:
    return _stream_of(t.device)


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _require_cuda_bf16(name: str, t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU")
    if t.dtype != torch.bfloat16:
        raise ValueError(f"{name} must be bfloat16, got {t.dtype}")


# ----------------------------------------------------------------------------------------------------
# hot ops: HIP kernels
# ----------------------------------------------------------------------------------------------------

@register_hip_op
def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """Scatter of K/V rows into the paged cache; layout rules of mops/triton/attention.py:30-38."""
    _require(key.dim() == 3 and value.shape == key.shape, "key/value must be [N, num_kv_heads, head_dim]")
    n, num_heads, head_dim = key.shape
    d = num_heads * head_dim
    for name, t in (("key", key), ("value", value), ("k_cache", k_cache), ("v_cache", v_cache)):
        _require_cuda_bf16(name, t)
    _require(key.stride(-1) == 1 and value.stride(-1) == 1, "key/value last dim must be contiguous")
    _require(key.stride(1) == head_dim and value.stride(1) == head_dim, "key/value head stride must be head_dim")
    _require(k_cache.dim() == 4 and v_cache.shape == k_cache.shape, "caches must be [blocks, block_size, heads, dim]")
    _require(k_cache.stride(1) == d and v_cache.stride(1) == d, "cache token stride must be num_kv_heads*head_dim")
    _require(k_cache.is_contiguous() and v_cache.is_contiguous(), "caches must be contiguous")
    _require(slot_mapping.numel() == n, "slot_mapping must have one entry per token")
    _require(slot_mapping.dtype == torch.int32 and slot_mapping.is_cuda and slot_mapping.is_contiguous(),
             "slot_mapping must be a contiguous int32 GPU tensor")
    lib = _capi.load()
    num_slots = k_cache.shape[0] * k_cache.shape[1]
    st = lib.mops_hip_store_kvcache(key.data_ptr(), key.stride(0) if n > 1 else max(key.stride(0), d),
                                    value.data_ptr(), value.stride(0) if n > 1 else max(value.stride(0), d),
                                    k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(),
                                    n, d, num_slots, _stream(key))
    _capi.check("mops_hip_store_kvcache", st)


@register_hip_op
def embedding(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """Row gather with the result shape of F.embedding (mops/torch/ops.py:57-59)."""
    _require_cuda_bf16("weight", weight)
    _require(weight.dim() == 2 and weight.stride(1) == 1, "weight must be [vocab, hidden] with contiguous rows")
    _require(x.is_cuda and x.dtype in (torch.int32, torch.int64), "ids must be an int32/int64 GPU tensor")
    ids = x if x.is_contiguous() else x.contiguous()
    vocab, hidden = weight.shape
    out = torch.empty((*x.shape, hidden), dtype=weight.dtype, device=weight.device)
    lib = _capi.load()
    st = lib.mops_hip_embedding(ids.data_ptr(), 1 if ids.dtype == torch.int64 else 0, weight.data_ptr(),
                                weight.stride(0), out.data_ptr(), ids.numel(), vocab, hidden, _stream(weight))
    _capi.check("mops_hip_embedding", st)
    return out


def _row_view(x: torch.Tensor):
    """Describes x[..., n] as rows_outer x rows_inner rows with two element strides, or returns None."""
    n = x.shape[-1]
    if x.stride(-1) != 1 and n > 1:
        return None
    lead = [(s, st) for s, st in zip(x.shape[:-1], x.stride()[:-1]) if s != 1]
    # merge adjacent leading dims that are contiguous with each other
    merged: list[list[int]] = []
    for size, stride in lead:
        if merged and merged[-1][1] == stride * size:
            merged[-1][0] *= size
            merged[-1][1] = stride
        else:
            merged.append([size, stride])
    if len(merged) == 0:
        return 1, 1, n, n
    if len(merged) == 1:
        return 1, merged[0][0], 0, merged[0][1]
    if len(merged) == 2:
        return merged[0][0], merged[1][0], merged[0][1], merged[1][1]
    return None


@register_hip_op
def rms_forward(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm returning a new tensor (mops/torch/ops.py:9-16); strided 3-D views are read in place."""
    _require_cuda_bf16("x", x)
    _require_cuda_bf16("weight", weight)
    n = x.shape[-1]
    _require(weight.dim() == 1 and weight.shape[0] == n and weight.is_contiguous(), "weight must be [n] contiguous")
    view = _row_view(x) if x.numel() else (0, 0, 0, 0)
    if view is None:
        x = x.contiguous()
        view = _row_view(x)
    rows_outer, rows_inner, stride_outer, stride_inner = view
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    lib = _capi.load()
    st = lib.mops_hip_rms_forward(x.data_ptr(), weight.data_ptr(), y.data_ptr(), rows_outer, rows_inner, n,
                                  stride_outer, stride_inner, float(eps), _stream(x))
    _capi.check("mops_hip_rms_forward", st)
    return y


@register_hip_op
def add_rms_forward(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """Fused residual add + RMSNorm; returns (y, new_residual) as new tensors (mops/torch/ops.py:18-30)."""
    _require_cuda_bf16("x", x)
    _require_cuda_bf16("residual", residual)
    _require_cuda_bf16("weight", weight)
    _require(x.shape == residual.shape, "x and residual must have the same shape")
    n = x.shape[-1]
    _require(weight.dim() == 1 and weight.shape[0] == n and weight.is_contiguous(), "weight must be [n] contiguous")
    x2 = x if x.dim() == 2 else x.reshape(-1, n)
    r2 = residual if residual.dim() == 2 else residual.reshape(-1, n)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    if r2.stride(1) != 1:
        r2 = r2.contiguous()
    rows = x2.shape[0]
    if x.is_contiguous():
        y, r_out = torch.empty_like(x), torch.empty_like(x)
    else:
        y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        r_out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    lib = _capi.load()
    st = lib.mops_hip_add_rms_forward(x2.data_ptr(), x2.stride(0) if rows > 1 else n, r2.data_ptr(),
                                      r2.stride(0) if rows > 1 else n, weight.data_ptr(), y.data_ptr(),
                                      r_out.data_ptr(), rows, n, float(eps), _stream(x))
    _capi.check("mops_hip_add_rms_forward", st)
    return y, r_out


_workspaces: dict = {}          # (device index, stream handle) -> current scratch tensor
_retired_workspaces: list = []  # superseded scratch tensors: captured graphs may still hold their addresses
_last_plan: dict = {}           # (device index, stream handle) -> description of the plan the scratch holds


def _workspace_key(device: torch.device):
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    return (device.index, _stream_of(device))


def _decode_workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Per-(device, stream) scratch for split-context partials, reused across calls on the same stream
    (kernels on one stream run in order, so reuse cannot race).  It grows on demand; a buffer that has been
    handed out is never freed, because a captured HIP graph replays with the address it was captured with.
    Callers that capture graphs size it once with reserve_decode_workspace() before the first capture."""
    key = _workspace_key(device)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired_workspaces.append(ws)
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
        _last_plan.pop(key, None)
    return ws


def reserve_decode_workspace(max_batch: int, hq: int, hkv: int, max_blocks: int, block_size: int = 256,
                             device=None) -> int:
    """Sizes the current stream's paged-decode scratch (scratch is kept per stream: make the stream that will
    capture current first) for problems of up to max_batch sequences, so that no later
    flash_attn_with_kvcache call on this stream with at most that many sequences allocates (the scratch size grows
    with the batch only).  Call it before capturing HIP graphs: captures of any batch size, in any order, then
    share one buffer that stays where it is.  Returns the size in bytes."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    nbytes = _capi.load().mops_hip_paged_decode_workspace_bytes(max_batch, hq, hkv, max_blocks, block_size)
    _require(nbytes > 0, "reserve_decode_workspace: sizes must be positive")
    _linear_workspace(device)   # the GEMM scratch of this stream has a fixed size; make it exist as well
    return _decode_workspace(device, nbytes).numel()


@register_hip_op
def flash_attn_with_kvcache(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cache_seqlens=None,
                            block_table=None, softmax_scale=None, causal=True, reuse_plan: bool = False,
                            **kwargs) -> torch.Tensor:
    """Paged decode attention, q [B, 1, Hq, D] -> [B, 1, Hq, D] (call form: nanovllm/layers/attention.py:40-42).

    reuse_plan (extension): skip the planning kernel and use the split the last planning call on this stream left
    in the scratch.  Only valid when that call had the same cache_seqlens and block_table tensors and the same
    head geometry, i.e. for layers 2..N of one decode step; anything else raises ValueError.  (The kernels
    themselves refuse a plan whose recorded batch or head geometry differs from their launch and write zeros.)
    The check compares tensors by address and shape, not by value: cache_seqlens and block_table must also still
    HOLD what the planning call saw.  A caller that rewrites them in place (static graph buffers) and then passes
    reuse_plan=True without planning again gets the old split applied to the new lengths - truncated or zero rows,
    silently.  Plan once per decode step, as the engine counterpart does at layer 0."""
    if kwargs:
        raise ValueError(f"unsupported arguments: {sorted(kwargs)}")
    _require(cache_seqlens is not None and block_table is not None, "cache_seqlens and block_table are required")
    _require_cuda_bf16("q", q)
    _require_cuda_bf16("k_cache", k_cache)
    _require_cuda_bf16("v_cache", v_cache)
    _require(q.dim() == 4 and q.shape[1] == 1, "q must be [batch, 1, heads, head_dim] (one query token per sequence)")
    batch, _, hq, d = q.shape
    _require(k_cache.dim() == 4 and k_cache.shape == v_cache.shape, "caches must be [blocks, block_size, kv_heads, dim]")
    _require(k_cache.is_contiguous() and v_cache.is_contiguous(), "caches must be contiguous")
    num_blocks, block_size, hkv, dk = k_cache.shape
    _require(dk == d and hq % hkv == 0, "head_dim / head-count mismatch between q and the cache")
    _require(q.stride(3) == 1 and q.stride(2) == d, "q heads must be contiguous")
    _require(cache_seqlens.dtype == torch.int32 and cache_seqlens.is_cuda and cache_seqlens.is_contiguous()
             and cache_seqlens.numel() == batch, "cache_seqlens must be a contiguous int32 GPU tensor of [batch]")
    _require(block_table.dtype == torch.int32 and block_table.is_cuda and block_table.dim() == 2
             and block_table.shape[0] == batch and block_table.stride(1) == 1,
             "block_table must be an int32 GPU tensor [batch, max_blocks] with contiguous rows")
    scale = float(softmax_scale) if softmax_scale is not None else 1.0 / math.sqrt(d)
    max_blocks = block_table.shape[1]
    out = torch.empty((batch, 1, hq, d), dtype=q.dtype, device=q.device)
    lib = _capi.load()
    nbytes = lib.mops_hip_paged_decode_workspace_bytes(batch, hq, hkv, max_blocks, block_size)
    ws = _decode_workspace(q.device, nbytes)
    # what the plan in the scratch depends on; a reused plan must have been made for exactly this
    plan = (ws.data_ptr(), batch, hq, hkv, block_size, cache_seqlens.data_ptr(), block_table.data_ptr(), tuple(block_table.shape))
    key = _workspace_key(q.device)
    if reuse_plan:
        _require(_last_plan.get(key) == plan,
                 "reuse_plan=True, but the last planning call on this stream was made for another batch, head geometry, "
                 "cache_seqlens or block_table (or there was none)")
    else:
        _last_plan[key] = plan
    st = lib.mops_hip_attn_paged_decode_planned_bf16(q.data_ptr(), q.stride(0) if batch > 1 else hq * d, k_cache.data_ptr(),
                                                     v_cache.data_ptr(), cache_seqlens.data_ptr(), block_table.data_ptr(),
                                                     block_table.stride(0) if batch > 1 else max_blocks, out.data_ptr(),
                                                     batch, hq, hkv, d, block_size, num_blocks, max_blocks, scale,
                                                     ws.data_ptr(), ws.numel(), 1 if reuse_plan else 0, _stream(q))
    _capi.check("mops_hip_attn_paged_decode_planned_bf16", st)
    return out


@register_hip_op
def flash_attn_varlen_func(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, max_seqlen_q=None, cu_seqlens_q=None,
                           max_seqlen_k=None, cu_seqlens_k=None, softmax_scale=None, causal=True, block_table=None,
                           **kwargs) -> torch.Tensor:
    """Varlen causal prefill attention over packed [T, H, D] queries (call form: nanovllm/layers/attention.py:34-37).
    With block_table given, k and v are the paged caches and each sequence's keys are its cu_seqlens_k span
    (cached prefix + new tokens), masked bottom-right aligned."""
    if kwargs:
        raise ValueError(f"unsupported arguments: {sorted(kwargs)}")
    _require(causal, "only causal attention is implemented")
    _require(cu_seqlens_q is not None and max_seqlen_q is not None, "cu_seqlens_q and max_seqlen_q are required")
    _require_cuda_bf16("q", q)
    _require(q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == q.shape[2], "q must be [T, H, D] with contiguous heads")
    total, hq, d = q.shape
    _require(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.is_cuda and cu_seqlens_q.is_contiguous(),
             "cu_seqlens_q must be a contiguous int32 GPU tensor")
    batch = cu_seqlens_q.numel() - 1
    if cu_seqlens_k is not None:
        _require(cu_seqlens_k.dtype == torch.int32 and cu_seqlens_k.is_cuda and cu_seqlens_k.is_contiguous()
                 and cu_seqlens_k.shape == cu_seqlens_q.shape, "cu_seqlens_k must be an int32 GPU tensor shaped like cu_seqlens_q")
    scale = float(softmax_scale) if softmax_scale is not None else 1.0 / math.sqrt(d)
    out = torch.empty((total, hq, d), dtype=q.dtype, device=q.device)
    lib = _capi.load()
    cu_k_ptr = cu_seqlens_k.data_ptr() if cu_seqlens_k is not None else None
    if block_table is None:
        for name, t in (("k", k), ("v", v)):
            _require_cuda_bf16(name, t)
            _require(t.dim() == 3 and t.stride(2) == 1 and t.stride(1) == t.shape[2], f"{name} must be [T, H, D] with contiguous heads")
        _require(k.shape == v.shape and k.shape[2] == d, "k/v must be [Tk, Hkv, D] matching q's head_dim")
        total_k, hkv = k.shape[0], k.shape[1]
        _require(cu_seqlens_k is not None or total_k == total, "k/v must have as many tokens as q when cu_seqlens_k is not given")
        ks = k.stride(0) if total_k > 1 else hkv * d
        vs = v.stride(0) if total_k > 1 else hkv * d
        bt_ptr, bt_stride, bs, nblk, maxblk = None, 0, 0, 0, 0
    else:
        _require(cu_seqlens_k is not None, "cu_seqlens_k is required with block_table")
        for name, t in (("k_cache", k), ("v_cache", v)):
            _require_cuda_bf16(name, t)
            _require(t.dim() == 4 and t.is_contiguous() and t.shape[3] == d, f"{name} must be a contiguous [blocks, block_size, kv_heads, D] cache")
        _require(k.shape == v.shape, "k_cache and v_cache must have the same shape")
        nblk, bs, hkv, _ = k.shape
        _require(block_table.dtype == torch.int32 and block_table.is_cuda and block_table.dim() == 2
                 and block_table.shape[0] == batch and block_table.stride(1) == 1,
                 "block_table must be an int32 GPU tensor [batch, max_blocks] with contiguous rows")
        maxblk = block_table.shape[1]
        bt_ptr, bt_stride = block_table.data_ptr(), (block_table.stride(0) if batch > 1 else maxblk)
        total_k, ks, vs = 0, 0, 0
    _require(hq % hkv == 0, "query heads must be a multiple of kv heads")
    st = lib.mops_hip_attn_varlen_causal_bf16(q.data_ptr(), q.stride(0) if total > 1 else hq * d, k.data_ptr(), ks,
                                              v.data_ptr(), vs, out.data_ptr(), hq * d, cu_seqlens_q.data_ptr(), cu_k_ptr,
                                              bt_ptr, bt_stride, bs, nblk, maxblk, batch, total, total_k, int(max_seqlen_q),
                                              hq, hkv, d, scale, _stream(q))
    _capi.check("mops_hip_attn_varlen_causal_bf16", st)
    return out


# ----------------------------------------------------------------------------------------------------
# remaining registry names: the two per-layer elementwise ops have kernels of their own; linear, sampler
# and softmax are library torch on the GPU, as in mops/torch/ops.py:5-7,37-43
# ----------------------------------------------------------------------------------------------------

_LINEAR_MAX_ROWS = 1024          # above this the GEMM is compute-bound and goes to the library through torch
_LINEAR_WORKSPACE_BYTES = 32 << 20
_linear_workspaces: dict = {}
_linear_pins_loaded = False


def _linear_workspace(device: torch.device) -> torch.Tensor:
    key = _workspace_key(device)
    ws = _linear_workspaces.get(key)
    if ws is None:
        ws = torch.empty(_LINEAR_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _linear_workspaces[key] = ws
    return ws


def load_linear_solutions(path=None) -> int:
    """Pins the hipBLASLt solutions listed in a file written by `python -m nano_vllm_ninetoothed_amd.tune_linear`
    (default: the table shipped in the package, measured on MI355X).  A table made with another library
    version or for another GPU architecture is ignored: solution indices do not carry over.  Returns the number of shapes pinned."""
    import json
    from pathlib import Path
    path = Path(path) if path is not None else Path(__file__).resolve().parents[2] / "data" / "linear_solutions_gfx950.json"
    if not path.exists():
        return 0
    table = json.loads(path.read_text())
    arch = torch.cuda.get_device_properties(torch.cuda.current_device()).gcnArchName.split(":")[0]
    if table.get("hip_version") != torch.version.hip or table.get("arch") != arch:
        return 0
    lib = _capi.load()
    for m, n, k, index in table["solutions"]:
        _capi.check("mops_hip_linear_pin_solution", lib.mops_hip_linear_pin_solution(m, n, k, index))
    return len(table["solutions"])


_linear_fn = None   # the bound C entry point, looked up once


@register_hip_op
def linear(x, weight, bias=None):
    """x @ weight.T (+ bias) (mops/torch/ops.py:5-7).  A library GEMM either way: bf16 problems with up to
    1024 rows (the decode step's projections, the lm head) call hipBLASLt through the C ABI, which lets a
    solution measured on cold weights be pinned per shape; everything else goes through torch."""
    global _linear_pins_loaded, _linear_fn
    # The decode step calls this 113 times with a 2-D activation and a weight seen before: what the general path below
    # found out about the weight (shape, row stride, address, that it qualifies) is kept on the tensor, and the call is
    # the checks that can change from call to call, the output allocation and the C call.
    info = getattr(weight, "_mops_linear_info", None)
    if info is not None and bias is None and x.dim() == 2:
        n, k, ldw, wptr = info
        m = x.shape[0]
        if (x.dtype is torch.bfloat16 and x.is_cuda and x.shape[1] == k and 0 < m <= _LINEAR_MAX_ROWS and x.stride(1) == 1
                and weight.data_ptr() == wptr):
            ldx = x.stride(0) if m > 1 else k
            xptr = x.data_ptr()
            if ldx % 8 == 0 and xptr % 16 == 0:
                y = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
                ws = _linear_workspace(x.device)
                st = _linear_fn(xptr, ldx, wptr, ldw, None, y.data_ptr(), n, m, n, k, ws.data_ptr(), _LINEAR_WORKSPACE_BYTES,
                                _stream_of(x.device))
                if st:
                    _capi.check("mops_hip_linear_bf16", st)
                return y
    if (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.stride(1) == 1 and x.dim() >= 1 and x.shape[-1] == weight.shape[1]
            and (bias is None or (bias.dtype == torch.bfloat16 and bias.is_contiguous() and bias.numel() == weight.shape[0]))):
        n, k = weight.shape
        x2 = x.reshape(-1, k)
        if x2.stride(1) != 1:
            x2 = x2.contiguous()
        m = x2.shape[0]
        ldx = x2.stride(0) if m > 1 else k
        ldw = weight.stride(0) if n > 1 else k
        if (0 < m <= _LINEAR_MAX_ROWS and k % 8 == 0 and n % 8 == 0 and ldx % 8 == 0 and ldw % 8 == 0
                and x2.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0 and (bias is None or bias.data_ptr() % 16 == 0)):
            if not _linear_pins_loaded:
                _linear_pins_loaded = True
                load_linear_solutions()
            if _linear_fn is None:
                _linear_fn = _capi.load().mops_hip_linear_bf16
            if bias is None and weight.is_contiguous():
                try:
                    weight._mops_linear_info = (n, k, ldw, weight.data_ptr())
                except (AttributeError, RuntimeError):
                    pass   # a tensor that takes no attributes keeps the general path
            y = torch.empty((m, n), dtype=x.dtype, device=x.device)
            ws = _linear_workspace(x.device)
            st = _capi.load().mops_hip_linear_bf16(x2.data_ptr(), ldx, weight.data_ptr(), ldw,
                                                   bias.data_ptr() if bias is not None else None, y.data_ptr(), n, m, n, k,
                                                   ws.data_ptr(), ws.numel(), _stream(x))
            _capi.check("mops_hip_linear_bf16", st)
            return y.view(*x.shape[:-1], n)
    return torch.nn.functional.linear(x, weight, bias)


@register_hip_op
def siluAndMul(x: torch.Tensor, y: torch.Tensor):
    """silu(x) * y with the two bf16 roundings of the library expression (mops/torch/ops.py:32-34); x and y
    are usually the two halves of one gate_up buffer and are read in place."""
    _require_cuda_bf16("x", x)
    _require_cuda_bf16("y", y)
    _require(x.shape == y.shape, "x and y must have the same shape")
    n = x.shape[-1]
    x2, y2 = x.reshape(-1, n), y.reshape(-1, n)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    if y2.stride(1) != 1:
        y2 = y2.contiguous()
    rows = x2.shape[0]
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    st = _capi.load().mops_hip_silu_and_mul(x2.data_ptr(), x2.stride(0) if rows > 1 else n, y2.data_ptr(),
                                            y2.stride(0) if rows > 1 else n, out.data_ptr(), rows, n, _stream(x))
    _capi.check("mops_hip_silu_and_mul", st)
    return out


@register_hip_op
def sampler_forward(logits: torch.Tensor, temperatures: torch.Tensor):
    """argmax(softmax(logits / T)) per row -> int64 [B] (mops/torch/ops.py:37-43; the reference samples
    greedily).  For positive temperatures that is the index of the largest logit (the first on ties), computed in
    one pass over the bf16 logits; a row with a NaN or +inf logit gives 0, as the library expression does.
    Assumes temperatures > 0: with T <= 0 the reference's expression produces inf/NaN garbage, which is not
    reproduced.  Other dtypes and layouts take the library expression."""
    if logits.is_cuda and logits.dtype == torch.bfloat16 and logits.dim() == 2 and logits.stride(1) == 1 \
            and logits.stride(0) % 8 == 0 and logits.data_ptr() % 16 == 0:
        rows, n = logits.shape
        out = torch.empty((rows,), dtype=torch.int64, device=logits.device)
        st = _capi.load().mops_hip_sampler_argmax(logits.data_ptr(), logits.stride(0) if rows > 1 else max(n, (n + 7) // 8 * 8),
                                                  out.data_ptr(), rows, n, _stream(logits))
        _capi.check("mops_hip_sampler_argmax", st)
        return out
    scaled = logits.float().div_(temperatures.unsqueeze(dim=1))
    return torch.argmax(torch.softmax(scaled, dim=-1), dim=-1)


@register_hip_op
def apply_rotary_emb(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Half-split rotary embedding, x [T, H, D] bf16, cos/sin [T, 1, D/2] fp32 (mops/torch/ops.py:45-54)."""
    _require_cuda_bf16("x", x)
    _require(x.dim() == 3 and x.stride(2) == 1, "x must be [tokens, heads, head_dim] with contiguous head_dim")
    t, h, d = x.shape
    _require(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_cuda and sin.is_cuda, "cos/sin must be fp32 GPU tensors")
    _require(cos.shape == sin.shape and cos.numel() == t * (d // 2) and cos.shape[-1] == d // 2 and cos.stride(-1) == 1
             and sin.stride(-1) == 1, "cos/sin must be [tokens, 1, head_dim/2] with a contiguous last dim")
    out = torch.empty((t, h, d), dtype=x.dtype, device=x.device)
    st = _capi.load().mops_hip_apply_rotary_emb(x.data_ptr(), x.stride(0) if t > 1 else h * d, x.stride(1) if h > 1 else d,
                                                cos.data_ptr(), cos.stride(0) if t > 1 else d // 2,
                                                sin.data_ptr(), sin.stride(0) if t > 1 else d // 2,
                                                out.data_ptr(), t, h, d, _stream(x))
    _capi.check("mops_hip_apply_rotary_emb", st)
    return out


@register_hip_op
def qk_norm_rope_store(qkv: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor, eps: float,
                       cos: torch.Tensor, sin: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                       slot_mapping: torch.Tensor, num_heads: int, num_kv_heads: int, need_k: bool = True):
    """Extension op (not one of the reference's eleven): q_norm, k_norm, rotary embedding of q and k and
    store_kvcache of the rotated k and of v in one launch; bit-identical to
    rms_forward x2 -> apply_rotary_emb x2 -> store_kvcache (nanovllm/models/qwen3.py:74-80,
    nanovllm/layers/attention.py:29-31).  qkv is the [tokens, (Hq + 2*Hkv) * 128] output of the qkv projection.
    Returns (q [tokens, Hq, 128], k [tokens, Hkv, 128] or None when need_k is False, v as a view of qkv)."""
    _require_cuda_bf16("qkv", qkv)
    for name, t in (("q_weight", q_weight), ("k_weight", k_weight), ("k_cache", k_cache), ("v_cache", v_cache)):
        _require_cuda_bf16(name, t)
    head_dim = q_weight.numel()
    heads = num_heads + 2 * num_kv_heads
    _require(qkv.dim() == 2 and qkv.shape[1] == heads * head_dim and qkv.stride(1) == 1, "qkv must be [tokens, (Hq + 2*Hkv) * head_dim]")
    _require(k_weight.numel() == head_dim and q_weight.is_contiguous() and k_weight.is_contiguous(), "norm weights must be [head_dim]")
    t = qkv.shape[0]
    half = head_dim // 2
    _require(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_cuda and sin.is_cuda, "cos/sin must be fp32 GPU tensors")
    _require(cos.shape == sin.shape and cos.numel() == t * half and cos.shape[-1] == half and cos.stride(-1) == 1
             and sin.stride(-1) == 1, "cos/sin must be [tokens, 1, head_dim/2] with a contiguous last dim")
    _require(k_cache.dim() == 4 and v_cache.shape == k_cache.shape and k_cache.is_contiguous() and v_cache.is_contiguous()
             and k_cache.shape[2] == num_kv_heads and k_cache.shape[3] == head_dim, "caches must be contiguous [blocks, block_size, Hkv, head_dim]")
    _require(slot_mapping.numel() == t and slot_mapping.dtype == torch.int32 and slot_mapping.is_cuda and slot_mapping.is_contiguous(),
             "slot_mapping must be a contiguous int32 GPU tensor with one entry per token")
    q = torch.empty((t, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    k = torch.empty((t, num_kv_heads, head_dim), dtype=qkv.dtype, device=qkv.device) if need_k else None
    st = _capi.load().mops_hip_qk_norm_rope_store(
        qkv.data_ptr(), qkv.stride(0) if t > 1 else heads * head_dim, q_weight.data_ptr(), k_weight.data_ptr(),
        cos.data_ptr(), cos.stride(0) if t > 1 else half, sin.data_ptr(), sin.stride(0) if t > 1 else half,
        slot_mapping.data_ptr(), q.data_ptr(), k.data_ptr() if need_k else None, k_cache.data_ptr(), v_cache.data_ptr(),
        t, num_heads, num_kv_heads, head_dim, k_cache.shape[0] * k_cache.shape[1], float(eps), _stream(qkv))
    _capi.check("mops_hip_qk_norm_rope_store", st)
    v = qkv[:, (num_heads + num_kv_heads) * head_dim:].view(t, num_kv_heads, head_dim)
    return q, k, v


@register_hip_op
def softmax(x: torch.Tensor, dim: int = -1):
    return torch.softmax(x, dim=dim)
