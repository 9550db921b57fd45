"""The C-ABI library loads without a GPU, exports every function include/mops_hip.h declares, and
rejects bad arguments on the host before any launch (no compute call is made here)."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "mops_hip.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mops_hip_\w+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from nano_vllm_ninetoothed_amd import _capi
    if not _capi.LIB_PATH.exists():
        from nano_vllm_ninetoothed_amd import build
        build.build(force=False)
    return _capi.load()


def test_header_and_binding_agree(lib):
    from nano_vllm_ninetoothed_amd import _capi
    names = declared_functions()
    assert len(names) >= 9
    assert set(names) == set(_capi.SIGNATURES), "include/mops_hip.h and _capi.SIGNATURES list different functions"
    raw = ctypes.CDLL(str(_capi.LIB_PATH))
    for n in names:
        assert hasattr(raw, n), f"{n} declared in the header but not exported by libmops_hip.so"
    assert lib.mops_hip_abi_version() == _capi.ABI_VERSION


def test_status_strings(lib):
    assert lib.mops_hip_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5):
        assert lib.mops_hip_status_string(code) not in (b"ok", b"unknown status")
    assert lib.mops_hip_status_string(-99) == b"unknown status"


def test_host_side_argument_validation(lib):
    A = 0x1000  # a 16-byte aligned non-null fake address; never dereferenced because validation fails first
    # store_kvcache
    assert lib.mops_hip_store_kvcache(None, 1024, A, 1024, A, A, A, 4, 1024, 1024, None) == -1
    assert lib.mops_hip_store_kvcache(A, 512, A, 1024, A, A, A, 4, 1024, 1024, None) == -1      # stride < row
    assert lib.mops_hip_store_kvcache(A, 1028, A, 1024, A, A, A, 4, 1024, 1024, None) == -3     # stride % 8
    assert lib.mops_hip_store_kvcache(A + 2, 1024, A, 1024, A, A, A, 4, 1024, 1024, None) == -3  # misaligned
    assert lib.mops_hip_store_kvcache(A, 1024, A, 1024, A, A, A, -1, 1024, 1024, None) == -1
    assert lib.mops_hip_store_kvcache(None, 1024, None, 1024, None, None, None, 0, 1024, 1024, None) == 0  # empty
    # embedding
    assert lib.mops_hip_embedding(A, 1, None, 1024, A, 4, 100, 1024, None) == -1
    assert lib.mops_hip_embedding(A, 1, A, 1024, A, 4, 100, 1020, None) == -3                    # hidden % 8
    assert lib.mops_hip_embedding(A, 0, A, 1024, A, 0, 100, 1024, None) == 0
    # rms
    assert lib.mops_hip_rms_forward(A, A, A, 1, 4, 32768, 0, 32768, 1e-6, None) == -2             # n too large
    assert lib.mops_hip_rms_forward(A, A, A, 1, 4, 1001, 0, 1001, 1e-6, None) == -3
    assert lib.mops_hip_rms_forward(A, None, A, 1, 4, 1024, 0, 1024, 1e-6, None) == -1
    assert lib.mops_hip_add_rms_forward(A, 1024, A, 1024, A, A, A, 4, 1024, 1e-6, None) == -1     # y aliases x
    # paged decode
    ws = lib.mops_hip_paged_decode_workspace_bytes(256, 16, 8, 16, 256)
    assert ws > 0 and ws % 256 == 0
    base = dict(q=A, qs=2048, k=A, v=A, sl=A, bt=A, bts=16, out=A, b=256, hq=16, hkv=8, d=128, bs=256, nb=4096, mb=16)

    def decode(**kw):
        a = dict(base, **kw)
        return lib.mops_hip_attn_paged_decode_bf16(a["q"], a["qs"], a["k"], a["v"], a["sl"], a["bt"], a["bts"], a["out"],
                                                   a["b"], a["hq"], a["hkv"], a["d"], a["bs"], a["nb"], a["mb"], 0.088,
                                                   a.get("ws"), a.get("wsb", 0), None)
    assert decode(d=64) == -2
    assert decode(bs=100) == -2
    assert decode(hq=12) == -1                    # not a multiple of kv heads
    assert decode(hq=256, hkv=8, qs=256 * 128) == -2  # group of 32 query heads per kv head
    assert decode(q=None) == -1
    assert decode(bts=8) == -1                    # row stride narrower than the table
    assert decode() == -4                         # workspace required and missing
    assert decode(ws=A, wsb=16) == -4
    assert decode(b=0) == 0
    # varlen prefill
    def prefill(**kw):
        a = dict(q=A, qs=2048, k=A, ks=1024, v=A, vs=4096, o=A, os=2048, cu=A, cuk=None, bt=None, bts=0, bs=0, nb=0, mb=0,
                 b=2, t=512, tk=512, ms=256, hq=16, hkv=8, d=128)
        a.update(kw)
        return lib.mops_hip_attn_varlen_causal_bf16(a["q"], a["qs"], a["k"], a["ks"], a["v"], a["vs"], a["o"], a["os"],
                                                    a["cu"], a["cuk"], a["bt"], a["bts"], a["bs"], a["nb"], a["mb"],
                                                    a["b"], a["t"], a["tk"], a["ms"], a["hq"], a["hkv"], a["d"], 0.088, None)
    assert prefill(d=64) == -2
    assert prefill(cu=None) == -1
    assert prefill(ks=512) == -1
    assert prefill(vs=4100) == -3
    assert prefill(hq=12) == -1
    assert prefill(tk=600) == -1                               # more keys than queries needs cu_seqlens_k
    assert prefill(bt=A, bts=4, bs=256, nb=8, mb=4) == -1      # paged form needs cu_seqlens_k
    assert prefill(bt=A, cuk=A, bts=2, bs=256, nb=8, mb=4) == -1   # table rows narrower than max_blocks
    assert prefill(bt=A, cuk=A, bts=4, bs=96, nb=8, mb=4) == -2    # block size not a multiple of 64
    assert prefill(t=0) == 0


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    from nano_vllm_ninetoothed_amd import _capi
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", tmp_path / "libmops_hip.so")
    with pytest.raises(ImportError):
        _capi.load()


def test_linear_argument_validation(lib):
    """linear: validation happens on the host before the GEMM library is touched."""
    A = 0x1000
    assert lib.mops_hip_linear_bf16(A, 1024, A, 1024, None, A, 4096, 0, 4096, 1024, None, 0, None) == 0       # no rows
    assert lib.mops_hip_linear_bf16(None, 1024, A, 1024, None, A, 4096, 4, 4096, 1024, None, 0, None) == -1
    assert lib.mops_hip_linear_bf16(A, 512, A, 1024, None, A, 4096, 4, 4096, 1024, None, 0, None) == -1    # x stride < k
    assert lib.mops_hip_linear_bf16(A, 1024, A, 1024, None, A, 4096, 4, 4096, 1020, None, 0, None) == -3   # k % 8
    assert lib.mops_hip_linear_bf16(A, 1024, A, 1024, None, A + 2, 4096, 4, 4096, 1024, None, 0, None) == -3
    assert lib.mops_hip_linear_bf16(A, 1024, A, 1024, None, A, 4096, 4, 4096, 1024, None, 64, None) == -1     # bytes without a pointer
    assert lib.mops_hip_linear_pin_solution(0, 4096, 1024, 5) == -1
    assert lib.mops_hip_linear_pin_solution(4, 4096, 1024, 5) == 0 and lib.mops_hip_linear_pin_solution(4, 4096, 1024, -1) == 0
    assert lib.mops_hip_linear_tune(0, 4096, 1024, 28, 1, None, 0, None, None, None) == -1
