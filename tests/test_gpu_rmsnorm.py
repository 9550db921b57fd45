"""GPU parity for rms_forward / add_rms_forward against the oracle on the same inputs.

Tolerance: 1 bf16 ulp at the normalisation rounding (helpers.assert_rms_parity): the output must be
bit-identical to the reference's second stage applied to a normalised value within 1 bf16 ulp of the
reference's, and >= 99.9 % of all elements must equal the reference output exactly."""
import pytest
import torch

from helpers import assert_bit_exact, assert_rms_parity
from nano_vllm_ninetoothed_amd import workloads as W

pytestmark = pytest.mark.gpu


def _normed(x, eps, residual=None):
    """The reference's value after its first rounding (mops/torch/ops.py:11-15 / 21-29)."""
    s = x.float() if residual is None else x.float() + residual.float()
    return (s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps)).to(torch.bfloat16)


@pytest.mark.parametrize("rows,hidden", [(512, 1024), (512, 4096), (1, 1024), (7, 128), (333, 128), (65, 2048),
                                         (9, 5120), (5, 8192), (3, 16384), (130, 64), (11, 1000)])
def test_rms_forward_2d(gpu, ops, rows, hidden):
    hip, ref = ops("rms_forward")
    d = W.rms_inputs(rows, hidden, seed=rows * 7 + hidden)
    want = ref(d["x"], d["weight"], d["eps"])
    x_g = d["x"].to(gpu)
    keep = x_g.clone()
    got = hip(x_g, d["weight"].to(gpu), d["eps"])
    assert got.data_ptr() != x_g.data_ptr()
    assert_bit_exact(x_g, keep, "input left intact")
    assert_rms_parity(got, _normed(d["x"], d["eps"]), d["weight"], want, f"rms_forward {rows}x{hidden}")


def test_rms_forward_strided_qk_views(gpu, ops):
    """q_norm / k_norm see [T, H, 128] views into the qkv projection output (row stride 4096)."""
    hip, ref = ops("rms_forward")
    g = torch.Generator("cpu").manual_seed(3)
    T = 200
    qkv = torch.randn((T, 4096), generator=g).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(128, generator=g)).to(torch.bfloat16)
    q, k, _ = qkv.split([2048, 1024, 1024], dim=-1)
    qkv_g = qkv.to(gpu)
    q_g, k_g, _ = qkv_g.split([2048, 1024, 1024], dim=-1)
    for name, cpu_view, gpu_view, heads in (("q", q, q_g, 16), ("k", k, k_g, 8)):
        cv, gv = cpu_view.view(T, heads, 128), gpu_view.view(T, heads, 128)
        assert not gv.is_contiguous()
        got = hip(gv, w.to(gpu), 1e-6)
        assert got.shape == (T, heads, 128) and got.is_contiguous()
        assert_rms_parity(got, _normed(cv, 1e-6), w, ref(cv, w, 1e-6), f"{name}_norm")
    assert_bit_exact(qkv_g, qkv, "qkv buffer untouched")


def test_rms_forward_3d_contiguous_and_empty(gpu, ops):
    hip, ref = ops("rms_forward")
    d = W.rms_inputs(24, 1024, seed=1)
    x3 = d["x"].view(2, 12, 1024)
    got = hip(x3.to(gpu), d["weight"].to(gpu), 1e-6)
    assert got.shape == (2, 12, 1024)
    assert_rms_parity(got, _normed(x3, 1e-6), d["weight"], ref(x3, d["weight"], 1e-6), "3-D")
    e = hip(torch.empty((0, 1024), dtype=torch.bfloat16, device=gpu), d["weight"].to(gpu), 1e-6)
    assert e.shape == (0, 1024)


@pytest.mark.parametrize("rows,hidden", [(512, 4096), (512, 1024), (1, 1024), (77, 2048), (6, 5120), (19, 128)])
def test_add_rms_forward(gpu, ops, rows, hidden):
    hip, ref = ops("add_rms_forward")
    d = W.rms_inputs(rows, hidden, seed=rows + hidden, with_residual=True)
    want_y, want_r = ref(d["x"], d["residual"], d["weight"], d["eps"])
    x_g, r_g = d["x"].to(gpu), d["residual"].to(gpu)
    got_y, got_r = hip(x_g, r_g, d["weight"].to(gpu), d["eps"])
    assert_bit_exact(got_r, want_r, "residual output (a single fp32 add, rounded once)")
    assert_rms_parity(got_y, _normed(d["x"], d["eps"], d["residual"]), d["weight"], want_y, f"add_rms_forward {rows}x{hidden}")
    assert_bit_exact(x_g, d["x"], "x untouched")
    assert_bit_exact(r_g, d["residual"], "residual input untouched")


def test_add_rms_with_zero_residual_equals_rms(gpu, ops):
    add_hip, _ = ops("add_rms_forward")
    rms_hip, _ = ops("rms_forward")
    d = W.rms_inputs(64, 1024, seed=11)
    x_g, w_g = d["x"].to(gpu), d["weight"].to(gpu)
    y1, r1 = add_hip(x_g, torch.zeros_like(x_g), w_g, 1e-6)
    assert_bit_exact(y1, rms_hip(x_g, w_g, 1e-6), "add(x, 0) == rms(x)")
    assert_bit_exact(r1, x_g, "residual == x")
