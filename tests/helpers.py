"""Comparison helpers shared by the parity tests."""
import torch


def bf16_bits(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF


def assert_bit_exact(a: torch.Tensor, b: torch.Tensor, what: str = ""):
    a, b = a.cpu(), b.cpu()
    assert a.shape == b.shape and a.dtype == b.dtype, f"{what}: shape/dtype {a.shape}/{a.dtype} vs {b.shape}/{b.dtype}"
    if a.dtype == torch.bfloat16:
        same = torch.equal(a.contiguous().view(torch.int16), b.contiguous().view(torch.int16))
    else:
        same = torch.equal(a, b)
    assert same, f"{what}: tensors differ bitwise"


def ulp_distance_bf16(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in representable bf16 steps between two finite bf16 tensors."""
    def key(t):
        bits = t.cpu().contiguous().view(torch.int16).to(torch.int32)
        mag = bits & 0x7FFF
        return torch.where(bits < 0, -mag, mag)
    return (key(a) - key(b)).abs()


def assert_within_one_ulp(a: torch.Tensor, b: torch.Tensor, what: str = ""):
    assert a.shape == b.shape and a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16
    assert torch.isfinite(a.float()).all() and torch.isfinite(b.float()).all(), f"{what}: non-finite values"
    d = ulp_distance_bf16(a, b)
    worst = int(d.max()) if d.numel() else 0
    assert worst <= 1, f"{what}: max distance {worst} bf16 ulp (allowed 1); {int((d > 1).sum())} elements off"


# attention tolerance stated by the benchmark definition: bf16 in/out, fp32 accumulate
ATTN_MAX_ABS = 2e-2
ATTN_MEAN_ABS = 2e-3


def assert_attention_close(got: torch.Tensor, want: torch.Tensor, what: str = ""):
    assert got.shape == want.shape and got.dtype == want.dtype, f"{what}: {got.shape}/{got.dtype} vs {want.shape}/{want.dtype}"
    g, w = got.float().cpu(), want.float().cpu()
    assert torch.isfinite(g).all(), f"{what}: non-finite output"
    if g.numel() == 0:
        return
    diff = (g - w).abs()
    assert diff.max().item() <= ATTN_MAX_ABS, f"{what}: max-abs {diff.max().item():.4g} > {ATTN_MAX_ABS}"
    assert diff.mean().item() <= ATTN_MEAN_ABS, f"{what}: mean-abs {diff.mean().item():.4g} > {ATTN_MEAN_ABS}"


def _step_bf16(t: torch.Tensor, direction: int) -> torch.Tensor:
    """Neighbouring representable bf16 in value order: direction +1 = next larger, -1 = next smaller."""
    bits = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    neg = bits >= 0x8000
    mag = bits & 0x7FFF
    # value order: positive numbers grow with mag, negative shrink
    delta = torch.where(neg, torch.full_like(mag, -direction), torch.full_like(mag, direction))
    new_mag = mag + delta
    flip = new_mag < 0                       # crossed zero
    new_mag = torch.where(flip, torch.ones_like(new_mag), new_mag)
    new_neg = torch.where(flip, ~neg, neg)
    out = (new_mag | (new_neg.to(torch.int32) << 15)).to(torch.int32)
    out = torch.where(out >= 0x8000, out - 0x10000, out).to(torch.int16)
    return out.view(torch.bfloat16)


def assert_rms_parity(got: torch.Tensor, normed_ref: torch.Tensor, weight: torch.Tensor, want: torch.Tensor, what: str = ""):
    """RMSNorm has two bf16 roundings: bf16(x * rstd), then bf16(that * w).  The row statistic is an fp32
    sum whose last bit depends on summation order, which can move the FIRST rounding by one bf16 step.
    Accepted: the output equals, bit for bit, what the reference's second stage produces from a
    normalised value at most 1 bf16 ulp from the reference's (normed_ref); at least 99.9 % of the
    elements equal the reference output exactly; and, measured on the final output, no element is more than
    2 bf16 ulp from the reference and at most one in 100 000 is more than 1 ulp away (a one-step move of the
    first rounding, multiplied by a weight, can land two steps away after the second rounding).  The
    measured distances are printed (pytest -s) and returned."""
    got = got.cpu()
    assert got.shape == want.shape and got.dtype == torch.bfloat16
    assert torch.isfinite(got.float()).all(), f"{what}: non-finite"
    cands = [normed_ref * weight, _step_bf16(normed_ref, +1) * weight, _step_bf16(normed_ref, -1) * weight]
    ok = torch.zeros(got.shape, dtype=torch.bool)
    gb = got.contiguous().view(torch.int16)
    for c in cands:
        ok |= gb == c.contiguous().view(torch.int16)
    # -0.0 vs +0.0 are the same value
    ok |= (got.float() == 0) & (want.float() == 0)
    bad = int((~ok).sum())
    assert bad == 0, f"{what}: {bad} elements are not reachable from a normalised value within 1 bf16 ulp"
    exact = (gb == want.contiguous().view(torch.int16)).float().mean().item()
    assert exact >= 0.999, f"{what}: only {exact:.5f} of the elements equal the reference bit for bit"
    dist = ulp_distance_bf16(got, want)
    worst = int(dist.max()) if dist.numel() else 0
    beyond_one = int((dist > 1).sum())
    allowed = -(-dist.numel() // 100000)    # ceil(numel / 1e5)
    print(f"[rms parity] {what}: {dist.numel()} elements, {exact * 100:.4f} % bit-equal, max {worst} bf16 ulp, "
          f"{beyond_one} beyond 1 ulp (allowed {allowed})")
    assert worst <= 2, f"{what}: an output is {worst} bf16 ulp from the reference (allowed 2)"
    assert beyond_one <= allowed, f"{what}: {beyond_one} outputs are more than 1 bf16 ulp from the reference (allowed {allowed})"
    return {"elements": dist.numel(), "bit_equal": exact, "max_ulp": worst, "beyond_one_ulp": beyond_one}
