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
