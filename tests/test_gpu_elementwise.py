"""GPU parity for the two per-layer elementwise ops with HIP kernels: apply_rotary_emb (bit-exact: fp32
products rounded separately, as the library expression does) and siluAndMul (two bf16 roundings: the
output must be what the reference's multiply produces from a silu value within 1 bf16 ulp of the
reference's, and >= 99.9 % of elements bit-equal — expf differs in the last fp32 bit between libraries)."""
import pytest
import torch

from helpers import assert_bit_exact, assert_rms_parity

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens,heads", [(256, 16), (1, 8), (37, 16), (512, 32)])
def test_rotary_matches_oracle(gpu, ops, tokens, heads):
    hip, ref = ops("apply_rotary_emb")
    g = torch.Generator().manual_seed(tokens + heads)
    x = torch.randn((tokens, heads, 128), generator=g).to(torch.bfloat16)
    pos = torch.randint(0, 4096, (tokens,), generator=g)
    inv = 1.0 / (1e6 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    fr = torch.outer(torch.arange(4096, dtype=torch.float32), inv)
    cache = torch.cat((fr.cos(), fr.sin()), -1).unsqueeze(1)
    cos, sin = cache[pos].chunk(2, dim=-1)                    # views with row stride 128, like the engine's
    want = ref(x, cos, sin)
    cg, sg = cache.to(gpu)[pos.to(gpu)].chunk(2, dim=-1)
    got = hip(x.to(gpu), cg, sg)
    assert_bit_exact(got, want, "rotary")


def test_rotary_on_strided_heads(gpu, ops):
    hip, ref = ops("apply_rotary_emb")
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn((64, 4096), generator=g).to(torch.bfloat16)
    cos = torch.rand((64, 1, 64), generator=g)
    sin = torch.rand((64, 1, 64), generator=g)
    k = qkv[:, 2048:3072].view(64, 8, 128)
    got = hip(qkv.to(gpu)[:, 2048:3072].view(64, 8, 128), cos.to(gpu), sin.to(gpu))
    assert_bit_exact(got, ref(k, cos, sin), "rotary on a strided view")


@pytest.mark.parametrize("rows,n", [(256, 3072), (1, 3072), (33, 1024), (512, 12288)])
def test_silu_and_mul_matches_oracle(gpu, ops, rows, n):
    hip, ref = ops("siluAndMul")
    g = torch.Generator().manual_seed(rows + n)
    gate_up = (torch.randn((rows, 2 * n), generator=g) * 2).to(torch.bfloat16)
    x, y = gate_up.chunk(2, -1)
    want = ref(x, y)
    xg, yg = gate_up.to(gpu).chunk(2, -1)
    got = hip(xg, yg)
    assert got.shape == (rows, n) and got.is_contiguous()
    assert_rms_parity(got, torch.nn.functional.silu(x), y, want, "siluAndMul")


def test_silu_and_mul_every_bf16_pattern(gpu, ops):
    """silu depends on one bf16 input, so all 65 536 patterns can be walked: the kernel's quick route (hardware exp2 and
    reciprocal, the exact route only near a rounding midpoint) gives the oracle's bits for every one of them, NaNs as NaNs,
    zeros of either sign as zeros; the product with y is a single rounding on both sides."""
    hip, ref = ops("siluAndMul")
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(64, 1024)
    for yv in (1.0, 1.3359375, -0.75):
        gate_up = torch.cat([x, torch.full((64, 1024), yv, dtype=torch.bfloat16)], dim=1).contiguous()
        a, b = gate_up.chunk(2, -1)
        want = ref(a, b)
        ag, bg = gate_up.to(gpu).chunk(2, -1)
        got = hip(ag, bg).cpu()
        nan_w, nan_g = torch.isnan(want.float()), torch.isnan(got.float())
        assert torch.equal(nan_w, nan_g)
        same = (got.view(torch.int16) == want.view(torch.int16)) | nan_w | ((got.float() == 0) & (want.float() == 0))
        bad = (~same).flatten().nonzero().flatten().tolist()
        assert not bad, (yv, [hex(i) for i in bad[:8]])


@pytest.mark.parametrize("rows,vocab", [(256, 151936), (1, 151936), (7, 1000), (33, 2048), (5, 12345)])
def test_sampler_matches_oracle(gpu, ops, rows, vocab):
    """Greedy sampler: same token ids as argmax(softmax(logits / T)); ties resolve to the first index."""
    hip, ref = ops("sampler_forward")
    g = torch.Generator().manual_seed(rows + vocab)
    pad = (vocab + 7) // 8 * 8
    buf = (torch.randn((rows, pad), generator=g) * 3).to(torch.bfloat16)
    logits = buf[:, :vocab]
    logits[0, 5] = 50.0
    logits[0, 3] = 50.0                      # a tie for the maximum: index 3 must win
    if rows > 1:
        logits[1, vocab - 1] = 60.0          # maximum in the last column
    temps = torch.rand(rows, generator=g) + 0.1
    want = ref(logits, temps)
    got = hip(buf.to(gpu)[:, :vocab], temps.to(gpu))
    assert got.dtype == torch.int64 and got.shape == (rows,)
    assert torch.equal(got.cpu(), want)
    assert int(got[0]) == 3


def test_sampler_on_rows_the_softmax_turns_into_nans(gpu, ops):
    """A NaN or +inf logit, or a row of -inf, makes softmax(logits / T) all NaN, and the library's argmax of an
    all-NaN row is 0; the kernel answers the same.  Rows around them are unaffected."""
    hip, ref = ops("sampler_forward")
    g = torch.Generator().manual_seed(77)
    logits = (torch.randn((6, 4096), generator=g) * 3).to(torch.bfloat16)
    logits[0, 100] = float("nan")
    logits[1, 4095] = float("inf")
    logits[2, :] = float("-inf")
    logits[3, 7] = float("nan"); logits[3, 9] = 80.0
    logits[4, 1234] = 70.0                           # an ordinary row
    logits[5, 17] = float("-inf")                    # -inf entries alone are harmless
    temps = torch.full((6,), 0.6)
    want = ref(logits, temps)
    got = hip(logits.to(gpu), temps.to(gpu)).cpu()
    assert torch.equal(got, want), (got.tolist(), want.tolist())
    assert got[:4].tolist() == [0, 0, 0, 0] and int(got[4]) == 1234


def test_sampler_rows_of_negative_logits_zeros_of_both_signs_and_short_rows(gpu, ops):
    """The kernel orders raw bf16 patterns: rows without a non-negative logit take the other branch of that order, -0 and
    +0 are one number with two patterns (the first of either wins), negative NaNs and -inf sit at the far end of the
    unsigned order, and a row may be shorter than one 16-byte piece or end in a partial one that holds the maximum."""
    hip, ref = ops("sampler_forward")
    g = torch.Generator().manual_seed(5)
    n = 8 * 1024 * 5 + 3                                   # five pieces per lane and a tail of three
    base = -(torch.rand((12, n), generator=g) * 20 + 0.5).to(torch.bfloat16)   # every logit negative
    logits = base.clone()
    logits[0, 4097] = -0.25                                # a row of negatives: the maximum is the smallest magnitude
    logits[1, 77] = -0.0                                   # -0 is the maximum of a negative row
    logits[2, 900] = 0.0; logits[2, 30] = -0.0            # -0 first, +0 later: one number, index 30
    logits[3, 30] = 0.0; logits[3, 900] = -0.0
    logits[4, n - 1] = 3.0                                 # the maximum in the partial last piece
    logits[5, n - 2] = -0.125                              # the same in a negative row
    logits[6, 10] = float("-inf"); logits[6, 4000] = -0.375
    logits[7, 123] = torch.tensor(-float("nan"))           # a NaN with the sign bit set
    logits[8, 5] = 7.0; logits[8, 2053] = 7.0; logits[8, 8192 * 3 + 5] = 7.0   # a tie across lanes and batches: the first wins
    logits[9, 3000] = 1e-38                                # a tiny positive among negatives
    logits[10, :] = -3.0                                   # all equal: index 0
    logits[11, 1024 * 8 * 2 + 5] = 0.5; logits[11, 5] = 0.25   # same lane, later batch holds the maximum
    temps = torch.full((12,), 0.7)
    want = ref(logits, temps)
    got = hip(logits.to(gpu), temps.to(gpu)).cpu()
    assert torch.equal(got, want), (got.tolist(), want.tolist())
    assert got.tolist()[:7] == [4097, 77, 30, 30, n - 1, n - 2, 4000] and int(got[7]) == 0 and int(got[8]) == 5
    for width in (1, 3, 7, 8, 9):
        small = (torch.randn((4, 16), generator=g) * 2).to(torch.bfloat16)
        t4 = torch.full((4,), 0.7)
        view = small[:, :width]
        assert torch.equal(hip(small.to(gpu)[:, :width], t4.to(gpu)).cpu(), ref(view, t4)), width


@pytest.mark.parametrize("tokens,hq,hkv,need_k", [(1, 16, 8, True), (5, 16, 8, False), (300, 16, 8, True), (64, 32, 8, False), (33, 8, 1, True)])
def test_fused_qk_norm_rope_store_equals_the_separate_ops(gpu, tokens, hq, hkv, need_k):
    """qk_norm_rope_store against the sequence it replaces, both through the hip backend: bit-identical q, k
    and caches, skipped slots untouched; and against the oracle's composition within the norm criterion."""
    import oracle.mops_torch  # noqa: F401
    from nano_vllm_ninetoothed_amd import mops
    d, block = 128, 256
    g = torch.Generator().manual_seed(tokens * 7 + hq)
    qkv = torch.randn((tokens, (hq + 2 * hkv) * d), generator=g).to(torch.bfloat16)
    wq = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    wk = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    pos = torch.randint(0, 4096, (tokens,), generator=g)
    inv = 1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    fr = torch.outer(pos.float(), inv)
    cos, sin = fr.cos().unsqueeze(1), fr.sin().unsqueeze(1)
    nblocks = (tokens + block - 1) // block + 1
    slots = torch.randperm(nblocks * block, generator=g)[:tokens].to(torch.int32)
    if tokens > 2:
        slots[1] = -1
    sentinel = torch.full((nblocks, block, hkv, d), -7.0, dtype=torch.bfloat16)

    def run(backend, device):
        kc, vc = sentinel.clone().to(device), sentinel.clone().to(device)
        args = [t.to(device) for t in (qkv, wq, wk)]
        c, s_, sl = cos.to(device), sin.to(device), slots.to(device)
        fused = mops.get_op("qk_norm_rope_store", backend)(args[0], args[1], args[2], 1e-6, c, s_, kc, vc, sl, hq, hkv, need_k=need_k)
        return fused, kc, vc, (args, c, s_, sl)

    (q_f, k_f, v_f), kc_f, vc_f, (a, c, s_, sl) = run("hip", gpu)
    # the separate hip ops
    q_in, k_in, v_in = a[0].split([hq * d, hkv * d, hkv * d], dim=-1)
    q_s = mops.get_op("apply_rotary_emb", "hip")(mops.get_op("rms_forward", "hip")(q_in.view(-1, hq, d), a[1], 1e-6), c, s_)
    k_s = mops.get_op("apply_rotary_emb", "hip")(mops.get_op("rms_forward", "hip")(k_in.view(-1, hkv, d), a[2], 1e-6), c, s_)
    kc_s, vc_s = sentinel.clone().to(gpu), sentinel.clone().to(gpu)
    mops.get_op("store_kvcache", "hip")(k_s, v_in.view(-1, hkv, d), kc_s, vc_s, sl)
    assert_bit_exact(q_f, q_s, "fused q vs rms_forward + apply_rotary_emb")
    if need_k:
        assert_bit_exact(k_f, k_s, "fused k vs rms_forward + apply_rotary_emb")
    else:
        assert k_f is None
    assert_bit_exact(kc_f, kc_s, "k cache after the fused op vs after store_kvcache")
    assert_bit_exact(vc_f, vc_s, "v cache after the fused op vs after store_kvcache")
    assert_bit_exact(v_f, v_in.view(-1, hkv, d), "v is the view of qkv")
    # oracle composition (CPU): same values up to the norm's double rounding
    (q_o, k_o, _), kc_o, vc_o, _ = run("torch", "cpu")
    assert (q_f.float().cpu() - q_o.float()).abs().max() <= 0.0625
    assert_bit_exact(vc_f, vc_o, "v cache vs oracle")
    assert ((kc_f.float().cpu() - kc_o.float()).abs() <= 0.0625).all()


@pytest.mark.parametrize("m,n,k,bias", [(256, 4096, 1024, False), (1, 1024, 2048, False), (37, 6144, 1024, True),
                                        (512, 1024, 3072, False), (16, 2048, 1024, True)])
def test_linear_matches_fp32_reference(gpu, m, n, k, bias):
    """linear through the C ABI (a library GEMM with fp32 accumulation) against x.float() @ w.float().T in
    fp32: the only error allowed is the bf16 rounding of the result and the order of the fp32 sums."""
    from nano_vllm_ninetoothed_amd import mops
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(gpu)
    w = (torch.randn(n, k, generator=g) * k ** -0.5).to(torch.bfloat16).to(gpu)
    b = torch.randn(n, generator=g).to(torch.bfloat16).to(gpu) if bias else None
    y = mops.linear(x, w, b)
    assert y.shape == (m, n) and y.dtype == torch.bfloat16
    ref = x.float() @ w.float().t()
    if bias:
        ref = ref + b.float()
    err = (y.float() - ref).abs()
    assert err.max().item() <= 2 ** -7 * ref.abs().max().item() + 1e-3
    # a strided input (a column slice of a wider buffer) and leading dimensions
    wide = torch.randn(2, max(m // 2, 1), k + 64, generator=g).to(torch.bfloat16).to(gpu)
    xs = wide[..., 32:32 + k]
    ys = mops.linear(xs, w, b)
    refs = xs.float() @ w.float().t() + (b.float() if bias else 0)
    assert ys.shape == (2, max(m // 2, 1), n)
    assert (ys.float() - refs).abs().max().item() <= 2 ** -7 * refs.abs().max().item() + 1e-3


def test_linear_with_a_pinned_solution_and_tuning(gpu):
    """mops_hip_linear_tune returns a solution index for a small shape; pinning it keeps the result within
    the same bound, and removing the pin goes back to the heuristic's choice."""
    import ctypes
    from nano_vllm_ninetoothed_amd import _capi, mops
    lib = _capi.load()
    m, n, k = 16, 256, 512
    g = torch.Generator().manual_seed(3)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(gpu)
    w = (torch.randn(n, k, generator=g) * k ** -0.5).to(torch.bfloat16).to(gpu)
    ref = x.float() @ w.float().t()
    y0 = mops.linear(x, w)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=gpu)
    best, best_us, heur_us = ctypes.c_int(-1), ctypes.c_float(-1), ctypes.c_float(-1)
    st = lib.mops_hip_linear_tune(m, n, k, 2, 1, ws.data_ptr(), ws.numel(), ctypes.byref(best), ctypes.byref(best_us), ctypes.byref(heur_us))
    assert st == 0 and best.value >= 0 and best_us.value > 0 and heur_us.value > 0
    assert lib.mops_hip_linear_pin_solution(m, n, k, best.value) == 0
    y1 = mops.linear(x, w)
    assert lib.mops_hip_linear_pin_solution(m, n, k, -1) == 0
    y2 = mops.linear(x, w)
    for y in (y0, y1, y2):
        assert (y.float() - ref).abs().max().item() <= 2 ** -7 * ref.abs().max().item() + 1e-3
    assert torch.equal(y0, y2)
    # a row count without a pin of its own borrows the pin of the next larger one of the same weight shape (a decode step
    # outside a graph runs any number of rows): 13 rows before, with and after a pin for 16 rows
    x13, ref13 = x[:13], ref[:13]
    z0 = mops.linear(x13, w)
    assert lib.mops_hip_linear_pin_solution(m, n, k, best.value) == 0
    z1 = mops.linear(x13, w)
    assert lib.mops_hip_linear_pin_solution(m, n, k, -1) == 0
    z2 = mops.linear(x13, w)
    for z in (z0, z1, z2):
        assert z.shape == (13, n) and (z.float() - ref13).abs().max().item() <= 2 ** -7 * ref.abs().max().item() + 1e-3
    assert torch.equal(z0, z2)
