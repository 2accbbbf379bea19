"""GPU checks at the full sizes of the benchmark configurations, through properties that do not need
the CPU oracle on the whole matrix: closed-form definitions evaluated with plain torch operations on
the device, invariants of 2:4 patterns, exactness on small-integer operands, and bit-exact oracle
comparisons on slabs of rows."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F16, BF16, F32, E4M3 = torch.float16, torch.bfloat16, torch.float32, torch.float8_e4m3fn


def _top2_mask(w):
    """Closed form of the magnitude rule: keep the two largest |x| of each group of 4, an equal
    magnitude at a later index wins.  Element i is kept iff fewer than two elements beat it."""
    a = w.float().abs().view(-1, 4)
    idx = torch.arange(4, device=w.device)
    beats = (a[:, None, :] > a[:, :, None]) | ((a[:, None, :] == a[:, :, None]) & (idx[None, None, :] > idx[None, :, None]))
    return (beats.sum(-1) < 2).view(w.shape)


def _meta_from_mask(mask, bits):
    """Nibble pos0 | pos1 << 2 per group (positions of the two kept elements, ascending), packed
    least-significant first into words of `bits` bits."""
    m = mask.view(mask.shape[0], -1, 4)
    pos = torch.arange(4, device=mask.device).expand_as(m)
    first = torch.where(m, pos, torch.full_like(pos, 9)).min(-1).values
    last = torch.where(m, pos, torch.full_like(pos, -1)).max(-1).values
    nib = (first | (last << 2)).to(torch.int64)
    per = bits // 4
    nib = nib.view(mask.shape[0], -1, per)
    shifts = (4 * torch.arange(per, device=mask.device)).view(1, 1, per)
    word = (nib << shifts).sum(-1)
    if bits == 16:
        return torch.where(word >= 32768, word - 65536, word).to(torch.int16)
    return torch.where(word >= 2 ** 31, word - 2 ** 32, word).to(torch.int32)


@pytest.fixture(scope="module")
def cfg2(cuda):
    g = torch.Generator(device=cuda).manual_seed(1)
    w = torch.randn(8192, 8192, device=cuda, generator=g).bfloat16()
    u = torch.rand(8192, 8192, device=cuda, generator=g)
    return w, u


def test_config2_magnitude_compress_closed_form(cuda, cfg2):
    import sparse
    w, _ = cfg2
    s = sparse.to_sparse_semi_structured(w, dtype=F16)
    mask = _top2_mask(w)
    assert int(mask.view(-1, 4).sum(-1).min()) == 2 and int(mask.view(-1, 4).sum(-1).max()) == 2
    want_dense = torch.where(mask, w, torch.zeros_like(w)).to(F16)
    assert torch.equal(s.to_dense().view(torch.int16), want_dense.view(torch.int16))
    assert torch.equal(s.indices(), _meta_from_mask(mask, 16))
    # the kept values in order are the compressed matrix
    kept = w.to(F16).view(-1)[mask.view(-1)].view(8192, 4096)
    assert torch.equal(s.values().view(torch.int16), kept.view(torch.int16))


def test_config2_mvue_slab_parity_and_invariants(cuda, cfg2):
    import sparse
    w, u = cfg2
    s = sparse.to_sparse_semi_structured(w, MVUE24=True, rand=u, dtype=F16)
    dense = s.to_dense()
    nz = (dense != 0).view(-1, 4).sum(-1)
    assert int(nz.max()) <= 2
    # kept values are x / p with p <= 1 (up to rounding): same sign, magnitude not below |x|
    kept = dense != 0
    assert bool((torch.sign(dense.float()[kept]) == torch.sign(w.float()[kept])).all())
    assert bool((dense.float().abs()[kept] >= w.float().abs()[kept] * (1 - 2 ** -9)).all())
    # bit-exact against the oracle on slabs of rows spread over the matrix
    rows = torch.cat([torch.arange(r, r + 32) for r in (0, 2048 + 32, 8192 - 32)])
    want_v, want_m, _ = oracle.mvue24(w[rows].cpu(), u[rows].cpu(), out_dtype=F16)
    assert torch.equal(s.values()[rows].cpu().view(torch.int16), want_v.view(torch.int16))
    assert torch.equal(s.indices()[rows].cpu(), want_m)


def test_config2_transposable_is_valid_and_optimal(cuda, cfg2):
    import sparse
    w, _ = cfg2
    sp, mask = sparse.TransposableSparse(abs=True)(w)
    blocks = mask.view(2048, 4, 2048, 4).permute(0, 2, 1, 3)                  # [bi, bj, r, c]
    assert bool((blocks.sum(-1) == 2).all()) and bool((blocks.sum(-2) == 2).all())
    assert torch.equal(sp.view(torch.int16), torch.where(mask, w, torch.zeros_like(w)).view(torch.int16))
    # score of the chosen pattern = best of the 90 patterns (float64 sums of the exact bf16 magnitudes)
    pats = oracle.transposable_patterns().to(cuda).double()                    # [90, 16]
    a = w.double().abs().view(2048, 4, 2048, 4).permute(0, 2, 1, 3).reshape(-1, 16)
    chosen = (a * blocks.reshape(-1, 16)).sum(-1)
    best = torch.empty_like(chosen)
    for lo in range(0, a.shape[0], 1 << 19):
        best[lo:lo + (1 << 19)] = (a[lo:lo + (1 << 19)] @ pats.t()).max(-1).values
    # the search adds in float32; a pattern it prefers can trail the float64 best by rounding only
    assert bool((chosen >= best * (1 - 1e-6)).all())
    assert float((chosen == best).double().mean()) > 0.999


def test_config2_soft_threshold_closed_form(cuda, cfg2):
    import sparse
    w, _ = cfg2
    sp, mk = sparse.soft_threshold24_triton(w)
    mask = _top2_mask(w)
    a = w.float().abs().view(-1, 4)
    thr = a.sort(-1).values[:, 1:2].expand(-1, 4).reshape(w.shape)            # second smallest magnitude
    x = w.float()
    shrunk = torch.where(x > 0, x - thr, x + thr)
    want = torch.where(mask, shrunk, torch.zeros_like(shrunk)).bfloat16()
    assert torch.equal(sp.view(torch.int16), want.view(torch.int16))
    assert torch.equal(mk.view(torch.int16), mask.to(BF16).view(torch.int16))


def test_config2_masked_add_closed_form(cuda, cfg2):
    import sparse
    w, _ = cfg2
    g = torch.Generator(device=cuda).manual_seed(7)
    grad = 1e-3 * torch.randn(8192, 8192, device=cuda, generator=g)
    p = w.float()
    mask = _top2_mask(w)
    prod = p * torch.tensor(2e-4, dtype=F32, device=cuda)                      # rounded product, then rounded sum
    want = torch.where(mask, grad, grad + prod)
    got = grad.clone()
    sparse.masked_add_(got, p, mask, alpha=2e-4)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


@pytest.fixture(scope="module")
def cfg3_ints(cuda):
    g = torch.Generator(device=cuda).manual_seed(3)
    x = torch.randint(-3, 4, (8192, 4096), device=cuda, generator=g).to(F16)
    w = torch.randint(-3, 4, (11008, 4096), device=cuda, generator=g).to(F16)
    dy = torch.randint(-3, 4, (8192, 11008), device=cuda, generator=g).to(F16)
    return x, w, dy


def test_config3_spmm_exact_on_small_integers(cuda, cfg3_ints):
    """Products and sums of small integers are exact in float32, so both products of the config must
    equal the dense float32 product of the masked weights rounded once to fp16."""
    import sparse
    x, w, dy = cfg3_ints
    ws = sparse.to_sparse_semi_structured(w)
    wd = ws.to_dense()
    y = torch.mm(x, ws.t())
    want = torch.mm(x.float(), wd.float().t()).to(F16)
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))
    _, tmask = sparse.TransposableSparse()(w)
    wt = sparse.to_sparse_semi_structured(w.t(), mask=tmask.t())
    dx = torch.mm(dy, wt.t())
    want = torch.mm(dy.float(), torch.where(tmask, w, torch.zeros_like(w)).float()).to(F16)
    assert torch.equal(dx.view(torch.int16), want.view(torch.int16))


def test_config3_spmm_random_and_linear(cuda):
    import sparse
    g = torch.Generator(device=cuda).manual_seed(3)
    x = torch.randn(8192, 4096, device=cuda, generator=g).half()
    w = (0.02 * torch.randn(11008, 4096, device=cuda, generator=g)).half()
    ws = sparse.to_sparse_semi_structured(w)
    y = torch.mm(x, ws.t())
    ref = torch.mm(x.float(), ws.to_dense().float().t())
    assert ((y.float() - ref).norm() / ref.norm()).item() < 1e-2
    # linearity in the dense operand: rows scaled by powers of two scale the output rows exactly
    scale = torch.where(torch.arange(8192, device=cuda) % 2 == 0, 2.0, 1.0).half().unsqueeze(1)
    y2 = torch.mm(x * scale, ws.t())
    normal = y.abs() >= 2.0 ** -13          # doubling commutes with the fp16 rounding outside the subnormal range
    assert torch.equal(y2[normal].view(torch.int16), (y * scale)[normal].view(torch.int16))
    assert float(normal.float().mean()) > 0.99


def test_config3_spmm_bf16(cuda):
    """bfloat16 at the size of config 3, both products: exact on small integers (sums stay below 2^24, one
    rounding to bf16) and within 1e-2 of the float32 product on the config's random data."""
    import sparse
    g = torch.Generator(device=cuda).manual_seed(3)
    x = torch.randint(-3, 4, (8192, 4096), device=cuda, generator=g).to(BF16)
    w = torch.randint(-3, 4, (11008, 4096), device=cuda, generator=g).to(BF16)
    dy = torch.randint(-3, 4, (8192, 11008), device=cuda, generator=g).to(BF16)
    ws = sparse.to_sparse_semi_structured(w, dtype=BF16)
    y = torch.mm(x, ws.t())
    want = torch.mm(x.float(), ws.to_dense().float().t()).to(BF16)
    assert y.dtype == BF16 and torch.equal(y.view(torch.int16), want.view(torch.int16))
    _, tmask = sparse.TransposableSparse()(w)
    wt = sparse.to_sparse_semi_structured(w.t(), mask=tmask.t(), dtype=BF16)
    dx = torch.mm(dy, wt.t())
    want = torch.mm(dy.float(), torch.where(tmask, w, torch.zeros_like(w)).float()).to(BF16)
    assert torch.equal(dx.view(torch.int16), want.view(torch.int16))
    del x, w, dy, want, y, dx
    x = torch.randn(8192, 4096, device=cuda, generator=g).to(BF16)
    w = (0.02 * torch.randn(11008, 4096, device=cuda, generator=g)).to(BF16)
    ws = sparse.to_sparse_semi_structured(w, dtype=BF16)
    y = torch.mm(x, ws.t())
    ref = torch.mm(x.float(), ws.to_dense().float().t())
    assert ((y.float() - ref).norm() / ref.norm()).item() < 1e-2


def test_config5_fp8_spmm_rows_against_float32(cuda):
    import sparse
    g = torch.Generator(device=cuda).manual_seed(5)
    a = torch.randn(16384, 8192, device=cuda, generator=g)
    b = torch.randn(8192, 8192, device=cuda, generator=g)
    u = torch.rand(8192, 8192, device=cuda, generator=g)
    sa, sb = 448.0 / a.abs().max().item(), 224.0 / b.abs().max().item()
    aq = (a * sa).to(E4M3)
    bs = (b * sb).bfloat16()
    del a, b
    s = sparse.to_sparse_semi_structured(bs, MVUE24=True, rand=u, dtype=E4M3)
    rows = torch.cat([torch.arange(r, r + 32) for r in (0, 4096, 8192 - 32)])
    want_v, want_m, _ = oracle.mvue24(bs[rows].cpu(), u[rows].cpu(), out_dtype=E4M3)
    assert torch.equal(s.values()[rows].cpu().view(torch.uint8), want_v.view(torch.uint8))
    assert torch.equal(s.indices()[rows].cpu(), want_m)
    out = sparse.sparse_semi_structured_linear(aq, s, out_dtype=BF16, scale=1.0 / (sa * sb))
    assert out.shape == (16384, 8192) and out.dtype == BF16
    sl = slice(16384 - 512, 16384)
    ref = torch.mm(aq[sl].float(), s.to_dense().float().t()) / (sa * sb)
    assert ((out[sl].float() - ref).norm() / ref.norm()).item() < 5e-2
    # the reference's own output type for 8-bit operands is float32 (.cu:729, 772): the same accumulators through the
    # 32-bit output pass, so rounding them to bf16 must give the bf16 product bit for bit, over all 2048 tiles
    out32 = sparse.sparse_semi_structured_linear(aq, s, scale=1.0 / (sa * sb))
    assert out32.dtype == torch.float32 and out32.shape == (16384, 8192)
    assert torch.equal(out32.to(BF16), out)
    assert ((out32[sl] - ref).norm() / ref.norm()).item() < 5e-2
