"""Pins the oracle's MVUE24, soft-threshold, transposable-search and masked-decay functions
against closed forms, invariants, brute force and the reference's own vectors (CPU only)."""
import hashlib
import math
import os
import re

import pytest
import torch

import oracle


# ---------------------------------------------------------------- MVUE24
def test_mvue_probabilities_closed_form():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 64, generator=g)
    p = oracle.mvue24_probabilities(x).double().reshape(-1, 4)
    assert torch.allclose(p.sum(-1), torch.full((p.shape[0],), 2.0, dtype=torch.float64), atol=1e-5)
    # analytic inclusion probability when drawing 2 of 4 without replacement, proportional to a
    a = (x.double().abs() + 1.19209e-07).reshape(-1, 4)
    t = a / a.sum(-1, keepdim=True)
    want = t + (t.unsqueeze(-1) * t.unsqueeze(-2) / (1 - t).unsqueeze(-1)).sum(-2) - t * t / (1 - t)
    assert torch.allclose(p, want, atol=1e-5)


def test_mvue_two_kept_and_unbiased():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 16, generator=g).repeat(20000, 1)           # same four groups, many draws
    u = torch.rand(20000, 16, generator=g)
    values, meta, mask = oracle.mvue24(x, u, out_dtype=torch.float16)
    assert mask.reshape(-1, 4).sum(-1).eq(2).all()
    dense = oracle.decompress24(values, meta).float()
    est = dense.mean(0)
    assert torch.allclose(est, x[0], atol=0.05), (est, x[0])
    # empirical inclusion frequency matches p
    p = oracle.mvue24_probabilities(x[:1])[0]
    assert torch.allclose(mask.float().mean(0), p, atol=0.02)


def test_mvue_degenerate_groups():
    x = torch.zeros(2, 16)
    u = torch.tensor([[0.1, 0.9, 0, 0, 0.9, 0.1, 0, 0] * 2, [0.3, 0.5, 0, 0, 0.6, 0.99, 0, 0] * 2])
    values, meta, mask = oracle.mvue24(x, u)
    assert values.eq(0).all() and mask.reshape(-1, 4).sum(-1).eq(2).all()
    p = oracle.mvue24_probabilities(x)
    assert torch.allclose(p, torch.full_like(p, 0.5), atol=1e-6)
    # r0 = 0.1 picks element 0 (t_i = 1/4 each); r1 = 0.9 then picks the last remaining one
    assert mask[0, :4].tolist() == [True, False, False, True]


def test_mvue_first_draw_inverse_cdf():
    x = torch.ones(1, 16)
    for r0, first in [(0.2, 0), (0.3, 1), (0.6, 2), (0.9, 3)]:
        u = torch.tensor([[r0, 0.0, 0, 0] * 4])    # r1 = 0 -> second draw degenerates onto d_0
        _, _, mask = oracle.mvue24(x, u)
        assert mask[0, first]


def test_mvue_dense_twin_matches_compressed():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(32, 64, generator=g).half()
    u = torch.rand(32, 64, generator=g)
    values, meta, mask = oracle.mvue24(x, u, out_dtype=torch.float16)
    dense = oracle.mvue24_dense(x, u)
    assert dense.equal(oracle.decompress24(values, meta))


# ---------------------------------------------------------------- soft threshold
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_soft_threshold_vs_sort(dtype):
    # sort-based statement of sparse/legacy.py:95-114, valid on tie-free groups
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 64, generator=g).to(dtype)
    grp = x.float().reshape(-1, 4)
    srt = grp.abs().sort(-1).values
    tie_free = (srt[:, 1:] != srt[:, :-1]).all(-1)
    thr = srt[:, 1:2]
    keep = grp.abs() > thr
    want = torch.where(keep, grp - thr * grp.sign(), torch.zeros_like(grp)).to(dtype)
    sparse, mask = oracle.soft_threshold24(x)
    assert sparse.dtype == dtype and mask.dtype == dtype
    assert sparse.reshape(-1, 4)[tie_free].equal(want[tie_free])
    assert mask.reshape(-1, 4)[tie_free].equal(keep[tie_free].to(dtype))
    assert mask.float().reshape(-1, 4).sum(-1).eq(2).all()
    kept = mask.bool()
    assert (sparse[kept].float().sign() * x[kept].float().sign() >= 0).all()
    assert (sparse[kept].float().abs() <= x[kept].float().abs()).all()


def test_soft_threshold_ties():
    x = torch.tensor([[1.0, 1.0, 1.0, 1.0, 0.0, 0.0, 2.0, -3.0]])
    sparse, mask = oracle.soft_threshold24(x)
    assert sparse.shape == x.shape
    assert mask.tolist() == [[0, 0, 1, 1, 0, 0, 1, 1]]
    assert sparse.tolist() == [[0, 0, 0, 0, 0, 0, 2.0, -3.0]]


# ---------------------------------------------------------------- transposable search
_TABLE_SHA256 = "94a9cb4ad801a250c0d013a9cf2d7720f452e4e4ed77334aa2fd0ea1b1274862"


def test_pattern_table_closed_form():
    pats = oracle.transposable_patterns()
    assert pats.shape == (90, 16)
    blocks = pats.reshape(90, 4, 4)
    assert blocks.sum(1).eq(2).all() and blocks.sum(2).eq(2).all()
    as_lists = [tuple(p.tolist()) for p in pats]
    assert len(set(as_lists)) == 90 and as_lists == sorted(as_lists, reverse=True)
    assert as_lists[0] == (1, 1, 0, 0, 1, 1, 0, 0, 0, 0, 1, 1, 0, 0, 1, 1)
    assert hashlib.sha256(bytes(pats.reshape(-1).tolist())).hexdigest() == _TABLE_SHA256
    # complement reverses the order
    assert (1 - pats).equal(pats.flip(0))


def test_pattern_table_equals_reference_text():
    path = "/root/reference/sparse/transposable_semi_structured.py"
    if not os.path.exists(path):
        pytest.skip("reference not mounted")
    rows = re.findall(r"\[((?:[01], ){15}[01])\]", open(path).read())
    table = torch.tensor([[int(c) for c in r.split(", ")] for r in rows])
    assert table.equal(oracle.transposable_patterns())


def _exact_data(gen, m, k, dtype):
    # integers / 8 in [-4, 4): all pattern sums are exact in float32, many exact ties
    return (torch.randint(-32, 32, (m, k), generator=gen).float() / 8).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("use_abs", [True, False])
def test_transposable_equals_bruteforce_on_exact_data(dtype, use_abs):
    g = torch.Generator().manual_seed(4)
    w = _exact_data(g, 64, 128, dtype)
    sparse, mask, idx = oracle.transposable_mask(w, use_abs=use_abs, return_index=True)
    bs, bm, bidx = oracle.transposable_mask_bruteforce(w, use_abs=use_abs)
    assert idx.equal(bidx) and mask.equal(bm) and sparse.equal(bs)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_transposable_equals_bruteforce_on_random(dtype):
    g = torch.Generator().manual_seed(5)
    w = torch.randn(128, 256, generator=g).to(dtype)
    _, mask, idx = oracle.transposable_mask(w, return_index=True)
    _, bm, bidx = oracle.transposable_mask_bruteforce(w)
    assert idx.equal(bidx) and mask.equal(bm)


def test_transposable_invariants():
    g = torch.Generator().manual_seed(6)
    w = torch.randn(64, 128, generator=g)
    sparse, mask = oracle.transposable_mask(w)
    assert mask.dtype == torch.bool and sparse.dtype == w.dtype
    blk = mask.reshape(16, 4, 32, 4)
    assert blk.sum(1).eq(2).all() and blk.sum(3).eq(2).all()      # valid 2:4 for W and W.T
    assert sparse.equal(w * mask)
    # score of the chosen pattern >= score of every other pattern (fp64)
    pats = oracle.transposable_patterns().double()
    b = w.abs().double().reshape(16, 4, 32, 4).permute(0, 2, 1, 3).reshape(-1, 16)
    chosen = (b * mask.reshape(16, 4, 32, 4).permute(0, 2, 1, 3).reshape(-1, 16)).sum(-1)
    assert (chosen.unsqueeze(-1) >= (b @ pats.t()) - 1e-6).all()
    # constant block -> pattern 0
    _, m0 = oracle.transposable_mask(torch.ones(32, 64))
    assert m0[:4, :4].long().reshape(-1).tolist() == oracle.transposable_patterns()[0].tolist()


def test_transposable_validation():
    with pytest.raises(RuntimeError):
        oracle.transposable_mask(torch.zeros(33, 64))
    with pytest.raises(RuntimeError):
        oracle.transposable_mask(torch.zeros(32, 32))
    with pytest.raises(RuntimeError):
        oracle.transposable_mask(torch.zeros(32, 64, dtype=torch.float64))


# ---------------------------------------------------------------- masked decay
def test_masked_add_reference_smoke_vector():
    # sparse/decay.py:41-45
    grad = torch.tensor([1.0, 1.0, 1.0, 1.0])
    p = torch.tensor([1.0, 2.0, 3.0, 4.0])
    mask = torch.tensor([1.0, 0.0, 1.0, 0.0])
    out = oracle.masked_add(grad, p, mask, alpha=0.03)
    assert torch.allclose(out, torch.tensor([1.0, 1.06, 1.0, 1.12]), atol=1e-7)


def test_masked_add_docstring_equivalence():
    g = torch.Generator().manual_seed(7)
    grad = 1e-3 * torch.randn(64, 64, generator=g)
    p = torch.randn(64, 64, generator=g)
    mask = torch.rand(64, 64, generator=g) < 0.5
    want = grad.clone().add_(p * (1 - mask.float()), alpha=2e-4)
    out = oracle.masked_add(grad, p, mask, alpha=2e-4)
    assert torch.allclose(out, want, rtol=0, atol=1e-9)
    assert out[mask].equal(grad[mask])


# ------------------------------------------------------------------ AdamW with masked decay
def test_adamw_oracle_matches_torch_adamw_and_closed_form():
    """The oracle's AdamW against torch.optim.AdamW (an independent implementation of the same
    update) over several steps, and the first step's closed form."""
    g = torch.Generator().manual_seed(21)
    p0 = torch.randn(64, 96, generator=g)
    hyp = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    ref_p = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([ref_p], foreach=False, fused=False, **hyp)
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    for step in range(1, 6):
        grad = torch.randn(64, 96, generator=g)
        ref_p.grad = grad.clone()
        opt.step()
        p_prev = p
        p, m, v = oracle.adamw_masked_decay(p, grad, m, v, None, step, **hyp)
        assert torch.allclose(p, ref_p.detach(), rtol=1e-5, atol=1e-7)
        if step == 1:       # m = (1-b1) g, v = (1-b2) g^2: update = -lr * g / (|g| + eps * sqrt(1-b2)... ) ~ -lr * sign(g)
            want = p_prev * (1 - hyp["lr"] * hyp["weight_decay"]) - hyp["lr"] * grad / (grad.abs() + hyp["eps"])
            assert torch.allclose(p, want, rtol=1e-5, atol=1e-7)
    # the decay term enters through the gradient exactly as masked_add_ followed by the plain update
    mask = torch.rand(64, 96, generator=g) > 0.5
    grad = torch.randn(64, 96, generator=g)
    a = oracle.adamw_masked_decay(p, grad, m, v, mask, 6, alpha=2e-4, **hyp)
    b = oracle.adamw_masked_decay(p, oracle.masked_add(grad, p, mask, 2e-4), m, v, None, 6, **hyp)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_gelu_glu_oracle_matches_torch_gelu_and_autograd():
    """The GELU-GLU oracle is pinned by torch's own tanh-GELU and by autograd's gradient of
    gelu(gate) * x: swapped halves, a dropped factor or a sign error fails one of them."""
    g = torch.Generator().manual_seed(31)
    inp = (3 * torch.randn(5, 7, 24, generator=g, dtype=torch.float64)).requires_grad_(True)
    go = torch.randn(5, 7, 12, generator=g, dtype=torch.float64)
    out = oracle.gelu_glu_forward(inp.detach())
    x, gate = inp[..., :12], inp[..., 12:]
    ref = torch.nn.functional.gelu(gate, approximate='tanh') * x
    assert torch.allclose(out, ref.detach(), rtol=1e-12, atol=1e-14)
    (want,) = torch.autograd.grad(ref, inp, go)
    got = oracle.gelu_glu_backward(go, inp.detach())
    assert got.shape == inp.shape and torch.allclose(got, want, rtol=1e-10, atol=1e-12)
    # special values: gate = 0 gives out = 0 and d/dgate = x/2; a large gate passes x through
    z = torch.tensor([[[2.0, -3.0, 0.0, 0.0]]], dtype=torch.float64)
    assert oracle.gelu_glu_forward(z).abs().max() == 0
    assert torch.allclose(oracle.gelu_glu_backward(torch.ones(1, 1, 2, dtype=torch.float64), z)[..., 2:], torch.tensor([1.0, -1.5], dtype=torch.float64))
    big = torch.tensor([[[2.0, -3.0, 30.0, -30.0]]], dtype=torch.float64)
    assert torch.allclose(oracle.gelu_glu_forward(big), torch.tensor([[[60.0, 0.0]]], dtype=torch.float64), atol=1e-9)


@pytest.mark.parametrize("amsgrad", [False, True])
def test_adamw_step_oracle_phase1_is_adamw(amsgrad):
    """Phase 1 of the STEP update is AdamW: compare with torch.optim.AdamW over several steps."""
    g = torch.Generator().manual_seed(51)
    p0 = torch.randn(37, 5, generator=g)
    ref_p = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([ref_p], lr=3e-3, betas=(0.8, 0.95), eps=1e-6, weight_decay=0.05, amsgrad=amsgrad)
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    vmax = torch.zeros_like(p0) if amsgrad else None
    for step in range(1, 7):
        grad = torch.randn(37, 5, generator=g) * (0.5 if step % 2 else 2.0)      # shrinking gradients exercise the running max
        ref_p.grad = grad.clone()
        opt.step()
        p, m, v, vmax, change = oracle.adamw_step_update(p, grad, m, v, step, lr=3e-3, betas=(0.8, 0.95), eps=1e-6,
                                                         weight_decay=0.05, max_exp_avg_sq=vmax)
        assert torch.allclose(p, ref_p.detach(), rtol=2e-6, atol=1e-7)
    assert (vmax is None) == (not amsgrad)


def test_adamw_step_oracle_phase2_and_statistic():
    g = torch.Generator().manual_seed(52)
    p0, grad = torch.randn(64, generator=g), torch.randn(64, generator=g)
    m0, v0 = torch.randn(64, generator=g) * 0.1, torch.rand(64, generator=g) + 0.1
    kw = dict(lr=1e-2, betas=(0.9, 0.99), eps=0.0, weight_decay=0.01)
    step = 5
    p1, m1, v1, _, change = oracle.adamw_step_update(p0, grad, m0, v0, step, **kw)
    bc2 = 1 - 0.99 ** step
    # with eps = 0 and the frozen variance v_t / bc2, phase 2 gives phase 1's update
    p2, m2, v2, _, _ = oracle.adamw_step_update(p0, grad, m0, v0, step, precond_variance=v1 / bc2, **kw)
    assert torch.allclose(p2, p1, rtol=1e-6, atol=1e-7) and m2.equal(m1) and v2.equal(v1)
    # with eps > 0 phase 2 adds eps^(3/4) to sqrt(frozen variance), not eps
    kw["eps"] = 1e-4
    frozen = torch.full((64,), 4.0)
    p3, m3, _, _, _ = oracle.adamw_step_update(p0, grad, m0, v0, step, precond_variance=frozen, **kw)
    want = p0 * (1 - 1e-2 * 0.01) - 1e-2 / (1 - 0.9 ** step) * m3 / (2.0 + 1e-3)
    assert torch.allclose(p3, want, rtol=1e-6, atol=1e-7)
    # statistic at step 1 from zero state: v_1 - v_0 = (1 - beta2) g^2
    _, _, _, _, c1 = oracle.adamw_step_update(p0, grad, torch.zeros(64), torch.zeros(64), 1, **kw)
    z1 = oracle.variance_change_statistic([c1[:40], c1[40:]], option=1)
    assert abs(z1 - 0.01 * (grad.double() ** 2).mean().item()) < 1e-6 * z1 + 1e-12
    z2 = oracle.variance_change_statistic([c1], option=2)
    assert abs(z2 - 0.01 * math.exp((grad.double() ** 2).log().mean().item())) < 1e-5 * z2
    assert oracle.variance_change_statistic([torch.zeros(4)], option=2) == 0.0


def test_philox_known_answers():
    """Philox4x32-10 against the known-answer vectors of the Random123 distribution."""
    import numpy as np
    kats = [([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
            ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
            ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0], [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1])]
    for counter, key, want in kats:
        got = oracle.philox4x32_10(np.array(counter, dtype=np.uint64), np.array(key, dtype=np.uint64))
        assert [int(x) for x in got] == want
    u = oracle.mvue_uniforms(seed=1234, offset=8, m=32, k=64)
    assert u.shape == (32, 32) and u.dtype == torch.float32 and (u >= 0).all() and (u < 1).all()
    assert abs(u.mean().item() - 0.5) < 0.05 and not u.equal(oracle.mvue_uniforms(1234, 12, 32, 64))
    # row r, unit q of the row uses counter index r * (k/8) + q: the first unit of row 1 is call number k/8
    words = oracle.philox4x32_10(np.array([8, 0, 8, 0], dtype=np.uint64), np.array([1234, 0], dtype=np.uint64))
    assert u[1, 0].item() == float(int(words[0]) & 0xffffff) * 2.0 ** -24
