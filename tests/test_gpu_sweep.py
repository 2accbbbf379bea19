"""GPU parity, randomized: seeded sweeps over shapes, dtypes, memory orders, padded leading
dimensions and operand positions that the hand-picked cases of test_gpu_parity.py do not enumerate.
The matmul is compared with the exact product of small-integer operands (every partial sum is an
integer below 2^24, so float32 accumulation in any order gives the same bits); the conversion
kernels with the oracle bit for bit (NaN positions, not NaN payloads).  A failing case prints its
parameters."""
import random

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F16, BF16, F32, E4M3, E5M2, I8 = (torch.float16, torch.bfloat16, torch.float32, torch.float8_e4m3fn,
                                  torch.float8_e5m2, torch.int8)
EIGHT_BIT = (E4M3, E5M2, I8)


def _ints(shape, seed, lo=-2, hi=3):
    return torch.randint(lo, hi, shape, generator=torch.Generator().manual_seed(seed)).float()


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t if t.dtype == torch.bool else t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def _same(a, b):
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    a, b = a.detach().cpu(), b.detach().cpu()
    if a.dtype.is_floating_point:
        na, nb = a.float().isnan(), b.float().isnan()
        if not na.equal(nb):
            return False
        zero = torch.zeros((), dtype=torch.float32)
        a, b = torch.where(na, zero, a.float()).to(a.dtype), torch.where(nb, zero, b.float()).to(b.dtype)
    return _bits(a).equal(_bits(b))


def _store(x, col_major, pad, dev):
    """x on the device, row- or column-major, with `pad` unused elements after every line."""
    if col_major:
        buf = torch.zeros((x.shape[1], x.shape[0] + pad), dtype=x.dtype, device=dev)
        buf[:, :x.shape[0]] = x.t().to(dev)
        return buf[:, :x.shape[0]].t()
    buf = torch.zeros((x.shape[0], x.shape[1] + pad), dtype=x.dtype, device=dev)
    buf[:, :x.shape[1]] = x.to(dev)
    return buf[:, :x.shape[1]]


@pytest.mark.parametrize("seed,large", [(1, False), (2, False), (3, True)])
def test_spmm_sweep(cuda, seed, large):
    """Every kernel of the matmul (one-pass, 64-, 128- and 256-wide tiles with and without k pieces,
    general) is reached by some of these shapes; all five operand dtypes, all operand positions."""
    import sparse
    rng = random.Random(seed)
    failures = []
    for case in range(40 if large else 150):
        dtype = rng.choice([F16, F16, BF16, E4M3, E5M2, I8])
        eight = dtype in EIGHT_BIT
        n = 32 * (rng.choice([8, 24, 33, 64, 96, 129, 172, 256, 344]) if large else rng.choice([1, 2, 3, 5, 8, 9, 10, 16, 17, 24, 33, 40]))
        k = (128 if eight else 64) * (rng.choice([16, 24, 33, 48, 64, 96, 128]) if large else rng.choice([1, 2, 3, 4, 7, 8, 16, 24, 32, 33, 64]))
        m = rng.choice([8, 16, 24, 40, 64, 72, 96, 128, 136, 200, 256, 264, 520])
        if eight and m % 16:
            m += 8
        form = rng.choice(["x@S.t", "xT@S.t", "S@xT", "S@xTc", "addmm", "linear_relu"])
        data_seed = rng.randrange(1 << 30)
        if n * k * m > 2 ** 33:
            continue
        w, x, bias = _ints((n, k), data_seed), _ints((m, k), data_seed + 1), _ints((n,), data_seed + 2)
        ref = x @ torch.where(oracle.prune24_mask(w), w, torch.zeros(())).t()
        src = w.to(I8) if dtype == I8 else w
        s = sparse.to_sparse_semi_structured(src.to(cuda), dtype=dtype)
        xg = x.to(dtype).to(cuda)
        if form == "x@S.t":
            out, want = torch.mm(xg, s.t()), ref
        elif form == "xT@S.t":
            out, want = torch.mm(xg.t().contiguous().t(), s.t()), ref
        elif form == "S@xT":
            out, want = torch.mm(s, xg.t()), ref.t()
        elif form == "S@xTc":
            out, want = torch.mm(s, xg.t().contiguous()), ref.t()
        else:
            bias_dtype = torch.int32 if dtype == I8 else F32 if eight else dtype
            bg = bias.to(bias_dtype).to(cuda)
            if form == "addmm":
                out, want = torch.addmm(bg, xg, s.t()), ref + bias
            else:
                out, want = sparse.sparse_semi_structured_linear(xg, s, bias=bg, activation="relu"), (ref + bias).clamp_min(0)
        want = want.to(out.dtype).double() if out.dtype.is_floating_point else want.double()
        got = out.double().cpu()
        if got.shape != want.shape or not got.equal(want):
            failures.append(f"case {case}: {dtype} n={n} k={k} m={m} {form} data_seed={data_seed}")
    assert not failures, failures


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_conversion_sweep(cuda, seed):
    """Magnitude / mask / MVUE24 (supplied and in-kernel uniforms) compression, the W + W^T pair,
    compression with row sums, the transposable mask, the soft threshold and the masked decay on
    random shapes, input and output dtypes, memory orders and padded leading dimensions."""
    import sparse
    rng = random.Random(seed)
    failures = []
    for case in range(200):
        op = rng.choice(["magnitude", "mask", "mvue", "seeded", "seeded", "pair", "rowsum", "transposable", "soft", "masked_add"])
        in_dtype = rng.choice([F32, F16, BF16])
        out_dtype = rng.choice([F16, F16, BF16, E4M3, E5M2])
        unit = 128 if out_dtype in EIGHT_BIT else 64
        m = unit * rng.choice([1, 2, 3, 5, 8]) if op == "pair" else 32 * rng.choice([1, 2, 3, 4, 6, 8, 11, 16, 40])
        k = unit * rng.choice([1, 2, 3, 5, 8, 13, 16])
        col = rng.random() < 0.5
        pad = 0 if op == "masked_add" else rng.choice([0, 0, 8, 16, 24])      # the masked decay wants dense memory
        data_seed = rng.randrange(1 << 30)
        g = torch.Generator().manual_seed(data_seed)
        w = torch.randn((m, k), generator=g)
        if rng.random() < 0.3:
            w = (w * 2).round() / 2                                             # ties, zeros, dominated groups
        w = w.to(in_dtype)
        wd = _store(w, col, pad, cuda)
        what = f"case {case}: {op} {in_dtype}->{out_dtype} m={m} k={k} col={col} pad={pad} data_seed={data_seed}"
        if op == "magnitude":
            v, mt = oracle.compress24(w, out_dtype=out_dtype)
            s = sparse.to_sparse_semi_structured(wd, dtype=out_dtype)
            ok = _same(s.values(), v) and _same(s.indices(), mt)
        elif op == "mask":
            mask = (torch.rand((m, k), generator=g) < 0.5) if rng.random() < 0.3 else oracle.transposable_mask(w.float())[1]
            mask = mask.to(rng.choice([torch.bool, BF16, F32, F16]))
            v, mt = oracle.compress24(w, mask=mask, out_dtype=out_dtype)
            s = sparse.to_sparse_semi_structured(wd, mask=_store(mask, col, pad, cuda), dtype=out_dtype)
            ok = _same(s.values(), v) and _same(s.indices(), mt)
        elif op in ("mvue", "rowsum"):
            u = torch.rand((m, k), generator=g)
            v, mt, _ = oracle.mvue24(w, u, out_dtype=out_dtype)
            if op == "mvue":
                s = sparse.to_sparse_semi_structured(wd, MVUE24=True, rand=_store(u, col, pad, cuda), dtype=out_dtype)
                ok = True
            else:
                s, sums = sparse.to_sparse_semi_structured_with_row_sums(wd, MVUE24=True, rand=_store(u, col, pad, cuda), dtype=out_dtype)
                # float32 sums rounded once to the input dtype: within an ulp of the input dtype of the float64 sum,
                # relative to the sum of magnitudes (cancellation)
                tol = {F32: 1e-5, F16: 2e-3, BF16: 1.6e-2}[in_dtype]
                ok = bool(((sums.double().cpu() - w.double().sum(1)).abs() <= tol * w.double().abs().sum(1) + 1e-6).all())
            ok = ok and _same(s.values(), v) and _same(s.indices(), mt)
        elif op == "seeded":
            sd, off = rng.randrange(1 << 62), 4 * rng.randrange(1 << 20)
            packed = oracle.mvue_uniforms(sd, off, m, k)
            u = torch.zeros((m, k))
            u[:, 0::4], u[:, 1::4] = packed[:, 0::2], packed[:, 1::2]
            v, mt, _ = oracle.mvue24(w, u, out_dtype=out_dtype)
            if col and out_dtype in (F16, BF16) and rng.random() < 0.5:
                s, _ = sparse.to_sparse_semi_structured_with_row_sums(wd, MVUE24=True, rand=(sd, off), dtype=out_dtype)
            else:
                s = sparse.to_sparse_semi_structured(wd, MVUE24=True, rand=(sd, off), dtype=out_dtype)
            ok = _same(s.values(), v) and _same(s.indices(), mt)
        elif op == "pair":
            mask = oracle.transposable_mask(w.float())[1]
            v, mt = oracle.compress24(w, mask=mask, out_dtype=out_dtype)
            vt, mtt = oracle.compress24(w.t().contiguous(), mask=mask.t().contiguous(), out_dtype=out_dtype)
            s, st = sparse.to_sparse_semi_structured_pair(wd, _store(mask, col, pad, cuda), dtype=out_dtype)
            ok = _same(s.values(), v) and _same(s.indices(), mt) and _same(st.values(), vt) and _same(st.indices(), mtt)
        elif op == "transposable":
            ws = torch.randint(-8, 9, (m, k), generator=g).to(in_dtype)         # exactly summable scores
            want, mask = oracle.transposable_mask(ws.float())
            out, mk = sparse.TransposableSparse(abs=True)(_store(ws, col, pad, cuda))
            ok = mk.cpu().equal(mask) and _same(out.cpu().float(), want.float())
        elif op == "soft":
            want = oracle.soft_threshold24(w)
            got = sparse.soft_threshold24(wd)
            want, got = (want[0] if isinstance(want, tuple) else want), (got[0] if isinstance(got, tuple) else got)
            ok = _same(got, want.to(got.dtype))
        else:
            mask = oracle.prune24_mask(w.float())
            p32, g32 = w.float(), torch.randn((m, k), generator=g)
            want = oracle.masked_add(g32.clone(), p32, mask, 2e-4)
            gd = _store(g32, col, 0, cuda)
            sparse.masked_add_(gd, _store(p32, col, 0, cuda), _store(mask, col, 0, cuda), alpha=2e-4)
            ok = _same(gd, want)
        if not ok:
            failures.append(what)
    assert not failures, failures
