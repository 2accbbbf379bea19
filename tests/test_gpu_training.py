"""GPU integration: SparseLinearTranspose forward/backward against a dense masked autograd model,
a short masked-decay training loop (BASELINE config 4, reduced), and the fp8 path of config 5."""
import pytest
import torch
import torch.nn.functional as F

import oracle

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


def test_sparse_linear_transpose_matches_dense_masked(cuda):
    import sparse
    torch.manual_seed(0)
    layer = sparse.SparseLinearTranspose(256, 512, bias=True).to(cuda)
    x = torch.randn(4, 64, 256, device=cuda, requires_grad=True)
    y = layer(x)
    assert y.shape == (4, 64, 512) and y.dtype == torch.float16
    w = layer.weight.detach()
    # the mask is the transposable one of the master weight (bit-exact with the oracle)
    _, want_mask = oracle.transposable_mask(w.float().cpu())
    assert layer.weight.mask.cpu().equal(want_mask)
    wm = (w * layer.weight.mask).half()
    y_ref = F.linear(x.detach().half(), wm, layer.bias.detach().half())
    assert _rel(y, y_ref) < 1e-2
    gy = torch.randn_like(y)
    y.backward(gy)
    dx_ref = gy.reshape(-1, 512).float() @ wm.float()
    assert _rel(x.grad.reshape(-1, 256), dx_ref) < 1e-2
    db_ref = gy.reshape(-1, 512).float().sum(0)
    assert _rel(layer.bias.grad, db_ref) < 1e-2
    # dW is an MVUE estimate of dY^T x (pruned along the token axis): unbiased, so the mean of
    # several draws converges to the dense gradient
    dw_ref = gy.reshape(-1, 512).float().t() @ x.detach().reshape(-1, 256).half().float()
    assert layer.weight.grad.shape == (512, 256)
    single = _rel(layer.weight.grad, dw_ref)
    draws = []
    for _ in range(24):
        layer.weight.grad = None
        layer.weight.cnt = 0
        x2 = x.detach().clone().requires_grad_(True)
        layer(x2).backward(gy)
        draws.append(layer.weight.grad.float())
    mean_err = _rel(torch.stack(draws).mean(0), dw_ref)
    assert single < 1.0 and mean_err < 0.25 and mean_err < 0.6 * single, (single, mean_err)


def test_layer_state_machine(cuda):
    import sparse
    torch.manual_seed(1)
    layer = sparse.SparseLinearTranspose(128, 128, bias=False).to(cuda)
    w = layer.weight
    assert (w.freq, w.cnt, w.counter, w.step, w.mode) == (40, 0, 0, 0, 'sparse')
    x = torch.randn(32, 128, device=cuda)
    layer(x)
    first = w.weight_sparse
    assert (w.cnt, w.counter, w.step) == (1, 1, 1)
    layer(x)                                     # gradient accumulation: no recompression
    assert w.weight_sparse is first and (w.cnt, w.counter, w.step) == (2, 1, 2)
    w.cnt = 0                                    # what the optimizer hook does
    layer(x)
    assert w.weight_sparse is not first and w.counter == 2
    w.mode = 'dense'
    y = layer(x)
    assert torch.allclose(y, F.linear(x, w), atol=1e-5)
    layer.eval()
    w.mode = 'sparse'
    before = (w.cnt, w.counter, w.step)
    layer(x)
    assert (w.cnt, w.counter, w.step) == before


def test_masked_decay_training_loop(cuda):
    """BASELINE config 4 at reduced size: GELU MLP of two SparseLinearTranspose layers, fused
    AdamW, masked decay alpha = 2e-4 before every optimizer step, mask refresh every 5 steps."""
    import sparse
    torch.manual_seed(2)
    tokens, d, h = 512, 128, 256
    fc, proj = sparse.SparseLinearTranspose(d, h).to(cuda), sparse.SparseLinearTranspose(h, d).to(cuda)
    for layer in (fc, proj):
        torch.nn.init.normal_(layer.weight, std=0.02)
        layer.weight.freq = 5
    params = list(fc.parameters()) + list(proj.parameters())
    opt = torch.optim.AdamW(params, lr=3e-3, weight_decay=0.0, fused=True)
    x = torch.randn(tokens, d, device=cuda)
    target = torch.tanh(x @ torch.randn(d, d, device=cuda) * 0.3)
    losses, masks = [], []
    for step in range(20):
        out = proj(F.gelu(fc(x)))
        loss = F.mse_loss(out.float(), target)
        opt.zero_grad(set_to_none=True)
        loss.backward()
        with torch.no_grad():
            for p in params:
                if hasattr(p, 'mask') and p.mode == 'sparse':
                    p.grad = p.grad.float()
                    before = p.grad.clone()
                    sparse.masked_add_(p.grad.data, p.data, p.mask, alpha=2e-4)
                    want = oracle.masked_add(before.cpu(), p.data.cpu(), p.mask.cpu(), alpha=2e-4)
                    assert p.grad.cpu().equal(want)
                    p.cnt = 0
        opt.step()
        losses.append(loss.item())
        masks.append(fc.weight.mask.clone())
        if step % 5 == 0:       # refreshed on this forward pass from the weights before the update
            blk = fc.weight.mask.reshape(h // 4, 4, d // 4, 4)
            assert blk.sum(1).eq(2).all() and blk.sum(3).eq(2).all()
    assert losses[-1] < 0.7 * losses[0], losses
    assert masks[1].equal(masks[4]) and fc.weight.counter == 20       # constant between refreshes
    assert all(torch.isfinite(torch.tensor(losses)))


def test_fp8_mvue_spmm_config5_reduced(cuda):
    """Config 5 at reduced size: per-tensor amax scaling to e4m3, B pruned by MVUE24 with seeded
    uniforms, fp8 SMFMAC product with bf16 output, against the dense fp32 masked product."""
    import sparse
    g = torch.Generator().manual_seed(5)
    A = torch.randn(512, 1024, generator=g)
    B = torch.randn(256, 1024, generator=g)
    U = torch.rand(256, 1024, generator=g)
    sa, sb = 448.0 / A.abs().max(), 224.0 / B.abs().max()        # headroom: MVUE rescales kept values by up to 2x+
    Aq = (A * sa).to(torch.float8_e4m3fn)
    Bs = (B * sb).bfloat16()
    want_v, want_m, mask = oracle.mvue24(Bs, U, out_dtype=torch.float8_e4m3fn)
    s = sparse.to_sparse_semi_structured(Bs.to(cuda), MVUE24=True, rand=U.to(cuda), dtype=torch.float8_e4m3fn)
    assert s.values().cpu().view(torch.uint8).equal(want_v.view(torch.uint8))
    assert s.indices().cpu().equal(want_m)
    dense_b = oracle.decompress24(want_v, want_m).float()
    ref = (Aq.float() @ dense_b.t()) / (sa * sb)
    out = sparse.sparse_semi_structured_linear(Aq.to(cuda), s, out_dtype=torch.bfloat16, scale=float(1.0 / (sa * sb)))
    assert out.dtype == torch.bfloat16 and out.shape == (512, 256)
    assert _rel(out.cpu(), ref) < 5e-2
    # default dispatch returns float32 like the reference's CUTLASS path
    out32 = torch.mm(Aq.to(cuda), s.t())
    assert out32.dtype == torch.float32 and _rel(out32.cpu() / (sa * sb), ref) < 5e-2
    # soft threshold on the bf16 operand, as config 5 applies every iteration
    sp, mk = sparse.soft_threshold24_triton(Bs.to(cuda))
    wsp, wmk = oracle.soft_threshold24(Bs)
    assert sp.cpu().view(torch.int16).equal(wsp.view(torch.int16)) and mk.cpu().view(torch.int16).equal(wmk.view(torch.int16))


def test_functional_linear_entry_point(cuda):
    import sparse
    g = torch.Generator().manual_seed(6)
    w = torch.randint(-3, 4, (64, 128), generator=g).half()
    x = torch.randint(-3, 4, (2, 9, 128), generator=g).half()
    bias = torch.randint(-3, 4, (64,), generator=g).half()
    mask = oracle.prune24_mask(w)
    wm = torch.where(mask, w, torch.zeros_like(w))
    s = sparse.to_sparse_semi_structured(w.to(cuda))
    ref = oracle.linear_ref(x, wm, bias)
    out = sparse.sparse_semi_structured_linear(x.to(cuda), s, bias=bias.to(cuda))
    assert out.float().cpu().equal(ref)
    out = sparse.sparse_semi_structured_linear(x.to(cuda), s.values(), s.indices(), bias=bias.to(cuda), activation="relu")
    assert out.float().cpu().equal(ref.clamp_min(0))
    out = sparse.sparse_semi_structured_linear(x.to(cuda), s, activation="silu")
    ref_silu = F.silu(oracle.linear_ref(x, wm))
    assert torch.allclose(out.float().cpu(), ref_silu, rtol=2e-3, atol=2e-3)
    out = sparse.sparse_semi_structured_linear(x.to(cuda), s, activation="gelu")          # exact (erf) GELU
    assert torch.allclose(out.float().cpu(), F.gelu(oracle.linear_ref(x, wm)), rtol=2e-3, atol=2e-3)
    with pytest.raises(RuntimeError):
        sparse.sparse_semi_structured_linear(x.to(cuda), s, activation="tanh")


def test_my_linear_and_sparse_linear_modules(cuda):
    """sparse/sparse_ops.py: MyLinear is nn.Linear; SparseLinear has the same forward and weight/bias
    gradients, and dX = dY . MVUE24(W^T)^T with the uniforms of torch's generator."""
    import sparse
    torch.manual_seed(3)
    ref = torch.nn.Linear(128, 64).to(cuda)
    x = torch.randn(8, 16, 128, device=cuda)
    gy = torch.randn(8, 16, 64, device=cuda)
    for cls in (sparse.MyLinear, sparse.SparseLinear):
        mod = cls(128, 64).to(cuda)
        mod.load_state_dict(ref.state_dict())
        xr, xm = x.clone().requires_grad_(), x.clone().requires_grad_()
        yr, ym = ref(xr), mod(xm)
        assert torch.allclose(ym, yr, atol=1e-5, rtol=1e-5)
        ref.zero_grad()
        yr.backward(gy)
        torch.manual_seed(11)
        ym.backward(gy)
        assert torch.allclose(mod.weight.grad, ref.weight.grad, atol=1e-4, rtol=1e-4)
        assert torch.allclose(mod.bias.grad, ref.bias.grad, atol=1e-4, rtol=1e-4)
        if cls is sparse.MyLinear:
            assert torch.allclose(xm.grad, xr.grad, atol=1e-5, rtol=1e-5)
        else:
            torch.manual_seed(11)
            w_est = sparse.MVUE24_approx_triton(mod.weight.detach().t()).t()
            want = (gy.reshape(-1, 64) @ w_est).view_as(x)
            assert torch.allclose(xm.grad, want, atol=1e-5, rtol=1e-5)
            assert ((w_est != 0).t().reshape(-1, 4).sum(-1) <= 2).all()        # 2:4 along the output axis


def test_soft_threshold_linear_module(cuda):
    """README S-STE recipe: forward uses scale * soft_threshold24(W); the gradient passes straight
    through to W; init_scale is the least-squares scale."""
    import sparse
    torch.manual_seed(4)
    mod = sparse.SoftThresholdLinear(128, 64).to(cuda)
    mod.init_scale()
    w = mod.weight.detach()
    ws, _ = oracle.soft_threshold24(w.cpu())
    want_scale = (w.cpu().flatten() @ ws.flatten()) / (ws.flatten() @ ws.flatten())
    assert abs(mod.scale.item() - want_scale.item()) < 1e-5 and mod.scale.item() > 1.0
    x = torch.randn(32, 128, device=cuda)
    y = mod(x)
    want = F.linear(x, ws.to(cuda) * mod.scale, mod.bias)
    assert torch.allclose(y, want, atol=1e-5, rtol=1e-5)
    gy = torch.randn_like(y)
    y.backward(gy)
    assert torch.allclose(mod.weight.grad, gy.t() @ x, atol=1e-4, rtol=1e-4)     # straight-through
    # STEP recipe: magnitude-pruned weight with a straight-through gradient
    w2 = torch.randn(64, 128, device=cuda, requires_grad=True)
    sp = sparse.Sparse24.apply(w2)
    want_sp, _ = oracle.sparse24_dense(w2.detach().cpu())
    assert sp.detach().cpu().equal(want_sp)
    sp.backward(torch.ones_like(sp))
    assert w2.grad.equal(torch.ones_like(w2))


@pytest.mark.parametrize("gdt", [torch.float32, torch.float16])
def test_masked_decay_adamw_kernel(cuda, gdt):
    """One fused pass against the oracle (float32; rtol 2e-6: torch's CPU ops may contract a
    multiply-add that the kernel rounds twice) and against the two-pass recipe it replaces."""
    import sparse
    g = torch.Generator().manual_seed(31)
    hyp = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    p0 = torch.randn(96, 200, generator=g)                      # 19200 elements + odd tail coverage below
    mask = torch.rand(96, 200, generator=g) > 0.5
    par = torch.nn.Parameter(p0.clone().to(cuda))
    par.mask, par.mode, par.cnt = mask.to(cuda), "sparse", 3
    plain = torch.nn.Parameter(torch.randn(1003, generator=g).to(cuda))        # no mask, unaligned tail
    if gdt != torch.float32:
        par.grad_dtype = plain.grad_dtype = None                 # let the float32 parameters hold half gradients
    opt = sparse.MaskedDecayAdamW([par, plain], alpha=2e-4, **hyp)
    ref_par = torch.nn.Parameter(p0.clone().to(cuda))
    ref_plain = torch.nn.Parameter(plain.detach().clone())
    ref_opt = torch.optim.AdamW([ref_par, ref_plain], foreach=False, fused=False, **hyp)
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    q, qm, qv = plain.detach().cpu().clone(), torch.zeros(1003), torch.zeros(1003)
    for step in range(1, 5):
        grad = torch.randn(96, 200, generator=g).to(gdt)
        grad2 = torch.randn(1003, generator=g).to(gdt)
        par.grad, plain.grad = grad.to(cuda), grad2.to(cuda)
        opt.step()
        assert par.cnt == 0
        p, m, v = oracle.adamw_masked_decay(p, grad, m, v, mask, step, alpha=2e-4, **hyp)
        q, qm, qv = oracle.adamw_masked_decay(q, grad2, qm, qv, None, step, **hyp)
        assert torch.allclose(par.detach().cpu(), p, rtol=2e-6, atol=1e-8)
        assert torch.allclose(opt.state[par]["exp_avg"].cpu(), m, rtol=2e-6, atol=1e-10)
        assert torch.allclose(opt.state[par]["exp_avg_sq"].cpu(), v, rtol=2e-6, atol=1e-12)
        assert torch.allclose(plain.detach().cpu(), q, rtol=2e-6, atol=1e-8)
        # the recipe it replaces: masked_add_ on the float32 gradient, then an AdamW step
        ref_par.grad = grad.to(cuda).float()
        sparse.masked_add_(ref_par.grad, ref_par.data, par.mask, alpha=2e-4)
        ref_plain.grad = grad2.to(cuda).float()
        ref_opt.step()
        assert torch.allclose(par.detach(), ref_par.detach(), rtol=1e-5, atol=1e-7)
        assert torch.allclose(plain.detach(), ref_plain.detach(), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
def test_masked_decay_adamw_step_count_on_the_device(cuda, gdt):
    """capturable=True: the step count is an int64 in device memory and the bias corrections 1 - beta^step are
    formed by the kernel.  Twelve updates must leave parameters and moments bit-equal to the optimizer with the
    count on the host (same double-precision formulas, rounded to float32 at the same places), for a masked
    parameter and an unmasked one with an odd length; then a single update recorded into a HIP graph and replayed
    three times must continue the same sequence (a recording with the count frozen in it would not)."""
    import sparse
    g = torch.Generator().manual_seed(33)
    hyp = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, alpha=2e-4)
    p0, q0 = torch.randn(96, 200, generator=g), torch.randn(1003, generator=g)
    mask = (torch.rand(96, 200, generator=g) > 0.5).to(cuda)
    models = []
    for capturable in (False, True):
        par, plain = torch.nn.Parameter(p0.clone().to(cuda)), torch.nn.Parameter(q0.clone().to(cuda))
        par.mask, par.mode, par.cnt = mask, "sparse", 0
        if gdt != torch.float32:
            par.grad_dtype = plain.grad_dtype = None
        par.grad, plain.grad = torch.zeros(96, 200, device=cuda, dtype=gdt), torch.zeros(1003, device=cuda, dtype=gdt)
        models.append((par, plain, sparse.MaskedDecayAdamW([par, plain], capturable=capturable, **hyp)))
    (hp, hq, hopt), (dp, dq, dopt) = models

    def same(step):
        for a, b in ((hp, dp), (hq, dq)):
            assert torch.equal(a, b), step
            assert torch.equal(hopt.state[a]["exp_avg"], dopt.state[b]["exp_avg"]), step
            assert torch.equal(hopt.state[a]["exp_avg_sq"], dopt.state[b]["exp_avg_sq"]), step
            assert int(dopt.state[b]["step"]) == hopt.state[a]["step"] == step

    grads = [(torch.randn(96, 200, generator=g).to(gdt).to(cuda), torch.randn(1003, generator=g).to(gdt).to(cuda)) for _ in range(15)]
    for step in range(1, 13):
        for par, plain, opt in models:
            par.grad.copy_(grads[step - 1][0]); plain.grad.copy_(grads[step - 1][1])
            opt.step()
        same(step)
    assert dopt.state[dp]["step"].is_cuda and dopt.state[dp]["step"].dtype == torch.int64
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        dopt.step()
    for step in range(13, 16):
        dp.grad.copy_(grads[step - 1][0]); dq.grad.copy_(grads[step - 1][1])
        graph.replay()
        hp.grad.copy_(grads[step - 1][0]); hq.grad.copy_(grads[step - 1][1])
        hopt.step()
        torch.cuda.synchronize()
        same(step)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.float16, 1e-3), (torch.bfloat16, 8e-3)])
@pytest.mark.parametrize("shape", [(4, 32, 256), (3, 5, 24), (2, 7, 10), (1, 1, 2)])
@pytest.mark.parametrize("transposed", [False, True])
def test_gelu_glu_forward_backward(cuda, dtype, tol, shape, transposed):
    """GELUglu against the float64 oracle.  Tolerances: float32 arithmetic then one rounding to the
    storage type, so 2e-6 (float32), 2^-10 (float16) and 2^-7 (bfloat16) of the largest
    magnitude; `transposed` stores the last dimension strided (the reference's 2-d path)."""
    import sparse
    g = torch.Generator().manual_seed(41)
    a, b, c = shape
    inp = (2 * torch.randn(a * b, c, generator=g)).to(dtype)
    go = torch.randn(a * b, c // 2, generator=g).to(dtype)
    dev_in = inp.to(cuda)
    if transposed:
        dev_in = dev_in.t().contiguous().t()                    # same values, column-major storage
    dev_in = dev_in.view(a, b, c).requires_grad_(True)
    out = sparse.GELUglu()(dev_in)
    want = oracle.gelu_glu_forward(inp.view(a, b, c))
    assert out.shape == (a, b, c // 2) and out.dtype == dtype
    scale = want.abs().max().item()
    assert (out.double().cpu() - want).abs().max().item() <= tol * scale + 1e-30
    out.backward(go.to(cuda).view(a, b, c // 2))
    want_g = oracle.gelu_glu_backward(go.view(a, b, c // 2), inp.view(a, b, c))
    assert dev_in.grad.shape == (a, b, c) and dev_in.grad.dtype == dtype
    gscale = want_g.abs().max().item()
    assert (dev_in.grad.double().cpu() - want_g).abs().max().item() <= tol * gscale + 1e-30


def test_gelu_glu_errors(cuda):
    import sparse
    with pytest.raises(RuntimeError):
        sparse.gelu_glu.apply(torch.zeros(2, 3, 5, device=cuda))          # odd last dimension
    with pytest.raises(RuntimeError):
        sparse.gelu_glu.apply(torch.zeros(2, 3, 4))                       # not on the GPU
    with pytest.raises(AssertionError):
        sparse.gelu_glu.apply(torch.zeros(6, 4, device=cuda))             # the reference asserts a 3-d input


@pytest.mark.parametrize("grad_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("amsgrad", [False, True])
@pytest.mark.parametrize("n,offset", [(4096, 0), (1031, 0), (2050, 1)])
def test_adamw_step_kernel_matches_oracle(cuda, grad_dtype, amsgrad, n, offset):
    """tf24_adamw_step against the oracle over several steps, both phases, with the variance-change
    partial sums; `offset` shifts the tensors off 16-byte alignment (scalar-access variant).
    Tolerance 2e-6 relative: float32 arithmetic, torch may contract the oracle's multiply-adds."""
    from sparse import _native as N
    lib = N.lib()
    g = torch.Generator().manual_seed(61)
    hp = dict(lr=2e-3, betas=(0.9, 0.98), eps=1e-7, weight_decay=0.02)

    def dev(t):                                   # a view that starts `offset` elements into its buffer
        buf = torch.zeros(t.numel() + 8, dtype=t.dtype, device=cuda)
        buf[offset:offset + t.numel()] = t.to(cuda)
        return buf[offset:offset + t.numel()]

    p = torch.randn(n, generator=g)
    m, v = torch.zeros(n), torch.zeros(n)
    vmax = torch.zeros(n) if amsgrad else None
    dp, dm, dv = dev(p), dev(m), dev(v)
    dx = dev(vmax) if amsgrad else None
    nz = lib.tf24_adamw_step_partials(n)
    assert nz == (n + 1023) // 1024
    frozen = None
    for step in range(1, 6):
        grad = (torch.randn(n, generator=g) * (1.5 if step % 2 else 0.3)).to(grad_dtype)
        dg = dev(grad)
        phase2 = step >= 4
        if phase2 and frozen is None:
            frozen = (vmax if amsgrad else v).clone()
            dfrozen = dev(frozen)
        for option in ([2, 1] if step == 2 else [1]):       # option 2 runs on copies first: the update itself is the same
            z = torch.full((nz,), float("nan"), dtype=torch.float32, device=cuda)
            args = [t.clone() for t in (dp, dm, dv)] if option == 2 else [dp, dm, dv]
            N.check(lib.tf24_adamw_step(
                args[0].data_ptr(), dg.data_ptr(), N.dtype_code(grad_dtype), args[1].data_ptr(), args[2].data_ptr(),
                (dx.clone() if option == 2 else dx).data_ptr() if amsgrad else None, dfrozen.data_ptr() if phase2 else None,
                n, hp["lr"], hp["betas"][0], hp["betas"][1], hp["eps"], hp["weight_decay"], step,
                None if phase2 else z.data_ptr(), 0 if phase2 else option, N.stream_ptr()))
            if not phase2:
                _, _, _, _, change = oracle.adamw_step_update(p, grad, m, v, step, max_exp_avg_sq=vmax, **hp)
                want_z = oracle.variance_change_statistic([change], option=option)
                got = z.double().sum().item() / n
                got = got if option == 1 else torch.exp(torch.tensor(got, dtype=torch.float64)).item()
                assert abs(got - want_z) <= 2e-5 * abs(want_z) + 1e-12, (step, option, got, want_z)
        p, m, v, vmax, _ = oracle.adamw_step_update(p, grad, m, v, step, max_exp_avg_sq=vmax,
                                                    precond_variance=frozen if phase2 else None, **hp)
        for got, want in ((dp, p), (dm, m), (dv, v)) + (((dx, vmax),) if amsgrad else ()):
            assert torch.allclose(got.cpu(), want, rtol=2e-6, atol=1e-9), step


def test_adamw_step_optimizer_phases(cuda):
    """The AdamW_STEP class: watches only parameters carrying `mask`, switches at t > T_max, freezes the
    variance, and from then on divides tracked parameters by it; untracked ones stay on AdamW."""
    import sparse
    torch.manual_seed(62)
    w = torch.nn.Parameter(torch.randn(48, 40, device=cuda))
    b = torch.nn.Parameter(torch.randn(40, device=cuda))
    w.mask = 'dense'
    hp = dict(lr=1e-2, betas=(0.9, 0.5), eps=1e-8, weight_decay=0.01)
    opt = sparse.AdamW_STEP([w, b], clipping=(1, 3), option=1, **hp)
    assert opt.T_omega == 2 and opt.mask == 'dense'
    ow, ob = w.detach().cpu().clone(), b.detach().cpu().clone()
    mw, vw, mb, vb = torch.zeros_like(ow), torch.zeros_like(ow), torch.zeros_like(ob), torch.zeros_like(ob)
    frozen = None
    g = torch.Generator().manual_seed(63)
    for t in range(1, 7):
        gw, gb = torch.randn(48, 40, generator=g), torch.randn(40, generator=g)
        w.grad, b.grad = gw.to(cuda), gb.to(cuda)
        opt.step()
        ow, mw, vw, _, change = oracle.adamw_step_update(ow, gw, mw, vw, t, precond_variance=frozen, **hp)
        ob, mb, vb, _, _ = oracle.adamw_step_update(ob, gb, mb, vb, t, **hp)
        assert torch.allclose(w.detach().cpu(), ow, rtol=3e-6, atol=1e-8), t
        assert torch.allclose(b.detach().cpu(), ob, rtol=3e-6, atol=1e-8), t
        if t <= 3:
            assert opt.mask == 'dense' and w.mask == 'dense' and len(opt.sliding_window) == min(t, 2)
            z = oracle.variance_change_statistic([change], option=1)
            assert abs(opt.sliding_window[-1].item() - z) <= 1e-5 * z
        elif t == 4:                                                      # t > T_max = 3: switched after this update
            assert opt.mask == 'sparse' and w.mask == 'sparse'
            frozen = vw.clone()
            assert torch.allclose(opt.state[w]['preconditioned_variance'].cpu(), frozen, rtol=3e-6, atol=1e-12)
            assert 'preconditioned_variance' not in opt.state[b]
    assert opt.t == 6 and len(opt.sliding_window) == 2                    # the window stops growing after the switch
    with pytest.raises(ValueError):
        sparse.AdamW_STEP([w], option=3)


def test_entry_points_under_graph_capture(cuda):
    """The library only launches kernels on the stream it is given (no allocation, no synchronisation,
    no memset), so its calls can be recorded into a HIP graph: compression, both matmul forms (the
    split one with its workspace and reduction) and the masked decay are captured once and replayed
    on new contents of the same buffers, with eager work between the replays; every replay must give
    the bits of the eager calls."""
    import sparse
    n, k, m = 512, 4096, 48
    gen = torch.Generator().manual_seed(71)
    w = torch.randn(n, k, generator=gen).half().to(cuda)
    x = torch.randn(m, k, generator=gen).half().to(cuda)
    g32 = torch.randn(n, k, generator=gen).to(cuda)

    def work():
        s = sparse.to_sparse_semi_structured(w)                     # magnitude rule: no random numbers
        y = torch.mm(x, s.t())                                      # few dense columns: k pieces + reduction
        z = torch.mm(s, w.t())                                      # [n, n]: k-strided dense operand
        grad = g32.clone()
        sparse.masked_add_(grad, w.float(), (s.to_dense() != 0), alpha=2e-4)
        return y, z, grad

    work()                                                          # warm up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            captured = work()
    torch.cuda.synchronize()
    for it in range(3):
        w.copy_(torch.randn(n, k, generator=gen).half())
        x.copy_(torch.randn(m, k, generator=gen).half())
        g32.copy_(torch.randn(n, k, generator=gen))
        eager = [t.clone() for t in work()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("x @ S.t", "S @ w.t", "masked decay"), captured, eager):
            assert torch.equal(a, b), (it, name)
