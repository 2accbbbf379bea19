"""BASELINE config 4 at its stated size under pytest: the SparseLinearTranspose training step of the
GPT-2-124M MLP (README.md:125-213 of the reference) -- 12 x 1024 = 12288 tokens, c_fc 768 -> 3072,
GELU, c_proj 3072 -> 768, weights N(0, 0.02), inputs N(0, 1), fp16 autocast, transposable mask
refreshed every 40 optimizer steps, both compressed copies rebuilt every step, masked decay
alpha = 2e-4, fused AdamW, 100 steps, seed 2.

What is checked, and against what:
  * masks: at steps 0, 40 and 80 the layer's mask equals oracle.transposable_mask of the master
    weight as it was before that step's update (bit-exact); in between it does not change;
  * one step's tensors (steps 0, 1, 40, 99) against a dense masked model in plain PyTorch on the same
    device: both forward products, both dX products and both bias gradients within rel-err 1e-2
    (fp16 products with fp32 accumulation on either side; the tolerance BASELINE states);
  * dW: the layer's MVUE24 sample is reproduced from the generator's (seed, offset) -- the uniforms
    through tf24_mvue_uniforms, the estimate through the dense-shaped MVUE24 operator (itself
    bit-exact against the oracle, and compared with the CPU oracle here once at full width) -- so
    dW = MVUE24(dY^T) . x can be compared value for value with a float32 product of the same
    operands: rel-err 1e-3 (exact fp16 products, float32 sums in different orders);
  * the loss curve against the same MLP trained dense-masked (straight-through) in plain PyTorch with
    exact dW: the MVUE noise of dW over 12288 tokens moves the curve by well under the band.
The run with MaskedDecayAdamW (decay folded into the optimizer) must reproduce the run with
masked_add_ + torch's fused AdamW: same generator stream, so same samples; the two differ by float32
rounding of the update only.
"""
import pytest
import torch
import torch.nn.functional as F

import oracle

pytestmark = pytest.mark.gpu

TOKENS, D, H = (12, 1024), 768, 3072
STEPS, FREQ, ALPHA, LR = 100, 40, 2e-4, 1e-3
CHECK_STEPS = (0, 1, 40, 99)
LOSS_BAND = 0.05          # |loss - loss_dense_masked| / loss_dense_masked, every step
# fp16 gradients need a loss scale (a mean over 12288 x 768 outputs puts dY at 1e-7, below fp16's
# normal range); a power of two, so scaling and unscaling are exact
LOSS_SCALE = 4096.0


def _loss(out, target):
    return F.mse_loss(out.float(), target)


def _rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


def _full_uniforms(seed, offset, m, k, device):
    """The [m, k] uniforms tensor whose entries [r, 4g], [r, 4g+1] are the two uniforms the seeded
    MVUE24 kernel draws for group g of row r (tf24_mvue_uniforms writes them packed as [m, k/2])."""
    from sparse import _native as N
    packed = torch.empty((m, k // 2), dtype=torch.float32, device=device)
    N.check(N.lib().tf24_mvue_uniforms(seed, offset, m, k, N.ROW_MAJOR, packed.data_ptr(), k // 2, N.stream_ptr()))
    full = torch.zeros((m, k), dtype=torch.float32, device=device)
    full[:, 0::4] = packed[:, 0::2]
    full[:, 1::4] = packed[:, 1::2]
    return full, packed


def _mvue_dw(grad_out2d, x2d, seed, offset):
    """MVUE24(dY^T) . x with the sample the layer's backward drew at (seed, offset), as a float32
    product of the dense-shaped estimate; also returns the estimate and the uniforms."""
    import sparse
    gt = grad_out2d.t()                                   # [features_out, tokens], column-major view
    u, packed = _full_uniforms(seed, offset, gt.shape[0], gt.shape[1], grad_out2d.device)
    est = sparse.MVUE24_approx(gt, rand=u)                # dense-shaped, zeros at dropped positions
    return est.float() @ x2d.float(), est, u, packed


def _make(cuda):
    import sparse
    torch.manual_seed(2)
    fc = sparse.SparseLinearTranspose(D, H).to(cuda)
    proj = sparse.SparseLinearTranspose(H, D).to(cuda)
    for layer in (fc, proj):
        torch.nn.init.normal_(layer.weight, std=0.02)
        assert layer.weight.freq == FREQ
    x = torch.randn(*TOKENS, D, device=cuda)
    teacher = torch.randn(D, D, device=cuda) * 0.05
    target = torch.tanh(x @ teacher)
    return fc, proj, x, target


def _dense_masked_twin(fc, proj):
    """Float32 master copies of the two layers for the plain-PyTorch model."""
    ps = [p.detach().clone().requires_grad_(True) for p in (fc.weight, fc.bias, proj.weight, proj.bias)]
    return ps, torch.optim.AdamW(ps, lr=LR, fused=True)


def _twin_step(ps, opt, masks, x, target, step):
    wfc, bfc, wproj, bproj = ps
    if step % FREQ == 0:
        masks[0] = oracle.transposable_mask(wfc.detach().float().cpu())[1].to(x.device)
        masks[1] = oracle.transposable_mask(wproj.detach().float().cpu())[1].to(x.device)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        # straight-through: the product uses W * mask, the gradient reaches every element of W
        mfc = wfc + (wfc * masks[0] - wfc).detach()
        mproj = wproj + (wproj * masks[1] - wproj).detach()
        out = F.linear(F.gelu(F.linear(x, mfc, bfc)), mproj, bproj)
    loss = _loss(out, target)
    opt.zero_grad(set_to_none=True)
    (loss * LOSS_SCALE).backward()
    with torch.no_grad():
        for p in ps:
            p.grad.mul_(1.0 / LOSS_SCALE)
        for w, mask in ((wfc, masks[0]), (wproj, masks[1])):
            w.grad.add_(torch.where(mask, torch.zeros_like(w), w), alpha=ALPHA)      # sparse/decay.py:28-31
    opt.step()
    return loss.item()


def _check_step(step, fc, proj, x, w_fc0, w_proj0, h_pre, h, out, seed, offset):
    """One step's tensors against the dense masked model and the reproduced MVUE sample."""
    wm_fc = (w_fc0 * fc.weight.mask).half()
    wm_proj = (w_proj0 * proj.weight.mask).half()
    x2d = x.detach().reshape(-1, D).half()
    h2d = h.detach().reshape(-1, H)
    # forward products (bias in the epilogue)
    assert _rel(h_pre.reshape(-1, H), F.linear(x2d, wm_fc, fc.bias.detach().half())) < 1e-2, step
    assert _rel(out.reshape(-1, D), F.linear(h2d, wm_proj, proj.bias.detach().half())) < 1e-2, step
    # dX products and bias gradients
    d_out, d_hpre = out.grad.reshape(-1, D), h_pre.grad.reshape(-1, H)
    assert d_out.dtype == torch.float16 and d_hpre.dtype == torch.float16
    assert _rel(h.grad.reshape(-1, H), d_out.float() @ wm_proj.float()) < 1e-2, step
    assert _rel(x.grad.reshape(-1, D), d_hpre.float() @ wm_fc.float()) < 1e-2, step
    assert _rel(proj.bias.grad, d_out.float().sum(0)) < 1e-2, step
    assert _rel(fc.bias.grad, d_hpre.float().sum(0)) < 1e-2, step
    # dW against the reproduced sample: proj's backward runs first and takes `offset`, fc's the next slot
    dw_proj, est, u, packed = _mvue_dw(d_out, h2d, seed, offset)
    assert proj.weight.grad.dtype == torch.float32 and proj.weight.grad.shape == (D, H)
    assert _rel(proj.weight.grad, dw_proj) < 1e-3, step
    if step == 0:
        # once at full width: uniforms and estimate bit-equal to the CPU oracle
        assert packed.cpu().equal(oracle.mvue_uniforms(seed, offset, D, d_out.shape[0]))
        want = oracle.mvue24_dense(d_out.t().cpu(), u.cpu())
        assert est.cpu().view(torch.int16).equal(want.view(torch.int16))
        kept = est.reshape(D, -1, 4).ne(0).sum(-1)
        assert kept.le(2).all()
    del est, u, packed
    dw_fc, _, _, _ = _mvue_dw(d_hpre, x2d, seed, offset + 4)
    assert fc.weight.grad.shape == (H, D)
    assert _rel(fc.weight.grad, dw_fc) < 1e-3, step
    # and the estimate is one of dY^T x: same scale, error of the size MVUE24 over 12288 tokens leaves
    dense_dw = d_hpre.float().t() @ x2d.float()
    assert _rel(fc.weight.grad, dense_dw) < 0.5, step


def _train(cuda, fused_decay, with_checks):
    import sparse
    fc, proj, x, target = _make(cuda)
    x.requires_grad_(True)                       # so that c_fc's dX product runs, as inside a model
    params = list(fc.parameters()) + list(proj.parameters())
    if fused_decay:
        opt = sparse.MaskedDecayAdamW(params, lr=LR, alpha=ALPHA)
    else:
        opt = torch.optim.AdamW(params, lr=LR, fused=True)
    twin, twin_opt = _dense_masked_twin(fc, proj)
    twin_masks = [None, None]
    gen = torch.cuda.default_generators[cuda.index or 0]
    seed = gen.initial_seed()
    losses, twin_losses, weights_after_first = [], [], None
    prev_masks = None
    for step in range(STEPS):
        w_fc0, w_proj0 = fc.weight.detach().clone(), proj.weight.detach().clone()
        h_pre = fc(x)
        h = F.gelu(h_pre)
        out = proj(h)
        loss = _loss(out, target)
        checking = with_checks and step in CHECK_STEPS
        if checking:
            for t in (h_pre, h, out):
                t.retain_grad()
        opt.zero_grad(set_to_none=True)
        x.grad = None
        offset = gen.get_offset()
        (loss * LOSS_SCALE).backward()
        assert gen.get_offset() == offset + 8                    # two MVUE24 draws per step, nothing else
        # ---- masks
        masks = (fc.weight.mask, proj.weight.mask)
        if step % FREQ == 0:
            for mask, w0 in zip(masks, (w_fc0, w_proj0)):
                assert mask.cpu().equal(oracle.transposable_mask(w0.float().cpu())[1]), step
        else:
            assert masks[0].equal(prev_masks[0]) and masks[1].equal(prev_masks[1]), step
        prev_masks = tuple(m.clone() for m in masks)
        if checking:
            _check_step(step, fc, proj, x, w_fc0, w_proj0, h_pre, h, out, seed, offset)
        # ---- masked decay + optimizer (README.md:205-213)
        with torch.no_grad():
            for p in params:
                p.grad.mul_(1.0 / LOSS_SCALE)
            if not fused_decay:
                for p in params:
                    if hasattr(p, "mask") and p.mode == "sparse":
                        p.grad = p.grad.float()
                        sparse.masked_add_(p.grad.data, p.data, p.mask, alpha=ALPHA)
                        p.cnt = 0
        opt.step()
        assert fc.weight.cnt == 0 and proj.weight.cnt == 0
        losses.append(loss.item())
        if step == 0:
            weights_after_first = [p.detach().clone() for p in params]
        if with_checks:
            twin_losses.append(_twin_step(twin, twin_opt, twin_masks, x.detach(), target, step))
    assert fc.weight.counter == STEPS and proj.weight.counter == STEPS
    return losses, twin_losses, weights_after_first, [p.detach().clone() for p in params]


def test_config4_training_run_full_size(cuda):
    losses, twin_losses, first, final = _train(cuda, fused_decay=False, with_checks=True)
    t = torch.tensor(losses)
    assert torch.isfinite(t).all()
    dev = max(abs(a - b) / b for a, b in zip(losses, twin_losses))
    print(f"config 4: loss {losses[0]:.5f} -> {losses[-1]:.5f}; dense-masked {twin_losses[0]:.5f} -> {twin_losses[-1]:.5f}; "
          f"largest relative deviation {dev:.4f}")
    assert abs(losses[0] - twin_losses[0]) / twin_losses[0] < 2e-3          # same model before any update
    assert dev < LOSS_BAND, (dev, losses[::10], twin_losses[::10])
    assert losses[-1] < 0.8 * losses[0], losses[::10]

    # the same run with the decay folded into the optimizer: same samples, float32 rounding apart
    losses_f, _, first_f, final_f = _train(cuda, fused_decay=True, with_checks=False)
    for a, b in zip(first, first_f):
        assert torch.allclose(a, b, rtol=0, atol=2e-6), (a - b).abs().max()
    assert abs(losses_f[0] - losses[0]) <= 1e-6 * abs(losses[0])
    dev_f = max(abs(a - b) / b for a, b in zip(losses_f, losses))
    print(f"MaskedDecayAdamW run: largest relative loss deviation from the masked_add_ run {dev_f:.5f}")
    assert dev_f < LOSS_BAND


def test_mean_reduced_loss_on_the_layer_output(cuda):
    """A loss that expands a scalar gradient over the layer's output (out.mean()) must keep the
    gradient's values: dX, db and the reproduced dW sample all carry the 1/N factor.  Input without
    grad: only dW and db are formed."""
    import sparse
    torch.manual_seed(3)
    layer = sparse.SparseLinearTranspose(256, 512).to(cuda)
    x = torch.randn(4, 128, 256, device=cuda, requires_grad=True)
    gen = torch.cuda.default_generators[cuda.index or 0]
    offset = gen.get_offset()
    layer(x).mean().backward()
    n = 4 * 128 * 512
    wm = (layer.weight.detach() * layer.weight.mask).half()
    gy = torch.full((4 * 128, 512), 1.0 / n, device=cuda, dtype=torch.float16)
    assert _rel(x.grad.reshape(-1, 256), gy.float() @ wm.float()) < 1e-2
    assert _rel(layer.bias.grad, gy.float().sum(0)) < 1e-2
    dw, _, _, _ = _mvue_dw(gy, x.detach().reshape(-1, 256).half(), gen.initial_seed(), offset)
    assert _rel(layer.weight.grad, dw) < 1e-3
    # first layer of a model: the input needs no gradient
    layer.weight.grad = layer.bias.grad = None
    layer.weight.cnt = 0
    offset = gen.get_offset()
    layer(x.detach()).mean().backward()
    dw, _, _, _ = _mvue_dw(gy, x.detach().reshape(-1, 256).half(), gen.initial_seed(), offset)
    assert _rel(layer.weight.grad, dw) < 1e-3
    assert _rel(layer.bias.grad, gy.float().sum(0)) < 1e-2


def test_reference_switch_for_an_expanded_gradient(cuda):
    """sparse_linear_transpose.ones_for_expanded_grad = True reproduces README.md:186-187: a 3-d grad_output whose
    strides are all zero (a scaled out.sum() taken directly on the layer's output) is replaced by ones, so the
    scale is dropped; by default the gradient's values are used."""
    import sparse
    torch.manual_seed(4)
    layer = sparse.SparseLinearTranspose(256, 512).to(cuda)
    x = torch.randn(4, 128, 256, device=cuda, requires_grad=True)
    fn = sparse.sparse_linear_transpose
    assert fn.ones_for_expanded_grad is False
    ones = torch.ones(4 * 128, 512, device=cuda)
    for switch, factor in ((False, 3.0), (True, 1.0)):
        x.grad = layer.weight.grad = layer.bias.grad = None
        layer.weight.cnt = 0
        fn.ones_for_expanded_grad = switch
        try:
            (layer(x).sum() * 3.0).backward()
        finally:
            fn.ones_for_expanded_grad = False
        wm = (layer.weight.detach() * layer.weight.mask).half()
        assert _rel(x.grad.reshape(-1, 256), factor * (ones @ wm.float())) < 1e-2, switch
        assert _rel(layer.bias.grad, factor * ones.sum(0)) < 1e-2, switch
