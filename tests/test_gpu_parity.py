"""GPU parity: every HIP kernel, called through the Python API -> ctypes -> C ABI, against the CPU
oracle on the same seeded inputs.  Bit-exact for masks, metadata, compressed values and the
element-wise operators; stated tolerances for the matmul."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F16, BF16, F32, E4M3, E5M2 = torch.float16, torch.bfloat16, torch.float32, torch.float8_e4m3fn, torch.float8_e5m2
FLOAT8 = (E4M3, E5M2)


def bits(t):
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bool:
        return t
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def assert_same(got, want, what=""):
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert got.dtype == want.dtype, (what, got.dtype, want.dtype)
    g, w = bits(got), bits(want)
    if not g.equal(w):
        bad = (g != w).nonzero()
        raise AssertionError(f"{what}: {bad.shape[0]} of {g.numel()} elements differ, first at {bad[0].tolist()}: "
                             f"got {got.detach().cpu()[tuple(bad[0])]} want {want[tuple(bad[0])]}")


def randn(shape, dtype, seed, scale=1.0, ties=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * scale
    if ties:   # coarse grid: many equal magnitudes inside groups
        x = torch.round(x * 2) / 2
    return x.to(dtype)


def maybe_t(x, col_major):
    """A logical tensor equal to x, stored column-major when asked (like W.T of a row-major W)."""
    return x.t().contiguous().t() if col_major else x


# ------------------------------------------------------------------ prune + compress
@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("in_dtype", [F16, BF16, F32])
@pytest.mark.parametrize("out_dtype", [F16, BF16, E4M3, E5M2])
@pytest.mark.parametrize("shape", [(32, 128), (96, 320 + 64), (64, 1024)])
def test_magnitude_compress(cuda, shape, in_dtype, out_dtype, col_major):
    import sparse
    w = randn(shape, in_dtype, 11, ties=(shape[0] == 96))
    want_v, want_m = oracle.compress24(w, out_dtype=out_dtype)
    s = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), col_major), dtype=out_dtype)
    assert s.shape == w.shape and s.dtype == out_dtype
    assert_same(s.values(), want_v, "values")
    assert_same(s.indices(), want_m, "meta")
    assert_same(s.to_dense(), oracle.decompress24(want_v, want_m), "to_dense")


@pytest.mark.parametrize("out_dtype", [F16, E4M3])
@pytest.mark.parametrize("col_major", [False, True])
def test_canonical_and_panel_storage_agree(cuda, out_dtype, col_major):
    """The same tensor compressed into the canonical and into the panel layout: identical
    values()/indices()/to_dense() and identical products."""
    import sparse
    cls = sparse.SparseSemiStructuredTensor
    w = randn((96, 384), F16, 18)
    x = randn((40 if out_dtype == F16 else 48, 384), F16, 19).to(cuda)
    want_v, want_m = oracle.compress24(w, out_dtype=out_dtype)
    outs = []
    try:
        for panel in (True, False):
            cls._PANEL_LAYOUT = panel
            s = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), col_major), dtype=out_dtype)
            assert s._store_layout == (1 if panel else 0)
            assert_same(s.values(), want_v, f"values panel={panel}")
            assert_same(s.indices(), want_m, f"meta panel={panel}")
            assert_same(s.to_dense(), oracle.decompress24(want_v, want_m), f"to_dense panel={panel}")
            outs.append(torch.mm(x.to(out_dtype), s.t()))
            outs.append(torch.mm(s, x.to(out_dtype).t().contiguous()))
    finally:
        cls._PANEL_LAYOUT = True
    assert_same(outs[0], outs[2], "x.W^T panel vs canonical")
    assert_same(outs[1], outs[3], "W.x^T panel vs canonical")
    # round trip through the canonical constructor arguments
    s2 = cls(None, original_shape=s.shape, sparse_tensor_cutlass=s.values(), meta_tensor_cutlass=s.indices(), dtype=out_dtype)
    assert_same(torch.mm(x.to(out_dtype), s2.t()), outs[0], "rebuilt from canonical pieces")


def test_docstring_known_answer(cuda):
    import sparse
    a = torch.tensor([0.0, 0.0, 1.0, 1.0]).tile((128, 32)).half().to(cuda)
    s = sparse.to_sparse_semi_structured(a)
    assert s.values().eq(1).all() and s.values().shape == (128, 64)
    assert s.indices().eq(-4370).all() and s.indices().dtype == torch.int16
    assert s.indices_cutlass().eq(-4370).all()


def test_config1_compress_and_mm(cuda):
    """BASELINE config 1 (the reference's CPU-runnable case), on the GPU path."""
    import sparse
    g = torch.Generator().manual_seed(0)
    w = (0.02 * torch.randn(3072, 768, generator=g)).half()
    x = torch.randn(12288, 768, generator=g)
    want_v, want_m = oracle.compress24(w)
    s = sparse.to_sparse_semi_structured(w.to(cuda))
    assert_same(s.values(), want_v, "values")
    assert_same(s.indices(), want_m, "meta")
    mask = oracle.prune24_mask(w)
    ref = oracle.spmm_ref(x.half(), torch.where(mask, w, torch.zeros_like(w)))
    out = torch.mm(x.half().to(cuda), s.t()).float().cpu()
    rel = (out - ref).norm() / ref.norm()
    assert out.shape == (12288, 3072) and rel < 1e-2, rel


@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("mask_dtype", [torch.bool, F16, F32])
@pytest.mark.parametrize("in_dtype,out_dtype", [(F32, F16), (F16, F16), (BF16, BF16), (F32, E4M3)])
def test_mask_compress(cuda, in_dtype, out_dtype, mask_dtype, col_major):
    import sparse
    w = randn((64, 256), in_dtype, 12)
    _, mask = oracle.transposable_mask(w.float())
    g = torch.Generator().manual_seed(13)
    mask[:8] = torch.rand(8, 256, generator=g) < 0.5            # invalid groups follow the truth table
    mask = mask.to(mask_dtype)
    want_v, want_m = oracle.compress24(w, mask=mask, out_dtype=out_dtype)
    s = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), col_major), mask=maybe_t(mask.to(cuda), col_major), dtype=out_dtype)
    assert_same(s.values(), want_v, "values")
    assert_same(s.indices(), want_m, "meta")


@pytest.mark.parametrize("mask_dtype", [torch.bool, BF16, F32])
@pytest.mark.parametrize("in_dtype,out_dtype,shape", [
    (F32, F16, (64, 64)), (F32, F16, (192, 320)), (F16, F16, (128, 448)), (BF16, BF16, (320, 128)),
    (F32, E4M3, (128, 384)), (BF16, E5M2, (256, 128))])
def test_mask_compress_pair(cuda, in_dtype, out_dtype, mask_dtype, shape):
    """W and W^T compressed from one read: each result must carry the bytes of the separate
    conversion of w / w.T (oracle), for transposable masks and for invalid groups."""
    import sparse
    from sparse import _native as N
    w = randn(shape, in_dtype, 15)
    _, mask = oracle.transposable_mask(w.float())
    g = torch.Generator().manual_seed(16)
    mask[:8] = torch.rand(8, shape[1], generator=g) < 0.5        # groups with 0..4 kept elements, both directions
    mask = mask.to(mask_dtype)
    want_v, want_m = oracle.compress24(w, mask=mask, out_dtype=out_dtype)
    want_vt, want_mt = oracle.compress24(w.t().contiguous(), mask=mask.t().contiguous(), out_dtype=out_dtype)
    s, s_t = sparse.to_sparse_semi_structured_pair(w.to(cuda), mask.to(cuda), dtype=out_dtype)
    assert s.shape == shape and s_t.shape == shape[::-1]
    assert s._store_layout == N.COMPRESSED_PANEL and s_t._store_layout == N.COMPRESSED_PANEL
    assert_same(s.values(), want_v, "values")
    assert_same(s.indices(), want_m, "meta")
    assert_same(s_t.values(), want_vt, "values of the transpose")
    assert_same(s_t.indices(), want_mt, "meta of the transpose")
    # canonical output through the C entry point, with padded rows of the dense matrix and the mask
    m, k = shape
    wide = torch.zeros((m, k + 24), dtype=in_dtype, device=cuda)
    wide[:, 8:8 + k] = w.to(cuda)
    mk = mask.to(cuda)
    mk = mk.view(torch.uint8) if mk.dtype == torch.bool else mk
    mwide = torch.zeros((m, k + 16), dtype=mk.dtype, device=cuda)
    mwide[:, 16:] = mk
    wv, mv = wide[:, 8:8 + k], mwide[:, 16:]
    idt = torch.int32 if out_dtype in FLOAT8 else torch.int16
    cv = torch.empty((m, k // 2), dtype=out_dtype, device=cuda)
    cvt = torch.empty((k, m // 2), dtype=out_dtype, device=cuda)
    cm = torch.empty((m, k // 8), dtype=torch.uint8, device=cuda)
    cmt = torch.empty((k, m // 8), dtype=torch.uint8, device=cuda)
    N.check(N.lib().tf24_prune_compress_dual(
        wv.data_ptr(), N.dtype_code(in_dtype), wv.stride(0), m, k, mv.data_ptr(), N.dtype_code(mv.dtype), mv.stride(0),
        cv.data_ptr(), cm.data_ptr(), cvt.data_ptr(), cmt.data_ptr(), N.dtype_code(out_dtype), N.COMPRESSED_CANONICAL, N.stream_ptr()))
    assert_same(cv, want_v)
    assert_same(cm.view(idt), want_m)
    assert_same(cvt, want_vt)
    assert_same(cmt.view(idt), want_mt)


def test_mask_compress_pair_falls_back_and_rejects(cuda):
    """Shapes only one direction supports run the two separate conversions (and raise where those
    raise); the C entry point refuses them."""
    import sparse
    from sparse import _native as N
    w = randn((96, 128), F16, 17)                               # 96 rows: fine for w, not for w.T (needs % 64)
    mask = oracle.prune24_mask(w)
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured_pair(w.to(cuda), mask.to(cuda))
    wt = randn((128, 192), F16, 18).t()                         # column-major input: separate conversions, same bytes
    _, mask = oracle.transposable_mask(wt.contiguous().float())
    s, s_t = sparse.to_sparse_semi_structured_pair(wt.to(cuda), mask.to(cuda))
    want_v, want_m = oracle.compress24(wt.contiguous(), mask=mask)
    want_vt, want_mt = oracle.compress24(wt.t().contiguous(), mask=mask.t().contiguous())
    assert_same(s.values(), want_v)
    assert_same(s.indices(), want_m)
    assert_same(s_t.values(), want_vt)
    assert_same(s_t.indices(), want_mt)
    lib = N.lib()
    assert lib.tf24_prune_compress_dual_validate(N.F16, 128, 96, 128, N.U8, 128, N.F16, N.COMPRESSED_PANEL) != 0
    assert lib.tf24_prune_compress_dual_validate(N.F16, 128, 128, 128, N.U8, 128, N.E4M3, N.COMPRESSED_PANEL) == 0
    assert lib.tf24_prune_compress_dual_validate(N.F16, 64, 128, 64, N.U8, 64, N.E4M3, N.COMPRESSED_PANEL) != 0
    assert lib.tf24_prune_compress_dual_validate(N.F16, 120, 128, 128, N.U8, 128, N.F16, N.COMPRESSED_PANEL) != 0   # ld < k
    assert lib.tf24_prune_compress_dual_validate(N.U8, 128, 128, 128, N.U8, 128, N.F16, N.COMPRESSED_PANEL) != 0


@pytest.mark.parametrize("mode", ["magnitude", "mvue"])
@pytest.mark.parametrize("dtype,shape", [(F16, (96, 320)), (BF16, (64, 128)), (F32, (160, 192)), (F16, (3072, 1024))])
def test_compress_with_row_sums(cuda, dtype, shape, mode):
    """Compression of a column-major matrix that also returns its row sums (the bias gradient when the
    matrix is dY^T): compressed bytes identical to the plain conversion, sums within float32
    accumulation error of the exact sum and one rounding to the input dtype."""
    import sparse
    from sparse import _native as N
    m, k = shape
    t = randn((k, m), dtype, 19).t()                             # [m, k] column-major
    rand = torch.rand((k // 2, m), generator=torch.Generator().manual_seed(20)).t() if mode == "mvue" else None
    kw = dict(MVUE24=mode == "mvue", dtype=F16, rand=None if rand is None else rand.to(cuda))
    plain = sparse.to_sparse_semi_structured(t.to(cuda), **kw)
    fused, sums = sparse.to_sparse_semi_structured_with_row_sums(t.to(cuda), **kw)
    assert fused._store_layout == N.COMPRESSED_PANEL
    assert_same(fused.values(), plain.values().cpu(), "values")
    assert_same(fused.indices(), plain.indices().cpu(), "meta")
    want = t.double().sum(1)
    assert sums.shape == (m,) and sums.dtype == dtype
    eps = {F16: 2.0 ** -11, BF16: 2.0 ** -8, F32: 2.0 ** -24}[dtype]
    tol = eps * want.abs() + 2e-7 * (k ** 0.5) * t.double().abs().sum(1) / k ** 0.5 + 1e-30
    assert ((sums.double().cpu() - want).abs() <= tol + eps * want.abs().max()).all()
    # deterministic: the same bits every time
    again = sparse.to_sparse_semi_structured_with_row_sums(t.to(cuda), **kw)[1]
    assert again.equal(sums)


def test_compress_with_row_sums_other_layouts(cuda):
    """Row-major input runs the two operations separately; the C entry point refuses it."""
    import sparse
    from sparse import _native as N
    t = randn((64, 128), F16, 21)
    s, sums = sparse.to_sparse_semi_structured_with_row_sums(t.to(cuda))
    want_v, want_m = oracle.compress24(t)
    assert_same(s.values(), want_v)
    assert_same(s.indices(), want_m)
    assert torch.allclose(sums.float().cpu(), t.float().sum(1), rtol=2e-3, atol=2e-2)
    d = t.to(cuda)
    v = torch.empty(64 * 64, dtype=F16, device=cuda)
    mt = torch.empty(64 * 16, dtype=torch.uint8, device=cuda)
    out = torch.empty(64, dtype=F16, device=cuda)
    ws = torch.empty(64, dtype=torch.float32, device=cuda)
    call = lambda layout, ws_bytes: N.lib().tf24_prune_compress_rowsum(
        d.data_ptr(), N.F16, layout, 128, 64, 128, N.PRUNE_MAGNITUDE, None, N.U8, 0, None, 0, v.data_ptr(), N.F16, mt.data_ptr(),
        N.COMPRESSED_PANEL, out.data_ptr(), N.F16, ws.data_ptr(), ws_bytes, N.stream_ptr())
    assert call(N.ROW_MAJOR, 256) == -5
    assert N.lib().tf24_prune_compress_rowsum_workspace_bytes(64, 128) == 256
    assert N.lib().tf24_prune_compress_rowsum_workspace_bytes(3072, 12288) == 96 * 3072 * 4


def test_mask_layout_mismatch_is_copied(cuda):
    import sparse
    w = randn((64, 128), F16, 14)
    mask = oracle.prune24_mask(w)
    want_v, want_m = oracle.compress24(w, mask=mask)
    # column-major dense with a row-major mask and vice versa
    s1 = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), True), mask=mask.to(cuda))
    s2 = sparse.to_sparse_semi_structured(w.to(cuda), mask=maybe_t(mask.to(cuda), True))
    for s in (s1, s2):
        assert_same(s.values(), want_v)
        assert_same(s.indices(), want_m)


@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("in_dtype,out_dtype", [(BF16, F16), (F16, F16), (F32, BF16), (BF16, E4M3), (F32, E4M3), (F32, E5M2)])
@pytest.mark.parametrize("shape", [(32, 128), (128, 640)])
def test_mvue_compress(cuda, shape, in_dtype, out_dtype, col_major):
    import sparse
    w = randn(shape, in_dtype, 15)
    w[0, :8] = 0                                                 # degenerate all-zero groups
    u = torch.rand(shape, generator=torch.Generator().manual_seed(16))
    u[1, 1] = 0.0                                                # r1 == 0: a single element may be kept
    want_v, want_m, _ = oracle.mvue24(w, u, out_dtype=out_dtype)
    s = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), col_major), MVUE24=True, rand=maybe_t(u.to(cuda), col_major), dtype=out_dtype)
    assert_same(s.values(), want_v, "values")
    assert_same(s.indices(), want_m, "meta")


@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("out_dtype", [F16, E4M3])
def test_mvue_compress_packed_uniforms(cuda, out_dtype, col_major):
    """A [m, k/2] uniform tensor holds exactly the uniforms the estimator uses: group g of a row
    takes columns 2g and 2g+1.  Same result as the full-shape tensor carrying them in columns 4g, 4g+1."""
    import sparse
    shape = (64, 384)
    w = randn(shape, BF16, 25)
    up = torch.rand((shape[0], shape[1] // 2), generator=torch.Generator().manual_seed(26))
    full = torch.full(shape, 0.5)
    full[:, 0::4], full[:, 1::4] = up[:, 0::2], up[:, 1::2]
    want_v, want_m, _ = oracle.mvue24(w, full, out_dtype=out_dtype)
    s = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), col_major), MVUE24=True, rand=maybe_t(up.to(cuda), col_major), dtype=out_dtype)
    assert_same(s.values(), want_v, "values")
    assert_same(s.indices(), want_m, "meta")
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(w.to(cuda), MVUE24=True, rand=up[:, :-8].to(cuda), dtype=out_dtype)


@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("in_dtype,out_dtype,shape", [(BF16, F16, (64, 128)), (F16, F16, (96, 320)), (F32, BF16, (32, 64)), (F16, E4M3, (64, 256))])
def test_mvue_seeded_uniforms(cuda, in_dtype, out_dtype, shape, col_major):
    """Uniforms generated inside the kernel: tf24_mvue_uniforms writes the oracle's Philox stream, and
    compressing with rand=(seed, offset) gives the bytes of compressing with that tensor supplied."""
    import sparse
    from sparse import _native as N
    m, k = shape
    seed, offset = 0x1234567890abcdef, 40
    want_u = oracle.mvue_uniforms(seed, offset, m, k)
    got = torch.empty((m, k // 2), dtype=torch.float32, device=cuda)
    N.check(N.lib().tf24_mvue_uniforms(seed, offset, m, k, N.ROW_MAJOR, got.data_ptr(), k // 2, N.stream_ptr()))
    assert got.cpu().equal(want_u)
    got_t = torch.empty((k // 2, m), dtype=torch.float32, device=cuda)
    N.check(N.lib().tf24_mvue_uniforms(seed, offset, m, k, N.COL_MAJOR, got_t.data_ptr(), m, N.stream_ptr()))
    assert got_t.t().cpu().equal(want_u)
    w = randn(shape, in_dtype, 23)
    full = torch.zeros(shape)
    full[:, 0::4], full[:, 1::4] = want_u[:, 0::2], want_u[:, 1::2]
    want_v, want_m, _ = oracle.mvue24(w, full, out_dtype=out_dtype)
    wd = maybe_t(w.to(cuda), col_major)
    s = sparse.to_sparse_semi_structured(wd, MVUE24=True, dtype=out_dtype, rand=(seed, offset))
    assert_same(s.values(), want_v, "values")
    assert_same(s.indices(), want_m, "meta")
    if col_major and out_dtype not in FLOAT8:
        s2, sums = sparse.to_sparse_semi_structured_with_row_sums(wd, MVUE24=True, dtype=out_dtype, rand=(seed, offset))
        assert_same(s2.values(), want_v)
        assert_same(s2.indices(), want_m)


def test_mvue_default_sampling_follows_torch_seed(cuda):
    """Without `rand` the (seed, offset) pair comes from torch's generator: torch.manual_seed makes the
    sampling reproducible, successive calls draw different uniforms, two values are kept per group."""
    import sparse
    w = randn((64, 256), F16, 24).to(cuda)
    torch.manual_seed(77)
    a1 = sparse.to_sparse_semi_structured(w, MVUE24=True)
    a2 = sparse.to_sparse_semi_structured(w, MVUE24=True)
    torch.manual_seed(77)
    b1 = sparse.to_sparse_semi_structured(w.t().contiguous().t(), MVUE24=True)      # same matrix, column-major storage
    assert a1.indices().equal(b1.indices()) and a1.values().equal(b1.values())
    assert not a1.indices().equal(a2.indices())
    dense = a1.to_dense()
    assert ((dense != 0).view(64, 64, 4).sum(-1) <= 2).all()
    # unbiased: the mean over many draws approaches w
    acc = torch.zeros_like(w, dtype=torch.float32)
    for _ in range(200):
        acc += sparse.to_sparse_semi_structured(w, MVUE24=True).to_dense().float()
    err = (acc / 200 - w.float()).abs().mean() / w.float().abs().mean()
    assert err < 0.12, err


def _wide_range(shape, seed):
    """float32 values whose exponents span denormals to 2^60, with zeros, negative zeros and groups
    dominated by one element (sum - a_i rounds to zero): operands the in-range division must hand
    to the general one."""
    g = torch.Generator().manual_seed(seed)
    expo = torch.randint(-140, 61, shape, generator=g).float()
    w = torch.randn(shape, generator=g) * torch.exp2(expo)
    flat = w.view(-1, 4)
    flat[0::7, 1] = 0.0
    flat[3::7, 2] = -0.0
    flat[5::11] = torch.tensor([1.0e6, 1.0e-7, 0.0, -1.0e-7])
    flat[6::13] = torch.tensor([3.0e38, 1.0, -2.0e38, 1.0e-30])
    return w


@pytest.mark.parametrize("col_major", [False, True])
def test_mvue_wide_dynamic_range(cuda, col_major):
    import sparse
    w = _wide_range((64, 256), 18)
    u = torch.rand(w.shape, generator=torch.Generator().manual_seed(19))
    want = oracle.mvue24_dense(w, u)
    got = sparse.MVUE24_approx_triton(maybe_t(w.to(cuda), col_major), rand=maybe_t(u.to(cuda), col_major)).cpu()
    assert torch.equal(got.isnan(), want.isnan())
    ok = ~want.isnan()
    assert_same(torch.where(ok, got, torch.zeros(())), torch.where(ok, want, torch.zeros(())), "mvue dense, wide range")
    want_v, want_m, _ = oracle.mvue24(w, u, out_dtype=BF16)
    s = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), col_major), MVUE24=True, rand=maybe_t(u.to(cuda), col_major), dtype=BF16)
    assert_same(s.indices(), want_m, "meta")
    gv = s.values().cpu()
    assert torch.equal(gv.isnan(), want_v.isnan())
    okv = ~want_v.isnan()
    assert_same(torch.where(okv, gv, torch.zeros((), dtype=BF16)), torch.where(okv, want_v, torch.zeros((), dtype=BF16)), "values, wide range")


def test_mvue_default_rand_keeps_two(cuda):
    import sparse
    w = randn((64, 128), F16, 17).to(cuda)
    torch.manual_seed(0)
    s = sparse.to_sparse_semi_structured(w, MVUE24=True)
    dense = s.to_dense()
    assert (dense != 0).reshape(-1, 4).sum(-1).le(2).all()


def test_compress_errors(cuda):
    import sparse
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(torch.zeros(32, 64, dtype=F16))                       # not on the GPU
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(torch.zeros(2, 32, 64, dtype=F16, device=cuda))       # not 2-d
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(torch.zeros(32, 64, dtype=F16, device=cuda), dtype=torch.float64)
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(torch.zeros(48, 64, dtype=F16, device=cuda))
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(torch.zeros(32, 64, dtype=F16, device=cuda), dtype=E4M3)  # needs k % 128
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(torch.zeros(32, 64, dtype=F16, device=cuda), MVUE24=True,
                                         mask=torch.ones(32, 64, dtype=torch.bool, device=cuda))


# ------------------------------------------------------------------ transposable search
@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("use_abs", [True, False])
@pytest.mark.parametrize("dtype", [F16, BF16, F32])
@pytest.mark.parametrize("ties", [False, True])
def test_transposable(cuda, dtype, use_abs, col_major, ties):
    import sparse
    w = randn((96, 192), dtype, 21, ties=ties)
    if ties:
        w[:4, :8] = 0
        w[4:8, :4] = 1
    want_s, want_m = oracle.transposable_mask(w, use_abs=use_abs)
    got_s, got_m = sparse.TransposableSparse(abs=use_abs)(maybe_t(w.to(cuda), col_major))
    assert got_m.dtype == torch.bool
    assert_same(got_m, want_m, "mask")
    assert_same(got_s, want_s, "sparse")
    if ties or dtype != F32:
        _, brute, _ = oracle.transposable_mask_bruteforce(w, use_abs=use_abs)
        if ties:
            assert_same(got_m, brute, "mask vs 90-way brute force")


def test_transposable_errors(cuda):
    import sparse
    ts = sparse.TransposableSparse()
    for shape in [(33, 64), (32, 32)]:
        with pytest.raises(RuntimeError):
            ts(torch.zeros(shape, device=cuda))
    with pytest.raises(RuntimeError):
        ts(torch.zeros(32, 64, dtype=torch.float64, device=cuda))
    with pytest.raises(RuntimeError):
        ts(torch.zeros(2, 32, 64, device=cuda))


# ------------------------------------------------------------------ dense-shaped operators
@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_soft_threshold(cuda, dtype, col_major):
    import sparse
    w = randn((64, 256), dtype, 31, ties=(dtype == F16))
    want_s, want_m = oracle.soft_threshold24(w)
    got_s, got_m = sparse.soft_threshold24_triton(maybe_t(w.to(cuda), col_major))
    assert_same(got_s, want_s, "sparse")
    assert_same(got_m, want_m, "mask")
    assert got_s.stride() == maybe_t(w, col_major).stride()


@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_sparse24_and_mvue_dense(cuda, dtype, col_major):
    import sparse
    w = randn((64, 256), dtype, 32)
    want_s, want_m = oracle.sparse24_dense(w)
    got_s, got_m = sparse.sparse24_triton(maybe_t(w.to(cuda), col_major))
    assert_same(got_s, want_s, "sparse24")
    assert_same(got_m, want_m, "mask24")
    u = torch.rand(w.shape, generator=torch.Generator().manual_seed(33))
    got = sparse.MVUE24_approx_triton(maybe_t(w.to(cuda), col_major), rand=maybe_t(u.to(cuda), col_major))
    assert_same(got, oracle.mvue24_dense(w, u), "mvue dense")


# ------------------------------------------------------------------ masked decay
@pytest.mark.parametrize("gdt,pdt,mdt", [(F32, F32, torch.bool), (F32, BF16, torch.bool), (F32, F32, F32),
                                         (BF16, BF16, BF16), (F16, F32, torch.uint8)])
@pytest.mark.parametrize("n", [(64, 64), (7, 13), (1000003,)])
def test_masked_add(cuda, gdt, pdt, mdt, n):
    import sparse
    g = torch.Generator().manual_seed(41)
    grad = (1e-3 * torch.randn(n, generator=g)).to(gdt)
    p = torch.randn(n, generator=g).to(pdt)
    mask = (torch.rand(n, generator=g) < 0.5).to(mdt)
    want = oracle.masked_add(grad, p, mask, alpha=2e-4)
    gg = grad.to(cuda)
    assert sparse.masked_add_(gg, p.to(cuda), mask.to(cuda), alpha=2e-4) is None
    assert_same(gg, want)


def test_masked_add_reference_vector(cuda):
    import sparse
    grad = torch.tensor([1.0, 1.0, 1.0, 1.0], device=cuda)
    sparse.masked_add_(grad, torch.tensor([1.0, 2.0, 3.0, 4.0], device=cuda), torch.tensor([1.0, 0.0, 1.0, 0.0], device=cuda), alpha=0.03)
    assert torch.allclose(grad.cpu(), torch.tensor([1.0, 1.06, 1.0, 1.12]), atol=1e-7)


# ------------------------------------------------------------------ 2:4 matmul
def _small_ints(shape, seed, lo=-3, hi=4):
    return torch.randint(lo, hi, shape, generator=torch.Generator().manual_seed(seed)).float()


@pytest.mark.parametrize("dtype", [F16, BF16, E4M3, E5M2])
@pytest.mark.parametrize("dims", [(32, 128, 16), (64, 256, 40), (96, 384, 200), (160, 1024, 72)])
def test_spmm_exact_small_integers(cuda, dtype, dims):
    """Small-integer operands: every product and partial sum is exact in float32, so the
    result must EQUAL the dense masked product -- pins operand and index layout."""
    import sparse
    n, k, m = dims
    if dtype in FLOAT8 and m % 16:
        m += 8
    w = _small_ints((n, k), 51).to(dtype)
    x = _small_ints((m, k), 52).to(dtype)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(())))
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    out = torch.mm(x.to(cuda), s.t())                      # second operand sparse: x . W^T
    assert out.shape == (m, n)
    assert out.dtype == (torch.float32 if dtype in FLOAT8 else dtype)
    ref = ref.to(out.dtype).float()                        # the kernel rounds the exact sum once
    assert out.float().cpu().equal(ref)
    # first operand sparse: W . B with B [k, j] row-major (k strided) and as a transposed view
    b = x.t().contiguous()
    out2 = torch.mm(s, b.to(cuda))
    assert out2.shape == (n, m) and out2.float().cpu().equal(ref.t())
    out3 = torch.mm(s, x.to(cuda).t())
    assert out3.float().cpu().equal(ref.t())
    # second operand sparse with a column-major x
    out4 = torch.mm(maybe_t(x.to(cuda), True), s.t())
    assert out4.float().cpu().equal(ref)


@pytest.mark.parametrize("dtype,tol", [(F16, 1e-2), (BF16, 1e-2), (E4M3, 5e-2), (E5M2, 5e-2)])
def test_spmm_random_tolerance(cuda, dtype, tol):
    import sparse
    n, k, m = 256, 512, 328 if dtype not in FLOAT8 else 336
    w = randn((n, k), F32, 53, scale=0.02)
    x = randn((m, k), F32, 54)
    if dtype in FLOAT8:
        sw, sx = 448.0 / w.abs().max(), 448.0 / x.abs().max()
        wq, xq = (w * sw).to(dtype), (x * sx).to(dtype)
    else:
        sw = sx = 1.0
        wq, xq = w.to(dtype), x.to(dtype)
    mask = oracle.prune24_mask(wq.float())
    ref = oracle.spmm_ref(xq.float(), torch.where(mask, wq.float(), torch.zeros(())))
    s = sparse.to_sparse_semi_structured(wq.float().to(cuda), dtype=dtype)
    out = torch.mm(xq.to(cuda), s.t()).float().cpu()
    rel = (out - ref).norm() / ref.norm()
    assert rel < tol, rel


def test_spmm_bias_linear_padding(cuda):
    import sparse
    n, k, m = 64, 128, 21                                   # m is padded to 24 and sliced back
    w = _small_ints((n, k), 55).half()
    x = _small_ints((3, 7, k), 56).half()
    bias = _small_ints((n,), 57).half()
    mask = oracle.prune24_mask(w)
    wm = torch.where(mask, w, torch.zeros_like(w))
    s = sparse.to_sparse_semi_structured(w.to(cuda))
    ref = oracle.linear_ref(x, wm, bias)
    out = torch.nn.functional.linear(x.to(cuda), s, bias.to(cuda))
    assert out.shape == (3, 7, n) and out.float().cpu().equal(ref)
    out = torch.addmm(bias.to(cuda), x.reshape(m, k).to(cuda), s.t())
    assert out.float().cpu().equal(ref.reshape(m, n))
    with torch.inference_mode():
        out = torch.nn.functional.linear(x.to(cuda), s, bias.to(cuda))
    assert out.float().cpu().equal(ref)


def test_dispatch_rules(cuda):
    import sparse
    w = _small_ints((32, 64), 58).half().to(cuda)
    s = sparse.to_sparse_semi_structured(w)
    assert s.t().transposed and s.t().shape == (64, 32) and not s.t().t().transposed
    assert s.detach()._store_values.data_ptr() == s._store_values.data_ptr()
    x = torch.ones(8, 64, dtype=F16, device=cuda)
    with pytest.raises(NotImplementedError):
        torch.mm(x, s)                                     # second operand must be transposed
    with pytest.raises(NotImplementedError):
        torch.mm(s.t(), x.t())                             # first operand must not be
    with pytest.raises(NotImplementedError):
        s + 1


@pytest.mark.parametrize("dtype,k", [(F16, 256), (F16, 320), (BF16, 704), (E4M3, 512), (E4M3, 640)])
def test_spmm_chained_tiles_with_partial_edges(cuda, dtype, k):
    """More 256 x 256 tiles than compute units: one workgroup per compute unit chains its tiles (the next
    tile's first copies ride in the current tile's last two stages).  17 x 17 tiles with partial last
    row and column of tiles, from the shortest k the chained form takes (4 stages) up; exact on small
    integers, with and without bias, against the float32 product; 16-bit and 8-bit operands."""
    import sparse
    n, m = 4128, 4112
    odt = torch.bfloat16 if dtype in FLOAT8 else dtype
    w = _small_ints((n, k), 71, -2, 3).to(dtype)
    x = _small_ints((m, k), 72, -2, 3).to(dtype)
    bias = _small_ints((n,), 73).to(odt)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(())))
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    xg = x.to(cuda)
    out = sparse.sparse_semi_structured_linear(xg, s, out_dtype=odt)
    assert out.shape == (m, n) and out.float().cpu().equal(ref.to(odt).float())
    out = sparse.sparse_semi_structured_linear(xg, s, bias_opt=bias.to(cuda), out_dtype=odt)
    assert out.float().cpu().equal((ref + bias.float()).to(odt).float())
    # twice in a row on the same buffers: nothing left over from the first launch
    again = sparse.sparse_semi_structured_linear(xg, s, bias_opt=bias.to(cuda), out_dtype=odt)
    assert again.equal(out)


@pytest.mark.parametrize("dtype,k,act,scale", [(F16, 256, "relu", 0.5), (BF16, 320, "relu", 1.0), (E4M3, 512, "relu", 0.25),
                                               (F16, 320, "silu", 0.5), (BF16, 256, "gelu", 1.0), (E4M3, 640, "gelu", 0.125),
                                               (F16, 256, "gelu", 1.0), (E5M2, 512, "silu", 1.0)])
def test_spmm_chained_tiles_activation_and_scale(cuda, dtype, k, act, scale):
    """The chained-tile kernel's output passes with an activation (the bias of a wave's rows reaches them through
    LDS; zeros without a bias): 17 x 17
    tiles of 256 x 256 with partial edge tiles, more tiles than compute units.  Scale and bias act on exact
    float32 sums of small integers, so ReLU results are exact (one rounding of an exact value); SiLU and
    GELU are compared with torch's float32 functions of the same exact argument within 2e-3 + one unit in
    the last place of the 16-bit output (the kernel's exp / erf differ from torch's by a few float32 ulps)."""
    import sparse
    n, m = 4128, 4112
    odt = torch.bfloat16 if dtype in FLOAT8 else dtype
    w = _small_ints((n, k), 74, -2, 3).to(dtype)
    x = _small_ints((m, k), 75, -2, 3).to(dtype)
    bias = (_small_ints((n,), 76) * 0.5).to(odt)
    mask = oracle.prune24_mask(w.float())
    pre = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(()))) * scale + bias.float()
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    out = sparse.sparse_semi_structured_linear(x.to(cuda), s, bias_opt=bias.to(cuda), activation_opt=act, out_dtype=odt, scale=scale)
    assert out.shape == (m, n) and out.dtype == odt
    got = out.float().cpu()
    if act == "relu":
        assert got.equal(pre.clamp_min(0).to(odt).float())
    else:
        want = torch.nn.functional.silu(pre) if act == "silu" else torch.nn.functional.gelu(pre)
        ulp = 2.0 ** -8 if odt == torch.bfloat16 else 2.0 ** -11
        err = (got - want).abs()
        assert bool((err <= 2e-3 + (2e-3 + ulp) * want.abs()).all()), float(err.max())
    again = sparse.sparse_semi_structured_linear(x.to(cuda), s, bias_opt=bias.to(cuda), activation_opt=act, out_dtype=odt, scale=scale)
    assert again.equal(out)
    # the same activation without a bias, right behind a launch that had one
    nobias = sparse.sparse_semi_structured_linear(x.to(cuda), s, activation_opt=act, out_dtype=odt, scale=scale).float().cpu()
    pre0 = pre - bias.float()
    if act == "relu":
        assert nobias.equal(pre0.clamp_min(0).to(odt).float())
    else:
        want0 = torch.nn.functional.silu(pre0) if act == "silu" else torch.nn.functional.gelu(pre0)
        err0 = (nobias - want0).abs()
        assert bool((err0 <= 2e-3 + (2e-3 + ulp) * want0.abs()).all()), float(err0.max())


@pytest.mark.parametrize("dtype,k,act,n,m", [(F16, 1024, None, 4128, 4112), (BF16, 704, "relu", 4128, 4112),
                                              (E4M3, 1152, "gelu", 4128, 4112), (F16, 576, "silu", 4128, 4112),
                                              (F16, 768, None, 3072, 12288), (E5M2, 2048, None, 4384, 4352),
                                              (F16, 3072, "gelu", 4128, 4112), (BF16, 3136, None, 4128, 4112),
                                              (E4M3, 6144, "relu", 4128, 4112), (E5M2, 6272, "silu", 4384, 4352),
                                              (F16, 2112, "relu", 1760, 12272), (E4M3, 4224, None, 1792, 12288),
                                              (BF16, 2048, "gelu", 2784, 8176), (F16, 2112, None, 800, 12272),
                                              (BF16, 3072, None, 768, 12288), (F16, 2112, None, 4128, 8176),
                                              (E4M3, 4224, "relu", 4128, 8176), (BF16, 2048, None, 4384, 8192)])
def test_spmm_partial_last_round_long_k(cuda, dtype, k, act, n, m):
    """More tiles than compute units with a partial last round and 8 to 49 stages of k (the chained-tile kernel
    with one to three full rounds before the leftover tiles; from 32 stages on in its 4-wave form -- the last three
    shapes but two on 256 x 192 tiles, which need no more rounds there than 256 x 256 ones: 7 x 64 and 11 x 43 tiles with partial edges;
    the next two on 4 x 64 and 3 x 64 such tiles in a single round, where 256 x 256 ones would leave compute units idle;
    the last three with two full rounds of 256 x 256 tiles and one or two more tile rows, which a second launch computes on
    256 x 128 tiles -- in the first two of them the partial row of tiles).  Sums of small integers are exact in float32, so the
    results must equal the oracle's bit for bit, with bias, scale and activation behind the sum, for k contiguous
    and k strided dense operands, on a second call, and through the C ABI without a workspace."""
    import sparse
    odt = torch.bfloat16 if dtype in FLOAT8 else dtype
    w = _small_ints((n, k), 84, -2, 3).to(dtype)
    x = _small_ints((m, k), 85, -2, 3).to(dtype)
    bias = (_small_ints((n,), 86) * 0.5).to(odt)
    mask = oracle.prune24_mask(w.float())
    pre = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(()))) * 0.5 + bias.float()
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    xg = x.to(cuda)
    run = lambda xin: sparse.sparse_semi_structured_linear(xin, s, bias_opt=bias.to(cuda), activation_opt=act, out_dtype=odt, scale=0.5)
    out = run(xg)
    got = out.float().cpu()
    if act in (None, "relu"):
        want = pre if act is None else pre.clamp_min(0)
        assert got.equal(want.to(odt).float())
    else:
        want = torch.nn.functional.silu(pre) if act == "silu" else torch.nn.functional.gelu(pre)
        ulp = 2.0 ** -8 if odt == torch.bfloat16 else 2.0 ** -11
        err = (got - want).abs()
        assert bool((err <= 2e-3 + (2e-3 + ulp) * want.abs()).all()), float(err.max())
    assert run(xg).equal(out)
    if dtype not in FLOAT8:
        assert run(maybe_t(xg, True)).equal(out)                # k strided dense operand
    y = torch.empty((m, n), dtype=odt, device=cuda)
    N = sparse._native
    N.check(N.lib().tf24_spmm(s._store_values.data_ptr(), s._store_meta.data_ptr(), s._store_layout, N.operand_code(s._store_values.dtype), n, k,
                              xg.data_ptr(), N.ROW_MAJOR, k, m, y.data_ptr(), N.operand_code(odt), N.COL_MAJOR, n,
                              bias.to(cuda).data_ptr(), 0.5, {None: N.ACT_NONE, "relu": N.ACT_RELU, "silu": N.ACT_SILU, "gelu": N.ACT_GELU}[act],
                              None, 0, N.stream_ptr()))
    assert y.equal(out)


@pytest.mark.parametrize("dtype", [F16, BF16, E4M3, E5M2])
def test_spmm_tiled_all_operand_positions(cuda, dtype):
    """Shapes large enough for the tiled kernel, with partial tiles: both operand positions, both
    layouts of the dense operand, bias, and the i-major / j-major LDS-staged epilogues."""
    import sparse
    n, k, m = 352, 640, 296 if dtype not in FLOAT8 else 304
    odt = torch.float32 if dtype in FLOAT8 else dtype           # 8-bit operands return float32
    w = _small_ints((n, k), 61).to(dtype)
    x = _small_ints((m, k), 62).to(dtype)
    bias = _small_ints((n,), 63).to(odt)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(())))
    ref_b = (ref + bias.float()).to(odt).float()
    ref = ref.to(odt).float()
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    xg = x.to(cuda)
    assert torch.mm(xg, s.t()).float().cpu().equal(ref)                          # k contiguous, j-major store
    assert torch.mm(maybe_t(xg, True), s.t()).float().cpu().equal(ref)           # k strided dense operand
    assert torch.mm(s, xg.t()).float().cpu().equal(ref.t())                      # sparse first, k contiguous view
    assert torch.mm(s, xg.t().contiguous()).float().cpu().equal(ref.t())         # sparse first, k strided
    assert torch.addmm(bias.to(cuda), xg, s.t()).float().cpu().equal(ref_b)
    out = sparse.sparse_semi_structured_linear(xg, s, bias=bias.to(cuda), activation="relu")
    assert out.float().cpu().equal(ref_b.clamp_min(0))
    # canonical values + metadata through the functional entry point: repacked once, same kernel
    out = sparse.sparse_semi_structured_linear(xg, s.values(), s.indices(), bias=bias.to(cuda))
    assert out.float().cpu().equal(ref_b)


@pytest.mark.parametrize("dims", [(256, 4096, 256), (96, 2048, 520), (352, 12288 // 4, 200)])
def test_spmm_split_k_is_exact_and_deterministic(cuda, dims):
    """k-heavy shapes whose tiles cannot fill the GPU take the split-K path (float32 partial tiles in a
    workspace + reduction launch); small-integer operands keep every partial sum exact."""
    import sparse
    from sparse import _native as N
    n, k, m = dims
    assert N.lib().tf24_spmm_workspace_bytes(N.F16, n, k, m) > 0
    w = _small_ints((n, k), 71, -2, 3).half()
    x = _small_ints((m, k), 72, -2, 3).half()
    bias = _small_ints((n,), 73).half()
    mask = oracle.prune24_mask(w)
    ref = oracle.spmm_ref(x, torch.where(mask, w, torch.zeros_like(w)))
    s = sparse.to_sparse_semi_structured(w.to(cuda))
    out = torch.mm(x.to(cuda), s.t())
    assert out.float().cpu().equal(ref.half().float())
    assert torch.mm(x.to(cuda), s.t()).equal(out)                                  # bit-reproducible
    assert torch.mm(s, x.to(cuda).t().contiguous()).float().cpu().equal(ref.t().half().float())
    outb = torch.addmm(bias.to(cuda), x.to(cuda), s.t())
    assert outb.float().cpu().equal((ref + bias.float()).half().float())


@pytest.mark.parametrize("dtype", [F16, BF16, torch.uint8])
@pytest.mark.parametrize("shape", [(64, 64), (200, 136), (1024, 768), (48, 4096)])
def test_transpose_copy(cuda, dtype, shape):
    from sparse import _native as N
    rows, cols = shape
    if dtype == torch.uint8:
        rows, cols = (rows + 15) // 16 * 16, (cols + 15) // 16 * 16
        t = torch.randint(0, 255, (rows, cols), dtype=torch.uint8, generator=torch.Generator().manual_seed(81))
    else:
        t = randn((rows, cols), dtype, 81)
    out = N.transposed_copy(t.to(cuda))
    assert out.shape == (cols, rows) and out.is_contiguous()
    assert_same(out, t.t().contiguous())


@pytest.mark.parametrize("dtype", [F16, E4M3, torch.int8])
def test_panel_form_is_the_documented_one(cuda, dtype):
    """The panel form as the C header states it, spelled out with torch views of the canonical tensors:
    values [k/KP][m][64 bytes] (KP = 128 / sizeof(value) dense columns), metadata [k/32][m][4 bytes]."""
    import sparse
    from sparse import _native as N
    m, k = 96, 640
    if dtype == torch.int8:
        w = torch.randint(-100, 101, (m, k), generator=torch.Generator().manual_seed(93)).to(torch.int8)
    else:
        w = randn((m, k), F32, 92)
    s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype)
    assert s._store_layout == N.COMPRESSED_PANEL
    want_v, want_m = oracle.compress24(w, out_dtype=dtype)
    kp = 128 // want_v.element_size()
    v_bytes = want_v.contiguous().view(torch.uint8).reshape(m, k // kp, 64).permute(1, 0, 2).contiguous()
    m_bytes = want_m.contiguous().view(torch.uint8).reshape(m, k // 32, 4).permute(1, 0, 2).contiguous()
    assert s._store_values.contiguous().view(torch.uint8).cpu().reshape(k // kp, m, 64).equal(v_bytes)
    assert s._store_meta.contiguous().view(torch.uint8).cpu().reshape(k // 32, m, 4).equal(m_bytes)


@pytest.mark.parametrize("dtype", [F16, E4M3])
def test_repack_between_canonical_and_panel(cuda, dtype):
    """tf24_repack on canonical values/metadata must give the bytes the compress kernel writes in
    panel form, and back."""
    import sparse
    from sparse import _native as N
    m, k = 96, 640
    w = randn((m, k), F32, 91)
    s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype)
    assert s._store_layout == N.COMPRESSED_PANEL
    pv, pm = s._store_values.contiguous(), s._store_meta.contiguous()
    cv, cm = s.values().contiguous(), s.indices().contiguous()
    want_v, want_m = oracle.compress24(w, out_dtype=dtype)
    assert cv.cpu().view(torch.uint8).equal(want_v.view(torch.uint8)) and cm.cpu().equal(want_m)
    ov, om = torch.empty_like(pv), torch.empty_like(pm)
    N.check(N.lib().tf24_repack(cv.data_ptr(), cm.data_ptr(), N.dtype_code(dtype), m, k, N.COMPRESSED_CANONICAL,
                                ov.data_ptr(), om.data_ptr(), N.stream_ptr()))
    assert ov.view(torch.uint8).equal(pv.view(torch.uint8)) and om.view(torch.uint8).equal(pm.view(torch.uint8))
    bv, bm = torch.empty_like(cv), torch.empty_like(cm)
    N.check(N.lib().tf24_repack(pv.data_ptr(), pm.data_ptr(), N.dtype_code(dtype), m, k, N.COMPRESSED_PANEL,
                                bv.data_ptr(), bm.data_ptr(), N.stream_ptr()))
    assert bv.view(torch.uint8).equal(cv.view(torch.uint8)) and bm.view(torch.uint8).equal(cm.view(torch.uint8))
    with pytest.raises(RuntimeError):
        N.check(N.lib().tf24_repack(cv.data_ptr(), cm.data_ptr(), N.dtype_code(dtype), m, k + 8, N.COMPRESSED_CANONICAL,
                                    ov.data_ptr(), om.data_ptr(), N.stream_ptr()))


@pytest.mark.parametrize("dtype,k", [(F16, 64), (F16, 128), (F16, 192), (F16, 256), (BF16, 320), (E4M3, 128), (E4M3, 256), (E5M2, 384)])
def test_spmm_tiled_short_k(cuda, dtype, k):
    """One to five pipeline stages: prologue, steady state and drain of the tiled kernel's stage ring
    each with fewer stages than the ring holds."""
    import sparse
    n, m = 128, 144
    w = _small_ints((n, k), 93).to(dtype)
    x = _small_ints((m, k), 94).to(dtype)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(())))
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    out = torch.mm(x.to(cuda), s.t())
    assert out.float().cpu().equal(ref.to(out.dtype).float())
    out = torch.mm(s, x.to(cuda).t())
    assert out.float().cpu().equal(ref.t().to(out.dtype).float())
    out = torch.mm(s, x.to(cuda).t().contiguous())                                 # k strided: transposing fragment reads
    assert out.float().cpu().equal(ref.t().to(out.dtype).float())


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_spmm_tiled_k_strided_padded_rows(cuda, dtype):
    """`S @ dense` with the dense operand a column slice of a wider row-major matrix: k is the strided
    dimension, rows are longer than the columns used, and the last column tile is partial."""
    import sparse
    n, k, j, ld = 320, 448, 520, 776
    w = _small_ints((n, k), 95).to(dtype)
    wide = _small_ints((k, ld), 96).to(dtype)
    x = wide[:, 8:8 + j]                                                            # [k, j], row pitch ld, 16-byte aligned start
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.t().float(), torch.where(mask, w.float(), torch.zeros(()))).t()   # [n, j]
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    xg = wide.to(cuda)[:, 8:8 + j]
    assert not xg.is_contiguous()
    out = torch.mm(s, xg)
    assert out.float().cpu().equal(ref.to(dtype).float())


# ------------------------------------------------------------------ int8 values and the integer product
def _int8(shape, seed, lo=-128, hi=128):
    return torch.randint(lo, hi, shape, generator=torch.Generator().manual_seed(seed), dtype=torch.int64).to(torch.int8)


@pytest.mark.parametrize("col_major", [False, True])
@pytest.mark.parametrize("use_mask", [False, True])
def test_int8_compress(cuda, col_major, use_mask):
    """int8 dense -> int8 values + int32 metadata (semi_structured.py:24-30, 323-331): magnitude rule
    on |x| with -128 the largest magnitude, ties to the larger index; masks as bytes or floats."""
    import sparse
    w = _int8((96, 384), 101)
    w[:, :8] = torch.tensor([-128, 127, -127, 128 - 256, 5, -5, 5, -5], dtype=torch.int8)   # extremes and ties
    mask = None
    if use_mask:
        _, mask = oracle.transposable_mask(w.float())
        mask[:4] = torch.rand(4, 384, generator=torch.Generator().manual_seed(102)) < 0.5
    want_v, want_m = oracle.compress24(w, mask=mask, out_dtype=torch.int8)
    assert want_v.dtype == torch.int8 and want_m.dtype == torch.int32
    for mk in ([None] if mask is None else [mask, mask.float()]):
        s = sparse.to_sparse_semi_structured(maybe_t(w.to(cuda), col_major),
                                             mask=None if mk is None else maybe_t(mk.to(cuda), col_major), dtype=torch.int8)
        assert s.dtype == torch.int8
        assert_same(s.values(), want_v, "values")
        assert_same(s.indices(), want_m, "meta")
        assert_same(s.to_dense(), oracle.decompress24(want_v, want_m), "to_dense")
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(w.to(cuda), dtype=torch.float16)          # int8 tensors give int8 values only
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(w.to(cuda).half(), dtype=torch.int8)
    with pytest.raises(RuntimeError):
        sparse.to_sparse_semi_structured(w.to(cuda), dtype=torch.int8, MVUE24=True)


def test_int8_compress_pair(cuda):
    import sparse
    w = _int8((256, 128), 103)
    _, mask = oracle.transposable_mask(w.float())
    want_v, want_m = oracle.compress24(w, mask=mask, out_dtype=torch.int8)
    want_vt, want_mt = oracle.compress24(w.t().contiguous(), mask=mask.t().contiguous(), out_dtype=torch.int8)
    s, s_t = sparse.to_sparse_semi_structured_pair(w.to(cuda), mask.to(cuda), dtype=torch.int8)
    assert_same(s.values(), want_v)
    assert_same(s.indices(), want_m)
    assert_same(s_t.values(), want_vt)
    assert_same(s_t.indices(), want_mt)


@pytest.mark.parametrize("dims", [(32, 128, 16), (64, 256, 40), (352, 640, 304), (256, 4096, 256), (96, 2048, 528)])
def test_int8_spmm_is_exact(cuda, dims):
    """int8 x int8 -> int32 (.cu:594-637) against an int64 product: general kernel, tiled kernel with
    partial tiles, split-K; both operand positions and dense layouts; int32 bias and ReLU."""
    import sparse
    n, k, m = dims
    w, x = _int8((n, k), 111), _int8((m, k), 112)
    bias = torch.randint(-100000, 100000, (n,), generator=torch.Generator().manual_seed(113), dtype=torch.int64).int()
    mask = oracle.prune24_mask(w.float())
    wm = torch.where(mask, w, torch.zeros_like(w))
    ref = oracle.spmm_ref_int(x, wm)
    s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=torch.int8)
    xg = x.to(cuda)
    out = torch.mm(xg, s.t())
    assert out.dtype == torch.int32 and out.cpu().equal(ref)
    assert torch.mm(maybe_t(xg, True), s.t()).cpu().equal(ref)                   # k strided dense operand
    assert torch.mm(s, xg.t()).cpu().equal(ref.t())                              # sparse first
    assert torch.mm(s, xg.t().contiguous()).cpu().equal(ref.t())
    assert torch.addmm(bias.to(cuda), xg, s.t()).cpu().equal(oracle.spmm_ref_int(x, wm, bias))
    out = sparse.sparse_semi_structured_linear(xg, s, bias=bias.to(cuda), activation="relu")
    assert out.cpu().equal(oracle.spmm_ref_int(x, wm, bias, relu=True))
    out = sparse.sparse_semi_structured_linear(xg, s.values(), s.indices())      # canonical pieces
    assert out.cpu().equal(ref)
    with pytest.raises(RuntimeError):
        sparse.sparse_semi_structured_linear(xg, s, activation="silu")           # .cu:610-612: none and ReLU only
    with pytest.raises(RuntimeError):
        torch.mm(xg.half(), s.t())                                               # operand dtypes must match


def test_int8_spmm_extreme_values(cuda):
    """All operands -128: every product is +16384, the sum over k = 2048 kept pairs stays in int32."""
    import sparse
    n, k, m = 64, 4096, 64
    w = torch.full((n, k), -128, dtype=torch.int8)
    x = torch.full((m, k), -128, dtype=torch.int8)
    s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=torch.int8)
    out = torch.mm(x.to(cuda), s.t())
    assert out.cpu().equal(torch.full((m, n), 16384 * (k // 2), dtype=torch.int32))


@pytest.mark.parametrize("dtype,m", [(F16, 8), (BF16, 8), (F16, 24), (BF16, 40), (E4M3, 16), (torch.int8, 16),
                                     (F16, 72), (BF16, 128), (E4M3, 80), (torch.int8, 128)])
@pytest.mark.parametrize("k", [512, 4096])
def test_spmm_narrow_dense_operand(cuda, dtype, m, k):
    """A handful of dense columns against a tall sparse operand: 8 columns take the one-pass kernel,
    up to 64 and up to 128 the tiled kernel on 256 x 64 and 256 x 128 tiles (with k pieces, whose
    partial tiles only cover the live 32-column slabs); every operand position and layout."""
    import sparse
    n = 320
    if dtype == torch.int8:
        w, x = _int8((n, k), 121, -3, 4), _int8((m, k), 122, -3, 4)
        ref = oracle.spmm_ref_int(x, torch.where(oracle.prune24_mask(w.float()), w, torch.zeros_like(w)))
        s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype)
    else:
        w, x = _small_ints((n, k), 121, -2, 3).to(dtype), _small_ints((m, k), 122, -2, 3).to(dtype)
        mask = oracle.prune24_mask(w.float())
        ref = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(())))
        s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    xg = x.to(cuda)
    same = lambda out, want: out.cpu().to(torch.float64).equal(want.to(out.dtype).to(torch.float64))
    assert same(torch.mm(xg, s.t()), ref)
    assert same(torch.mm(maybe_t(xg, True), s.t()), ref)
    assert same(torch.mm(s, xg.t()), ref.t())
    assert same(torch.mm(s, xg.t().contiguous()), ref.t())


@pytest.mark.parametrize("dtype", [F16, E4M3, torch.int8])
@pytest.mark.parametrize("n,k", [(320, 1024), (8192, 1408 * 2)])
def test_spmm_16_columns_without_workspace(cuda, dtype, n, k):
    """Through the C ABI with no workspace the tiled kernel cannot cut k into pieces, and 16 dense
    columns take the one-pass kernel (four waves that split k at 320 rows, the LDS-shared form at 8192)."""
    import sparse
    from sparse import _native as N
    m = 16
    if dtype == torch.int8:
        w, x = _int8((n, k), 141, -3, 4), _int8((m, k), 142, -3, 4)
        ref = oracle.spmm_ref_int(x, torch.where(oracle.prune24_mask(w.float()), w, torch.zeros_like(w)))
        s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype)
        out_dtype, out_code = torch.int32, N.I32
    else:
        w, x = _small_ints((n, k), 141, -2, 3).to(dtype), _small_ints((m, k), 142, -2, 3).to(dtype)
        ref = oracle.spmm_ref(x.float(), torch.where(oracle.prune24_mask(w.float()), w.float(), torch.zeros(())))
        s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
        out_dtype, out_code = torch.float32, N.F32
    xg = x.to(cuda)
    out = torch.empty(m, n, dtype=out_dtype, device=cuda)
    N.check(N.lib().tf24_spmm(s._store_values.data_ptr(), s._store_meta.data_ptr(), N.COMPRESSED_PANEL, N.operand_code(dtype), n, k,
                              xg.data_ptr(), N.ROW_MAJOR, k, m, out.data_ptr(), out_code, N.COL_MAJOR, n, None, 1.0, 0,
                              None, 0, N.stream_ptr()))
    torch.cuda.synchronize()
    assert out.cpu().to(torch.float64).equal(ref.to(torch.float64))


@pytest.mark.parametrize("panels", [1, 17, 22])
@pytest.mark.parametrize("n", [8192, 10272])
@pytest.mark.parametrize("dtype", [F16, E4M3])
def test_spmm_narrow_one_wave_per_block(cuda, dtype, n, panels):
    """Many sparse rows and few dense columns: the one-pass kernel whose waves own one 16-row block each
    and share the dense operand through LDS (two blocks per workgroup at 8192 rows, four at 10272, where
    the last workgroup has two idle waves and 16 columns also take this kernel; fewer rows split k over
    four waves: test_spmm_narrow_dense_operand); k not a multiple of the 16-panel chunks."""
    import sparse
    k, m = panels * (64 if dtype == F16 else 128), 16      # 1 panel, one chunk + 1, 22 panels
    w, x = _small_ints((n, k), 131, -2, 3).to(dtype), _small_ints((m, k), 132, -2, 3).to(dtype)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(())))
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    bias = _small_ints((n,), 133).to(torch.float32 if dtype == E4M3 else dtype)
    out = torch.mm(x.to(cuda), s.t())
    assert out.float().cpu().equal(ref.to(out.dtype).float())
    out = torch.mm(s, x.to(cuda).t())
    assert out.float().cpu().equal(ref.t().to(out.dtype).float())
    out = sparse.sparse_semi_structured_linear(x.to(cuda)[:8], s, bias=bias.to(cuda), activation="relu")
    want = (ref[:8] + bias.float()).clamp_min(0)
    assert out.float().cpu().equal(want.to(out.dtype).float())


def test_narrowing_edge_values(cuda):
    """Float32 -> e4m3 / e5m2 / bf16 / f16 on the device (hardware conversions where gfx950 has them) against
    torch's casts, byte for byte, on the values where narrowing rules differ between implementations:
    the largest finite value and the first one past it (e4m3: 448, ties at 464, NaN from 480 on -- not
    saturation), e5m2's 57344 / 61440 and overflow to infinity, signed infinities and NaNs, signed zeros,
    the subnormal boundaries and halfway cases of each type."""
    import sparse
    edge = [448.0, 449.0, 456.0, 463.99, 464.0, 464.01, 472.0, 479.9, 480.0, 512.0, 1e6, 57344.0, 59000.0, 61439.0, 61440.0, 61441.0,
            65503.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e30, float("inf"), float("nan"), 0.0,
            2.0 ** -6, 2.0 ** -7, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -10 * 1.0001, 2.0 ** -11, 2.0 ** -14, 2.0 ** -16,
            2.0 ** -17, 1.5 * 2.0 ** -17, 2.0 ** -18, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 2.0 ** -126, 2.0 ** -133, 2.0 ** -149,
            1.0, 1.0625, 1.09375, 1.125, 1.1875, 3.3895e38, 3.4e38, 240.0, 248.0, 0.0146484375, 0.015625]
    vals = torch.tensor(edge + [-v for v in edge], dtype=torch.float32)
    vals = torch.cat([vals, torch.tensor([0x7fa00001, 0xffc00123 - (1 << 32)], dtype=torch.int32).view(torch.float32)])   # NaNs with payloads
    n = vals.numel()
    k = 128
    rows = (n + 1) // 2 * 4 // k + 1
    rows = (rows + 31) // 32 * 32
    # every value sits at position 0 or 1 of a group whose mask keeps exactly those two positions
    dense = torch.zeros(rows * k, dtype=torch.float32)
    idx = torch.arange(n)
    dense[(idx // 2) * 4 + idx % 2] = vals
    dense = dense.view(rows, k)
    mask = torch.zeros(rows, k, dtype=torch.bool)
    mask.view(-1, 4)[:, :2] = True
    for odt in (E4M3, E5M2, BF16, F16):
        s = sparse.to_sparse_semi_structured(dense.to(cuda), mask=mask.to(cuda), dtype=odt)
        got = s.values().cpu().reshape(-1)[:n]
        want = vals.to(odt)
        gb, wb = got.view(torch.uint8 if odt in FLOAT8 else torch.int16), want.view(torch.uint8 if odt in FLOAT8 else torch.int16)
        nan = vals != vals
        assert gb[~nan].equal(wb[~nan]), (odt, vals[~nan][gb[~nan] != wb[~nan]])
        assert bool((got[nan].float() != got[nan].float()).all()), odt          # NaN stays NaN (payloads are not compared for 16-bit types)
        if odt in FLOAT8:
            assert gb[nan].equal(wb[nan]), odt                                   # one NaN byte per sign, as torch's


@pytest.mark.parametrize("dtype,k,act", [(E4M3, 512, None), (E4M3, 4224, "relu"), (E5M2, 640, "silu"), (F16, 320, "relu"),
                                         (BF16, 2112, None), (torch.int8, 512, None), (torch.int8, 4224, "relu")])
def test_spmm_chained_tiles_32bit_output(cuda, dtype, k, act):
    """More tiles than compute units with a 32-bit output -- float32 from 8-bit operands and int32 from int8, the
    output types the reference gives them (.cu:729, 772; .cu:594-637), float32 from 16-bit ones -- on the chained-tile
    kernel (4 to 5 stages: 8 waves; 33 stages: 4 waves) with its staged 32-bit output pass: 17 x 17 tiles with partial
    edges, bias, activation, against the oracle on exact data, and a second call."""
    import sparse
    n, m = 4128, 4112
    if dtype == torch.int8:
        w, x = _int8((n, k), 121, -20, 21), _int8((m, k), 122, -20, 21)
        bias = torch.randint(-1000, 1000, (n,), generator=torch.Generator().manual_seed(123), dtype=torch.int64).int()
        mask = oracle.prune24_mask(w.float())
        want = oracle.spmm_ref_int(x, torch.where(mask, w, torch.zeros_like(w))) + bias
        if act == "relu":
            want = want.clamp_min(0)
        s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=torch.int8)
        out = sparse.sparse_semi_structured_linear(x.to(cuda), s, bias_opt=bias.to(cuda), activation_opt=act)
        assert out.dtype == torch.int32 and out.shape == (m, n)
        assert out.cpu().equal(want.int())
        assert sparse.sparse_semi_structured_linear(x.to(cuda), s, bias_opt=bias.to(cuda), activation_opt=act).equal(out)
        return
    w = _small_ints((n, k), 124, -2, 3).to(dtype)
    x = _small_ints((m, k), 125, -2, 3).to(dtype)
    bias = _small_ints((n,), 126) * 0.5
    mask = oracle.prune24_mask(w.float())
    pre = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(()))) * 0.25 + bias
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    run = lambda: sparse.sparse_semi_structured_linear(x.to(cuda), s, bias_opt=bias.to(cuda), activation_opt=act, out_dtype=torch.float32, scale=0.25)
    out = run()
    assert out.dtype == torch.float32 and out.shape == (m, n)
    got = out.cpu()
    if act in (None, "relu"):
        assert got.equal(pre if act is None else pre.clamp_min(0))
    else:
        want = torch.nn.functional.silu(pre)
        assert bool(((got - want).abs() <= 2e-6 + 2e-6 * want.abs()).all())
    assert run().equal(out)
