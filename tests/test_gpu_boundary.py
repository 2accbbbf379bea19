"""The Python seam of the reference on the GPU: keyword names of the matmul forwarder, the
CUTLASS-ordered metadata export for 8-bit values, the tensor-subclass flatten protocol, the
`*_torch` operator names."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _small_ints(shape, seed, lo=-3, hi=4):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi, shape, generator=g).float()


def test_forwarder_takes_the_reference_keywords(cuda):
    """sparse/sparse_semi_structured_linear.py:4: (input, weight, meta, bias_opt=None, activation_opt=None)."""
    import sparse
    w = _small_ints((128, 256), 1).half()
    x = _small_ints((72, 256), 2).half().to(cuda)
    bias = _small_ints((128,), 3).half()
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float().cpu(), torch.where(mask, w.float(), torch.zeros(()))) + bias.float()
    s = sparse.to_sparse_semi_structured(w.to(cuda))
    values, meta = s.values(), s.indices()
    fn = sparse.sparse_semi_structured_linear
    assert fn(x, values, meta, bias_opt=bias.to(cuda)).float().cpu().equal(ref)
    assert fn(x, values, meta, bias.to(cuda), "relu").float().cpu().equal(ref.clamp_min(0))              # positional, as the binding
    assert fn(x, values, meta, bias_opt=bias.to(cuda), activation_opt="relu").float().cpu().equal(ref.clamp_min(0))
    assert fn(x, values, meta, bias=bias.to(cuda)).float().cpu().equal(ref)                               # the reference's own call (semi_structured.py:433-438)
    with pytest.raises(TypeError):
        fn(x, values, meta, bias_opt=bias.to(cuda), bias=bias.to(cuda))
    with pytest.raises(RuntimeError):
        fn(x, values, meta, activation_opt="tanh")


def test_forwarder_sees_every_rewrite_of_raw_operands(cuda):
    """Raw (values, meta) tensors are repacked on every call: a rewrite that no version counter records
    (`.data`, a kernel writing through the raw pointer) must change the product; inference-mode tensors
    (which have no version counter) are accepted; a wrapper keeps its own panel copy."""
    import sparse
    from sparse import _native as N
    w = _small_ints((128, 256), 4).half()
    x = _small_ints((64, 256), 5).half().to(cuda)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float().cpu(), torch.where(mask, w.float(), torch.zeros(())))
    s = sparse.to_sparse_semi_structured(w.to(cuda))
    values, meta = s.values().clone(), s.indices().clone()
    fn = sparse.sparse_semi_structured_linear
    assert fn(x, values, meta).float().cpu().equal(ref)
    version = values._version
    values.data.mul_(2)                                              # does not move the version counter
    assert values._version == version
    assert fn(x, values, meta).float().cpu().equal(2 * ref)
    # rewritten through the C ABI: the library's own kernels write through raw pointers
    w2 = _small_ints((128, 256), 6).half()
    mask2 = oracle.prune24_mask(w2.float())
    ref2 = oracle.spmm_ref(x.float().cpu(), torch.where(mask2, w2.float(), torch.zeros(())))
    w2g = w2.to(cuda)
    N.check(N.lib().tf24_prune_compress(w2g.data_ptr(), N.F16, N.ROW_MAJOR, 256, 128, 256, N.PRUNE_MAGNITUDE, None, N.U8, 0, None, 0,
                                        values.data_ptr(), N.F16, meta.data_ptr(), N.COMPRESSED_CANONICAL, N.stream_ptr()))
    assert fn(x, values, meta).float().cpu().equal(ref2)
    with torch.inference_mode():
        vi, mi = values.clone(), meta.clone()
        assert fn(x, vi, mi).float().cpu().equal(ref2)
    # a wrapper owns its storage: the panel copy made by the first product is kept
    wrapper = sparse.SparseSemiStructuredTensor(None, original_shape=torch.Size([128, 256]), sparse_tensor_cutlass=values,
                                                meta_tensor_cutlass=meta, dtype=torch.float16)
    assert fn(x, wrapper).float().cpu().equal(ref2)
    assert wrapper._store_layout == N.COMPRESSED_PANEL
    kept = wrapper._store_values.data_ptr()
    assert fn(x, wrapper).float().cpu().equal(ref2) and wrapper._store_values.data_ptr() == kept


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.int8, torch.float16])
def test_indices_cutlass_matches_the_oracle(cuda, dtype):
    """The CUTLASS-reordered metadata export (reorder_meta + ColumnMajorInterleaved<2>, .cu:826-851), also
    for the int32 metadata words of 8-bit values; the oracle's reorder is pinned by upstream PyTorch's
    converter for int16 and int32 words."""
    import sparse
    m, k = 64, 256
    if dtype == torch.int8:
        w = _small_ints((m, k), 6, -20, 21).to(torch.int8)
        want_v, want_m = oracle.compress24(w, out_dtype=torch.int8)
        s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=torch.int8)
    else:
        w = _small_ints((m, k), 6).bfloat16()
        want_v, want_m = oracle.compress24(w, out_dtype=dtype)
        s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype)
    assert want_m.dtype == (torch.int16 if dtype == torch.float16 else torch.int32)
    assert s.indices().cpu().equal(want_m)
    got = s.indices_cutlass().cpu()
    assert got.dtype == want_m.dtype and got.equal(oracle.cutlass_reorder_meta(want_m))
    assert oracle.cutlass_unreorder_meta(got).equal(want_m)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float8_e4m3fn])
def test_tensor_flatten_round_trip(cuda, dtype):
    """__tensor_flatten__ / __tensor_unflatten__ (reference semi_structured.py:293-321): the inner
    tensors and the context rebuild an equivalent wrapper, transposed or not."""
    import sparse
    w = _small_ints((64, 256), 7).bfloat16()
    x = _small_ints((32, 256), 8).to(dtype).to(cuda)
    for s in (sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype), sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype).t()):
        names, ctx = s.__tensor_flatten__()
        assert len(names) == 2
        inner = {n: getattr(s, n) for n in names}
        assert all(isinstance(t, torch.Tensor) and not isinstance(t, sparse.SparseSemiStructuredTensor) for t in inner.values())
        r = sparse.SparseSemiStructuredTensor.__tensor_unflatten__(inner, ctx, s.shape, None)
        assert isinstance(r, sparse.SparseSemiStructuredTensor)
        assert r.shape == s.shape and r.transposed == s.transposed and r.dtype == s.dtype
        assert r.values().view(torch.uint8).equal(s.values().view(torch.uint8)) and r.indices().equal(s.indices())
        assert r.to_dense().view(torch.uint8).equal(s.to_dense().view(torch.uint8))
        a, b = (s, r) if s.transposed else (s.t(), r.t())
        assert torch.mm(x, a).equal(torch.mm(x, b))
    with pytest.raises(RuntimeError):
        sparse.SparseSemiStructuredTensor.__tensor_unflatten__({"_store_values": inner["_store_values"]}, ctx, s.shape, None)


def test_torch_named_operators(cuda):
    """sparse24_torch / soft_threshold24_torch / MVUE24_approx_torch (sparse/legacy.py:26-40, :96-117,
    :227-268): any shape, groups of 4 along the flattened tensor, int32 mask."""
    import sparse
    g = torch.Generator().manual_seed(9)
    w = torch.randn(6, 16, 40, generator=g)
    for dt in (torch.float32, torch.bfloat16):
        wd = w.to(dt)
        sp, mask = sparse.sparse24_torch(wd.to(cuda))
        want_sp, want_mask = oracle.sparse24_dense(wd.reshape(-1, 40))
        assert mask.dtype == torch.int32 and mask.shape == w.shape and sp.shape == w.shape
        assert sp.cpu().reshape(-1, 40).equal(want_sp) and mask.cpu().reshape(-1, 40).eq(want_mask.int()).all()
        st, mask = sparse.soft_threshold24_torch(wd.to(cuda))
        want_st, want_mask = oracle.soft_threshold24(wd.reshape(-1, 40))
        assert st.cpu().reshape(-1, 40).equal(want_st) and mask.cpu().reshape(-1, 40).eq(want_mask.int()).all()
        u = torch.rand(w.shape, generator=g)
        est = sparse.MVUE24_approx_torch(wd.to(cuda), rand=u.to(cuda))
        assert est.cpu().reshape(-1, 40).equal(oracle.mvue24_dense(wd.reshape(-1, 40), u.reshape(-1, 40)))
    flat = torch.randn(24, generator=g)                                      # one dimension, 8 | numel
    sp, mask = sparse.sparse24_torch(flat.to(cuda))
    assert sp.cpu().equal(oracle.sparse24_dense(flat.view(-1, 8))[0].view(-1)) and mask.sum().item() == 12


@pytest.mark.parametrize("dtype,m,k", [(torch.float16, 64, 256), (torch.bfloat16, 352, 704), (torch.float8_e4m3fn, 96, 640),
                                       (torch.int8, 32, 128), (torch.float16, 32, 64)])
def test_repack_to_and_from_the_reference_storage(cuda, dtype, m, k):
    """tf24_repack_to between the canonical, panel and CUTLASS-reordered forms (int16 and int32 metadata
    words), against the oracle's reorder (pinned by upstream PyTorch's converter); tf24_decompress from the
    reordered form."""
    import sparse
    from sparse import _native as N
    if dtype == torch.int8:
        w = _small_ints((m, k), 11, -20, 21).to(torch.int8)
    else:
        w = _small_ints((m, k), 11).bfloat16()
    want_v, want_m = oracle.compress24(w, out_dtype=dtype)
    want_r = oracle.cutlass_reorder_meta(want_m)
    s = sparse.to_sparse_semi_structured(w.to(cuda), dtype=dtype)
    code = N.operand_code(dtype)
    pv, pm = s._store_values.contiguous(), s._store_meta.contiguous()
    cv, cm = s.values().contiguous(), s.indices().contiguous()
    lib = N.lib()

    def repack(vin, min_, frm, to, with_values=True):
        ov, om = torch.empty_like(pv), torch.empty_like(pm)
        N.check(lib.tf24_repack_to(vin.data_ptr() if with_values else None, min_.data_ptr(), code, m, k, frm, to,
                                   ov.data_ptr() if with_values else None, om.data_ptr(), N.stream_ptr()))
        return ov, om

    def same(t, want):
        return t.view(torch.uint8).cpu().reshape(-1).equal(want.contiguous().view(torch.uint8).reshape(-1))

    rv, rm = repack(cv, cm, N.COMPRESSED_CANONICAL, N.COMPRESSED_CUTLASS)          # the reference's reordering step
    assert same(rv, want_v) and same(rm, want_r)
    _, rm2 = repack(cv, cm, N.COMPRESSED_CANONICAL, N.COMPRESSED_CUTLASS, with_values=False)
    assert same(rm2, want_r)
    rv3, rm3 = repack(pv, pm, N.COMPRESSED_PANEL, N.COMPRESSED_CUTLASS)
    assert same(rv3, want_v) and same(rm3, want_r)
    bv, bm = repack(rv, rm, N.COMPRESSED_CUTLASS, N.COMPRESSED_CANONICAL)          # import: back to the nibble stream
    assert same(bv, want_v) and same(bm, want_m)
    qv, qm = repack(rv, rm, N.COMPRESSED_CUTLASS, N.COMPRESSED_PANEL)              # import: straight to the matmul's form
    assert same(qv, pv.cpu()) and same(qm, pm.cpu())
    dense = torch.empty((m, k), dtype=dtype, device=cuda)
    N.check(lib.tf24_decompress(rv.data_ptr(), code, rm.data_ptr(), N.COMPRESSED_CUTLASS, m, k, dense.data_ptr(), N.stream_ptr()))
    assert same(dense, oracle.decompress24(want_v, want_m))
    with pytest.raises(RuntimeError):
        N.check(lib.tf24_repack_to(cv.data_ptr(), cm.data_ptr(), code, m, k, N.COMPRESSED_CUTLASS, N.COMPRESSED_CUTLASS,
                                   rv.data_ptr(), rm.data_ptr(), N.stream_ptr()))
    with pytest.raises(RuntimeError):
        N.check(lib.tf24_repack_to(cv.data_ptr(), cm.data_ptr(), code, m, k + 8, N.COMPRESSED_CANONICAL, N.COMPRESSED_CUTLASS,
                                   rv.data_ptr(), rm.data_ptr(), N.stream_ptr()))


@pytest.mark.parametrize("dtype,n,k,j", [(torch.float16, 32, 128, 24), (torch.float16, 352, 640, 296), (torch.bfloat16, 4128, 256, 520),
                                         (torch.float8_e4m3fn, 352, 640, 304), (torch.int8, 96, 256, 48)])
def test_product_from_reference_ordered_metadata(cuda, dtype, n, k, j):
    """x . W^T with W given the way the reference's binding takes it (sparse_semi_structured_linear.py:4-5): row-major
    values + CUTLASS-reordered metadata made by the oracle, never seen by this library's compression.  Through
    the functional entry point (`meta_layout`), through the C ABI directly (the general kernel reads the
    reordered words) and through a wrapper built with the class flag; exact on small integers."""
    import sparse
    from sparse import _native as N
    lo, hi = (-20, 21) if dtype == torch.int8 else (-3, 4)
    w = _small_ints((n, k), 21, lo, hi).to(dtype)
    x = _small_ints((j, k), 22, -2, 3).to(dtype)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(())))
    values, meta = oracle.compress24(w.float(), out_dtype=dtype) if dtype != torch.int8 else oracle.compress24(w, out_dtype=dtype)
    reordered = oracle.cutlass_reorder_meta(meta)
    vg, mg, xg = values.to(cuda), reordered.to(cuda), x.to(cuda)
    odt = torch.int32 if dtype == torch.int8 else torch.float32 if dtype in (torch.float8_e4m3fn, torch.float8_e5m2) else dtype
    want = ref.to(odt).float()
    out = sparse.sparse_semi_structured_linear(xg, vg, mg, meta_layout="cutlass")
    assert out.dtype == odt and out.float().cpu().equal(want)
    if not reordered.equal(meta):
        assert not sparse.sparse_semi_structured_linear(xg, vg, mg, meta_layout="canonical").float().cpu().equal(want)
    # the C ABI on the reference's storage as it is
    c = torch.empty((j, n), dtype=odt, device=cuda)
    N.check(N.lib().tf24_spmm(vg.data_ptr(), mg.data_ptr(), N.COMPRESSED_CUTLASS, N.operand_code(dtype), n, k,
                              xg.data_ptr(), N.ROW_MAJOR, k, j, c.data_ptr(), N.operand_code(odt), N.COL_MAJOR, n,
                              None, 1.0, N.ACT_NONE, None, 0, N.stream_ptr()))
    assert c.float().cpu().equal(want)
    # the reference's tensor contract: constructor argument and indices() speak the reordered form
    cls = sparse.SparseSemiStructuredTensor
    cls._CUTLASS_METADATA = True
    try:
        s = cls(None, original_shape=torch.Size([n, k]), sparse_tensor_cutlass=vg, meta_tensor_cutlass=mg, dtype=dtype)
        assert s.indices().cpu().equal(reordered) and s.meta_tensor_cutlass.cpu().equal(reordered)
        assert s.indices_canonical().cpu().equal(meta)
        assert s.values().cpu().view(torch.uint8).equal(values.view(torch.uint8))
        assert torch.mm(xg, s.t()).float().cpu().equal(want)
        assert s.to_dense().cpu().view(torch.uint8).equal(oracle.decompress24(values, meta).view(torch.uint8))
        fresh = sparse.to_sparse_semi_structured(w.to(cuda) if dtype == torch.int8 else w.float().to(cuda), dtype=dtype)
        assert fresh.indices().cpu().equal(reordered) and fresh.indices_cutlass().cpu().equal(reordered)
        assert sparse.sparse_semi_structured_linear(xg, fresh.values(), fresh.indices()).float().cpu().equal(want)
    finally:
        cls._CUTLASS_METADATA = False
    assert fresh.indices().cpu().equal(meta)


@pytest.mark.parametrize("dtype,n,k,j,sparse_first", [
    (torch.float16, 96, 256, 8, False),            # one-pass kernel for a few dense columns
    (torch.float16, 352, 640, 48, False),          # 256 x 64 tiles
    (torch.bfloat16, 352, 640, 120, False),        # 256 x 128 tiles
    (torch.float16, 352, 640, 296, False),         # 256 x 256 tiles, one workgroup per tile
    (torch.float16, 352, 640, 296, True),          # i-major output, k strided dense operand
    (torch.float16, 256, 4096, 264, False),        # k pieces through the workspace
    (torch.bfloat16, 4128, 320, 4112, False),      # chained tiles, 8 waves
    (torch.float16, 4128, 2112, 4112, False),      # chained tiles, 4 waves (33 stages)
    (torch.float8_e4m3fn, 4128, 4224, 4112, False),
    (torch.float8_e4m3fn, 352, 640, 304, False)])
def test_spmm_padded_leading_dimensions(cuda, dtype, n, k, j, sparse_first):
    """tf24_spmm through the C ABI with ldb and ldc larger than the rows they address (operands that are slices of
    wider buffers): the product must equal the contiguous one bit for bit and nothing outside the [rows, cols]
    window of the output buffer may be written (it is pre-filled with a sentinel)."""
    import sparse
    N = sparse._native
    odt = torch.bfloat16 if dtype == torch.float8_e4m3fn else dtype
    pad_b, pad_c = 16 * 3, 8 * 5
    w = _small_ints((n, k), 91, -2, 3).to(dtype)
    x = _small_ints((j, k), 92, -2, 3).to(dtype)
    bias = (_small_ints((n,), 93) * 0.5).to(odt).to(cuda)
    s = sparse.to_sparse_semi_structured(w.float().to(cuda), dtype=dtype)
    mask = oracle.prune24_mask(w.float())
    want = (oracle.spmm_ref(x.float(), torch.where(mask, w.float(), torch.zeros(()))) + bias.float().cpu()).to(odt)     # [j, n]
    if sparse_first:
        # S @ dense with dense [k, j] row-major in a wider buffer (k strided), output [n, j] row-major in a wider buffer
        wide_b = torch.zeros(k, j + pad_b, dtype=dtype, device=cuda)
        wide_b[:, :j] = x.to(cuda).t()
        wide_c = torch.full((n, j + pad_c), 7.0, dtype=odt, device=cuda)
        b_layout, ldb, c_layout, ldc = N.COL_MAJOR, j + pad_b, N.ROW_MAJOR, j + pad_c
        want = want.t()
    else:
        wide_b = torch.zeros(j, k + pad_b, dtype=dtype, device=cuda)
        wide_b[:, :k] = x.to(cuda)
        wide_c = torch.full((j, n + pad_c), 7.0, dtype=odt, device=cuda)
        b_layout, ldb, c_layout, ldc = N.ROW_MAJOR, k + pad_b, N.COL_MAJOR, n + pad_c
    code = N.operand_code(dtype)
    ws_bytes = N.lib().tf24_spmm_workspace_bytes(code, n, k, j)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=cuda)
    N.check(N.lib().tf24_spmm(s._store_values.data_ptr(), s._store_meta.data_ptr(), s._store_layout, code, n, k,
                              wide_b.data_ptr(), b_layout, ldb, j, wide_c.data_ptr(), N.operand_code(odt), c_layout, ldc,
                              bias.data_ptr(), 1.0, N.ACT_NONE, ws.data_ptr() if ws_bytes else None, ws_bytes, N.stream_ptr()))
    torch.cuda.synchronize()
    rows, cols = want.shape
    assert wide_c[:, :cols].float().cpu().equal(want.float())
    assert bool((wide_c[:, cols:] == 7.0).all())


@pytest.mark.parametrize("dtype,m,k", [(torch.float16, 352, 704), (torch.float8_e4m3fn, 96, 640)])
def test_repack_to_one_part_only(cuda, dtype, m, k):
    """tf24_repack_to with NULL for the part not wanted: values only between the canonical and the panel form,
    metadata only between any two forms -- each equal to that part of the full conversion, the other output untouched."""
    import sparse
    N = sparse._native
    w = _small_ints((m, k), 131).to(cuda)
    s = sparse.to_sparse_semi_structured(w, dtype=dtype)
    assert s._store_layout == N.COMPRESSED_PANEL
    code = N.operand_code(dtype)
    pv, pm = s._store_values, s._store_meta
    cv, cm = torch.empty_like(pv), torch.empty_like(pm)
    N.check(N.lib().tf24_repack_to(pv.data_ptr(), pm.data_ptr(), code, m, k, N.COMPRESSED_PANEL, N.COMPRESSED_CANONICAL, cv.data_ptr(), cm.data_ptr(), N.stream_ptr()))
    bytes_of = lambda t: t.contiguous().view(torch.uint8)
    for from_layout, to_layout, vin, min_, vwant, mwant in ((N.COMPRESSED_PANEL, N.COMPRESSED_CANONICAL, pv, pm, cv, cm),
                                                           (N.COMPRESSED_CANONICAL, N.COMPRESSED_PANEL, cv, cm, pv, pm)):
        v = torch.full_like(pv.view(torch.uint8), 0x5a)
        N.check(N.lib().tf24_repack_to(vin.data_ptr(), None, code, m, k, from_layout, to_layout, v.data_ptr(), None, N.stream_ptr()))
        assert v.equal(bytes_of(vwant).view_as(v))
        mt = torch.full_like(pm.view(torch.uint8), 0x5a)
        N.check(N.lib().tf24_repack_to(None, min_.data_ptr(), code, m, k, from_layout, to_layout, None, mt.data_ptr(), N.stream_ptr()))
        assert mt.equal(bytes_of(mwant).view_as(mt))
    # the reordered form: metadata straight from the panel words, and back
    want = oracle.cutlass_reorder_meta(s.indices_canonical().cpu())
    got = torch.empty_like(pm)
    N.check(N.lib().tf24_repack_to(None, pm.data_ptr(), code, m, k, N.COMPRESSED_PANEL, N.COMPRESSED_CUTLASS, None, got.data_ptr(), N.stream_ptr()))
    assert bytes_of(got).cpu().equal(bytes_of(want).view(-1).view_as(bytes_of(got).cpu()))
    back = torch.empty_like(pm)
    N.check(N.lib().tf24_repack_to(None, got.data_ptr(), code, m, k, N.COMPRESSED_CUTLASS, N.COMPRESSED_PANEL, None, back.data_ptr(), N.stream_ptr()))
    assert bytes_of(back).equal(bytes_of(pm))
    assert N.lib().tf24_repack_to(None, None, code, m, k, N.COMPRESSED_PANEL, N.COMPRESSED_CANONICAL, None, None, N.stream_ptr()) != 0
