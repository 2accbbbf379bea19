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


def test_forwarder_keeps_the_panel_copy_of_canonical_operands(cuda):
    """Canonical (values, meta) tensors are repacked once, not per call; an in-place update of the
    values is seen."""
    import sys
    import sparse
    mod = sys.modules["sparse.sparse_semi_structured_linear"]     # the module; the package attribute of that name is the function
    w = _small_ints((128, 256), 4).half()
    x = _small_ints((64, 256), 5).half().to(cuda)
    mask = oracle.prune24_mask(w.float())
    ref = oracle.spmm_ref(x.float().cpu(), torch.where(mask, w.float(), torch.zeros(())))
    s = sparse.to_sparse_semi_structured(w.to(cuda))
    values, meta = s.values().clone(), s.indices().clone()
    mod._PANEL_CACHE.clear()
    assert sparse.sparse_semi_structured_linear(x, values, meta).float().cpu().equal(ref)
    assert len(mod._PANEL_CACHE) == 1
    wrapper = next(iter(mod._PANEL_CACHE.values()))[1]
    panel_ptr = wrapper._store_values.data_ptr()
    assert sparse.sparse_semi_structured_linear(x, values, meta).float().cpu().equal(ref)
    assert next(iter(mod._PANEL_CACHE.values()))[1] is wrapper and wrapper._store_values.data_ptr() == panel_ptr
    values.mul_(2)                                                   # in place: version counter moves, entry is rebuilt
    assert sparse.sparse_semi_structured_linear(x, values, meta).float().cpu().equal(2 * ref)
    mod._PANEL_CACHE.clear()


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
