"""Golden vectors (tests/golden/): the known answers the reference's own files hold, and the seeded
64 x 128 case written by tests/golden/make_fixtures.py.  Without a GPU they pin the oracle; with one
(-m gpu) the HIP path must reproduce the same bytes."""
import json
import os

import numpy as np
import pytest
import torch

import oracle

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def known():
    with open(os.path.join(HERE, "reference_known_answers.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def case():
    return dict(np.load(os.path.join(HERE, "conversion_64x128.npz")))


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).view(dtype)
    if dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return t.view(dtype)
    if dtype == torch.bool:
        return t != 0
    return t


def _same(got, want_bits):
    g = got.detach().cpu().contiguous()
    if g.dtype in (torch.float16, torch.bfloat16):
        g = g.view(torch.int16)
    elif g.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        g = g.view(torch.uint8)
    elif g.dtype == torch.bool:
        g = g.to(torch.uint8)
    w = torch.from_numpy(np.ascontiguousarray(want_bits))
    if w.dtype == torch.uint16:
        w = w.view(torch.int16)
    assert g.shape == w.shape and g.dtype == w.dtype, (g.shape, g.dtype, w.shape, w.dtype)
    assert g.equal(w)


# ------------------------------------------------------------------ the reference's own vectors, on the oracle
def test_oracle_nibble_table(known):
    for quad, nibble in known["nibble_table"]["mask_to_nibble"]:
        idx0, idx1 = oracle.encode24(torch.tensor([quad], dtype=torch.bool))
        assert (idx0.item() | (idx1.item() << 2)) == nibble, quad


def test_oracle_docstring_example(known):
    ex = known["docstring_example"]
    a = torch.tensor(ex["row_pattern"], dtype=torch.float16).tile(ex["shape"][0], ex["shape"][1] // 4)
    v, m = oracle.compress24(a)
    assert (v == ex["values"]).all() and (m == ex["metadata_int16"]).all() and m.dtype == torch.int16
    assert (oracle.cutlass_reorder_meta(m) == ex["metadata_int16"]).all()          # constant: invariant under the reordering


def test_oracle_masked_add_smoke(known):
    ex = known["masked_add_smoke"]
    out = oracle.masked_add(torch.tensor(ex["grad"], dtype=torch.float32), torch.tensor(ex["p"], dtype=torch.float32),
                            torch.tensor(ex["mask"]), ex["alpha"])
    assert torch.allclose(out, torch.tensor(ex["result"]), rtol=0, atol=1e-6)


def test_oracle_reproduces_the_seeded_case(case):
    w, wb, u = _t(case["w_f16"], torch.float16), _t(case["w_bf16"], torch.bfloat16), _t(case["u_f32"])
    _same(oracle.prune24_mask(w), case["magnitude_mask"])
    v, m = oracle.compress24(w)
    _same(v, case["magnitude_values_f16"]); _same(m, case["magnitude_meta_i16"])
    _same(oracle.cutlass_reorder_meta(m), case["cutlass_reordered_meta_i16"])
    v8, m8 = oracle.compress24(wb, out_dtype=torch.float8_e4m3fn)
    _same(v8, case["magnitude_bf16_values_e4m3"]); _same(m8, case["magnitude_bf16_meta_i32"])
    mv, mm, mmask = oracle.mvue24(wb, u)
    _same(mv, case["mvue_values_f16"]); _same(mm, case["mvue_meta_i16"]); _same(mmask, case["mvue_mask"])
    sp, smask = oracle.soft_threshold24(wb)
    _same(sp, case["soft_sparse_bf16"]); _same(smask, case["soft_mask_bf16"])
    tsp, tmask = oracle.transposable_mask(wb)
    _same(tsp, case["transposable_sparse_bf16"]); _same(tmask, case["transposable_mask"])
    _same(oracle.masked_add(_t(case["grad_f32"]), w.float(), tmask, 2e-4).float(), case["masked_add_f32"])


# ------------------------------------------------------------------ the same vectors on the GPU path
@pytest.mark.gpu
def test_gpu_known_answers(cuda, known):
    import sparse
    ex = known["docstring_example"]
    a = torch.tensor(ex["row_pattern"], dtype=torch.float16).tile(ex["shape"][0], ex["shape"][1] // 4).to(cuda)
    s = sparse.to_sparse_semi_structured(a)
    assert (s.values() == ex["values"]).all() and (s.indices() == ex["metadata_int16"]).all()
    assert (s.indices_cutlass() == ex["metadata_int16"]).all()
    # every row of the table as a mask-driven compression: the kept positions are those of the nibble
    vals = torch.tensor([10.0, 20.0, 30.0, 40.0], dtype=torch.float16)
    for quad, nibble in known["nibble_table"]["mask_to_nibble"]:
        w = vals.tile(32, 16).to(cuda)
        mask = torch.tensor(quad, dtype=torch.bool).tile(32, 16).to(cuda)
        s = sparse.to_sparse_semi_structured(w, mask=mask)
        want = torch.tensor([vals[nibble & 3], vals[nibble >> 2]], dtype=torch.float16).tile(32, 16)
        assert s.values().cpu().equal(want), quad
        word = sum(nibble << (4 * i) for i in range(4))
        assert (s.indices().cpu().view(torch.int16).to(torch.int32) & 0xffff == word).all(), quad
    ex = known["masked_add_smoke"]
    grad = torch.tensor(ex["grad"], dtype=torch.float32, device=cuda)
    sparse.masked_add_(grad, torch.tensor(ex["p"], dtype=torch.float32, device=cuda), torch.tensor(ex["mask"], device=cuda) != 0, alpha=ex["alpha"])
    assert torch.allclose(grad.cpu(), torch.tensor(ex["result"]), rtol=0, atol=1e-6)


@pytest.mark.gpu
def test_gpu_reproduces_the_seeded_case(cuda, case):
    import sparse
    w, wb = _t(case["w_f16"], torch.float16).to(cuda), _t(case["w_bf16"], torch.bfloat16).to(cuda)
    u, x, grad = _t(case["u_f32"]).to(cuda), _t(case["x_f16"], torch.float16).to(cuda), _t(case["grad_f32"]).to(cuda)
    s = sparse.to_sparse_semi_structured(w)
    _same(s.values(), case["magnitude_values_f16"]); _same(s.indices(), case["magnitude_meta_i16"])
    _same(s.indices_cutlass(), case["cutlass_reordered_meta_i16"])
    s8 = sparse.to_sparse_semi_structured(wb, dtype=torch.float8_e4m3fn)
    _same(s8.values(), case["magnitude_bf16_values_e4m3"]); _same(s8.indices(), case["magnitude_bf16_meta_i32"])
    sm = sparse.to_sparse_semi_structured(wb, MVUE24=True, rand=u)
    _same(sm.values(), case["mvue_values_f16"]); _same(sm.indices(), case["mvue_meta_i16"])
    sp, smask = sparse.soft_threshold24(wb)
    _same(sp, case["soft_sparse_bf16"]); _same(smask, case["soft_mask_bf16"])
    tsp, tmask = sparse.TransposableSparse()(wb)
    _same(tsp, case["transposable_sparse_bf16"]); _same(tmask, case["transposable_mask"])
    st = sparse.to_sparse_semi_structured(wb.T, mask=tmask.T)
    _same(st.values(), case["transposed_mask_values_f16"]); _same(st.indices(), case["transposed_mask_meta_i16"])
    g = grad.clone()
    sparse.masked_add_(g, w.float(), tmask, alpha=2e-4)
    _same(g, case["masked_add_f32"])
    out = torch.mm(x, s.t()).float().cpu()
    want = _t(case["spmm_f32"])
    assert ((out - want).norm() / want.norm()).item() < 1e-2          # fp16 output against the float32 product
