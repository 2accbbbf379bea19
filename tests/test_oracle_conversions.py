"""Pins the oracle's prune / encode / compress functions against the reference's own
known answers and against independent closed forms (CPU only)."""
import itertools

import pytest
import torch

import oracle


def _topk_closed_form(x):
    """Keep the two elements ranking highest under the key (|x|, index)."""
    g = x.float().abs().reshape(-1, 4)
    mask = torch.zeros_like(g, dtype=torch.bool)
    for row in range(g.shape[0]):
        order = sorted(range(4), key=lambda i: (g[row, i].item(), i), reverse=True)[:2]
        mask[row, order] = True
    return mask.reshape(x.shape)


def test_mask_bruteforce_all_tie_shapes():
    # every 4-tuple over a 6-symbol alphabet (signs included): 1296 groups, all tie shapes
    alphabet = [0.0, -1.0, 1.0, 2.0, -2.0, 3.0]
    groups = torch.tensor(list(itertools.product(alphabet, repeat=4)), dtype=torch.float32)
    x = groups.reshape(-1, 4)
    got = oracle.prune24_mask(x)
    assert got.sum(-1).eq(2).all()
    assert got.equal(_topk_closed_form(x))
    # all-equal group keeps the two LAST elements
    assert oracle.prune24_mask(torch.ones(1, 4)).tolist() == [[False, False, True, True]]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_mask_equals_topk_on_random(dtype):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 128, generator=g).to(dtype)
    got = oracle.prune24_mask(x)
    assert got.equal(_topk_closed_form(x))


# the 16-row truth table in the comment of _semi_structured_conversions.py:46-71
_TRUTH = {
    (1, 1, 0, 0): 0b0100, (1, 0, 1, 0): 0b1000, (0, 1, 1, 0): 0b1001, (1, 0, 0, 1): 0b1100,
    (0, 1, 0, 1): 0b1101, (0, 0, 1, 1): 0b1110, (0, 0, 0, 0): 0b1110, (0, 0, 0, 1): 0b1110,
    (0, 0, 1, 0): 0b1110, (0, 1, 0, 0): 0b1101, (0, 1, 1, 1): 0b1001, (1, 0, 0, 0): 0b1100,
    (1, 0, 1, 1): 0b1000, (1, 1, 0, 1): 0b0100, (1, 1, 1, 0): 0b1000, (1, 1, 1, 1): 0b1000,
}


def test_encode_truth_table():
    assert len(_TRUTH) == 16
    for bits, code in _TRUTH.items():
        idx0, idx1 = oracle.encode24(torch.tensor([bits], dtype=torch.bool))
        assert int(idx0 | (idx1 << 2)) == code, bits


def test_docstring_known_answer():
    # semi_structured.py:604-627: [0,0,1,1] tiled to 128x128 fp16 -> values all 1, meta all -4370
    a = torch.tensor([0.0, 0.0, 1.0, 1.0]).tile((128, 32)).half()
    values, meta = oracle.compress24(a)
    assert values.shape == (128, 64) and values.dtype == torch.float16 and values.eq(1).all()
    assert meta.shape == (128, 8) and meta.dtype == torch.int16 and meta.eq(-4370).all()
    # constant meta is invariant under the CUTLASS reordering
    assert oracle.cutlass_reorder_meta(meta).eq(-4370).all()


def test_config1_shapes_and_invariants():
    # BASELINE config 1: W[3072,768] fp16 ~ N(0, 0.02), seed 0
    g = torch.Generator().manual_seed(0)
    w = (0.02 * torch.randn(3072, 768, generator=g)).half()
    mask = oracle.prune24_mask(w)
    values, meta = oracle.compress24(w)
    assert values.shape == (3072, 384) and meta.shape == (3072, 48) and meta.dtype == torch.int16
    assert mask.reshape(-1, 4).sum(-1).eq(2).all()
    idx0, idx1 = oracle.encode24(mask)
    assert (idx0 < idx1).all()
    dense = oracle.decompress24(values, meta)
    assert dense.equal(torch.where(mask, w, torch.zeros_like(w)))
    # kept magnitudes dominate dropped ones in every group
    kept_min = torch.where(mask, w.abs().float(), torch.tensor(float("inf"))).reshape(-1, 4).min(-1).values
    drop_max = torch.where(mask, torch.tensor(-1.0), w.abs().float()).reshape(-1, 4).max(-1).values
    assert (kept_min >= drop_max).all()


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16, torch.float8_e4m3fn])
def test_compress_roundtrip(out_dtype):
    g = torch.Generator().manual_seed(3)
    w = torch.randn(64, 256, generator=g).bfloat16()
    mask = oracle.prune24_mask(w)
    values, meta = oracle.compress24(w, out_dtype=out_dtype)
    assert meta.dtype == oracle.meta_dtype_for(out_dtype)
    expect = torch.where(mask, w, torch.zeros_like(w)).to(out_dtype)
    got = oracle.decompress24(values, meta)
    assert got.view(torch.uint8).equal(expect.view(torch.uint8))


def test_mask_mode_follows_given_mask_and_truth_table():
    g = torch.Generator().manual_seed(4)
    w = torch.randn(32, 64, generator=g).half()
    # arbitrary (also invalid) masks: encoding follows the truth table row by row
    mask = torch.rand(32, 64, generator=g) < 0.5
    values, meta = oracle.compress24(w, mask=mask)
    nibbles = torch.stack([(meta.long() >> (4 * i)) & 0xF for i in range(4)], -1).reshape(32, 16)
    for r in range(32):
        for gi in range(16):
            bits = tuple(int(b) for b in mask[r, 4 * gi:4 * gi + 4])
            code = _TRUTH[bits]
            assert int(nibbles[r, gi]) == code
            assert values[r, 2 * gi] == w[r, 4 * gi + (code & 3)]
            assert values[r, 2 * gi + 1] == w[r, 4 * gi + (code >> 2)]


@pytest.mark.parametrize("dtype,shape", [(torch.float16, (32, 128)), (torch.float16, (64, 256)),
                                         (torch.bfloat16, (64, 128)), (torch.int8, (32, 128)),
                                         (torch.int8, (64, 256))])
def test_cutlass_reorder_matches_upstream_torch(dtype, shape):
    """On an already-2:4 matrix the reference reduces to upstream PyTorch's converter
    (selection by `dense != 0`), which ships in the installed torch and runs on CPU."""
    conv = pytest.importorskip("torch.sparse._semi_structured_conversions")
    g = torch.Generator().manual_seed(5)
    m, k = shape
    vals = torch.randint(1, 9, (m, k), generator=g).float()
    keep = torch.zeros(m, k // 4, 4, dtype=torch.bool)
    pos = torch.stack([torch.randperm(4, generator=g)[:2] for _ in range(m * k // 4)]).reshape(m, k // 4, 2)
    keep.scatter_(-1, pos, True)
    dense = (vals * keep.reshape(m, k)).to(dtype)
    up_values, up_meta = conv.sparse_semi_structured_from_dense_cutlass(dense)
    values, meta = oracle.compress24(dense, mask=dense != 0, out_dtype=dtype)
    assert values.equal(up_values)
    assert oracle.cutlass_reorder_meta(meta).equal(up_meta)
    assert oracle.cutlass_unreorder_meta(up_meta).equal(meta)
    assert conv.sparse_semi_structured_to_dense_cutlass(values, oracle.cutlass_reorder_meta(meta)).equal(dense)


def test_sparse24_dense():
    g = torch.Generator().manual_seed(6)
    w = torch.randn(32, 64, generator=g).bfloat16()
    sparse, mask = oracle.sparse24_dense(w)
    assert mask.dtype == w.dtype and sparse.dtype == w.dtype
    assert sparse.equal(w * mask)
