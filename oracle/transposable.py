"""Oracle: transposable 4x4 mask search over the 90 row-and-column 2:4 patterns.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/transposable_semi_structured.py:8-47 (kernel), :50-94 (wrapper) and the pattern
table at :105-196: for every aligned 4x4 block B of |W| (W itself when abs=False) score each of
the 90 patterns P by sum(P * B), take the first maximum, mask = that pattern, sparse = W * mask.

The table is a closed form: all 4x4 0/1 matrices whose rows and columns each sum to 2,
flattened row-major, in lexicographically DESCENDING order.  Equivalently, pattern index order
is ascending lexicographic order of (q0, q1, q2, q3), q_r being row r's column pair in the
order (0,1) (0,2) (0,3) (1,2) (1,3) (2,3).

Arithmetic (the reference accumulates on tensor cores in an unspecified order): float32,
  s[r][q] = B[r][c1(q)] + B[r][c2(q)]
  top[q0,q1] = s[0][q0] + s[1][q1]        bottom[q2,q3] = s[2][q2] + s[3][q3]
  score = top + bottom
and the search is two-level: for each class of bottoms with the same column-count vector keep
the first maximal bottom; for each top (in order) add the best compatible bottom; keep the first
maximal total.  Rounding is monotone, so the score found is the maximum of the 90 rounded
scores, and whenever the float32 sums are exact (always for exact ties such as equal or zero
entries) the pattern found is the first of the maximal ones, like the reference's argmax.
"""
import itertools

import torch

PAIRS = ((0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3))


def _row_bits(q):
    c1, c2 = PAIRS[q]
    return [1 if c in (c1, c2) else 0 for c in range(4)]


def transposable_patterns():
    """int64 [90, 16] pattern table in the reference's order (descending lexicographic)."""
    rows = []
    for qs in itertools.product(range(6), repeat=4):
        mat = [_row_bits(q) for q in qs]
        if all(sum(mat[r][c] for r in range(4)) == 2 for c in range(4)):
            rows.append([b for r in mat for b in r])
    rows.sort(reverse=True)
    return torch.tensor(rows, dtype=torch.int64)


def _counts(qa, qb):
    ra, rb = _row_bits(qa), _row_bits(qb)
    return tuple(ra[c] + rb[c] for c in range(4))


def _tables():
    combos = list(itertools.product(range(6), repeat=2))          # index = qa*6 + qb
    classes = sorted({_counts(*c) for c in combos})
    cls_of = [classes.index(_counts(*c)) for c in combos]
    comp_of = [classes.index(tuple(2 - v for v in _counts(*c))) for c in combos]
    return combos, classes, cls_of, comp_of


_COMBOS, _CLASSES, _CLS_OF, _COMP_OF = _tables()


def _blocks(x):
    m, k = x.shape
    return x.reshape(m // 4, 4, k // 4, 4).permute(0, 2, 1, 3)     # [m/4, k/4, r, c]


def _check(dense):
    if dense.dim() != 2:
        raise RuntimeError(f"Expected 2-dimensional dense tensor, got {dense.dim()}-dimensional tensor")
    if dense.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise RuntimeError(f"Invalid datatype {dense.dtype} of dense matrix")
    m, k = dense.shape
    if m % 32:
        raise RuntimeError(f"Number rows columns of dense matrix {m} must be divisible by 32")
    if k % 64:
        raise RuntimeError(f"Number of columns of dense matrix {k} must be divisible by 64")


def transposable_mask(dense, use_abs=True, return_index=False):
    """Returns (sparse, mask): sparse = dense*mask in dense's dtype, mask bool."""
    _check(dense)
    m, k = dense.shape
    blk = _blocks(dense.float())
    if use_abs:
        blk = blk.abs()
    s = torch.stack([blk[..., PAIRS[q][0]] + blk[..., PAIRS[q][1]] for q in range(6)], dim=-1)  # [.., r, q]
    top = [s[..., 0, qa] + s[..., 1, qb] for qa, qb in _COMBOS]
    bot = [s[..., 2, qa] + s[..., 3, qb] for qa, qb in _COMBOS]
    # first maximal bottom of every class
    best_b = [None] * len(_CLASSES)
    best_bi = [None] * len(_CLASSES)
    for b in range(36):
        c = _CLS_OF[b]
        if best_b[c] is None:
            best_b[c] = bot[b]
            best_bi[c] = torch.full(bot[b].shape, b, dtype=torch.int64)
        else:
            upd = bot[b] > best_b[c]
            best_b[c] = torch.where(upd, bot[b], best_b[c])
            best_bi[c] = torch.where(upd, torch.full_like(best_bi[c], b), best_bi[c])
    # first maximal top + best compatible bottom
    best = best_t = best_bsel = None
    for t in range(36):
        c = _COMP_OF[t]
        cand = top[t] + best_b[c]
        if best is None:
            best, best_t, best_bsel = cand, torch.full(cand.shape, t, dtype=torch.int64), best_bi[c]
        else:
            upd = cand > best
            best = torch.where(upd, cand, best)
            best_t = torch.where(upd, torch.full_like(best_t, t), best_t)
            best_bsel = torch.where(upd, best_bi[c], best_bsel)
    qs = torch.stack((best_t // 6, best_t % 6, best_bsel // 6, best_bsel % 6), dim=-1)            # [.., r]
    rowbits = torch.tensor([_row_bits(q) for q in range(6)], dtype=torch.bool)
    mask = rowbits[qs]                                                                          # [m/4,k/4,r,c]
    mask = mask.permute(0, 2, 1, 3).reshape(m, k)
    sparse = torch.where(mask, dense, torch.zeros_like(dense))
    if return_index:
        pats = transposable_patterns()
        lut = {tuple(p.tolist()): i for i, p in enumerate(pats)}
        flat = rowbits[qs].reshape(-1, 16).long()
        idx = torch.tensor([lut[tuple(r.tolist())] for r in flat]).reshape(m // 4, k // 4)
        return sparse, mask, idx
    return sparse, mask


def transposable_mask_bruteforce(dense, use_abs=True):
    """Plain 90-way enumeration with float64 scores and first-max argmax (checker for the
    two-level search on data whose sums are exact)."""
    _check(dense)
    m, k = dense.shape
    blk = _blocks(dense.double())
    if use_abs:
        blk = blk.abs()
    pats = transposable_patterns()
    scores = blk.reshape(m // 4, k // 4, 16) @ pats.double().t()
    idx = scores.argmax(dim=-1)
    mask = pats[idx].bool().reshape(m // 4, k // 4, 4, 4).permute(0, 2, 1, 3).reshape(m, k)
    return torch.where(mask, dense, torch.zeros_like(dense)), mask, idx
