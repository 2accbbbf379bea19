"""Oracle: magnitude 2:4 mask, nibble encoding, compression and decompression.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/_semi_structured_conversions.py:10-328 of the reference (pure-PyTorch spec),
extended to 8-bit value types the way the reference's Triton kernel does (:664-1069).
The metadata produced here is the CANONICAL row-major nibble stream (reference :88-108,
before its CUTLASS reordering at :178-213); the reordering is a separate function.
"""
import torch

_META_DTYPE = {
    torch.float16: torch.int16, torch.bfloat16: torch.int16,
    torch.int8: torch.int32, torch.float8_e4m3fn: torch.int32, torch.float8_e5m2: torch.int32,
}


def meta_dtype_for(values_dtype):
    """int16 for 16-bit values, int32 for 8-bit values (semi_structured.py:323-331)."""
    return _META_DTYPE[values_dtype]


def _groups(x):
    m, k = x.shape
    if k % 4:
        raise RuntimeError(f"k={k} is not a multiple of 4")
    return x.reshape(m, k // 4, 4)


def prune24_mask(dense):
    """Magnitude 2:4 mask, bool [m, k].

    Six strict '>' compares of |x| and the boolean forms of
    _semi_structured_conversions.py:42-44 (same at utils.py:62-69).
    """
    a, b, c, d = _groups(dense.float().abs()).unbind(-1)
    x1, x2, x3, x4, x5, x6 = a > b, a > c, a > d, b > c, b > d, c > d
    m0 = x2 & x3 | x1 & x2 | x1 & x3
    m1 = ~x1 & x5 | x4 & x5 | ~x1 & x4
    m2 = ~x2 & ~x4 | ~x2 & x6 | ~x4 & x6
    m3 = ~x3 & ~x5 | ~x3 & ~x6 | ~x5 & ~x6
    return torch.stack((m0, m1, m2, m3), dim=-1).reshape(dense.shape)


def encode24(mask):
    """Positions (idx0 < idx1 for valid masks) of the two kept elements of each group.

    _semi_structured_conversions.py:77-82; masks with != 2 trues follow the table at :46-71.
    Returns two int64 tensors [m, k/4].
    """
    m0, m1, m2, _ = _groups(mask != 0).unbind(-1)
    bit0 = ~m0 & m1
    bit1 = ~m0 & ~m1
    bit2 = bit1 | ~m2
    bit3 = bit0 | ~m1 | m2
    idx0 = bit0.long() | (bit1.long() << 1)
    idx1 = bit2.long() | (bit3.long() << 1)
    return idx0, idx1


def pack_meta(idx0, idx1, values_dtype):
    """Nibbles idx0 | idx1<<2, packed LSB-first, 4 per int16 or 8 per int32 (:88-108)."""
    mdt = meta_dtype_for(values_dtype)
    per = 4 if mdt == torch.int16 else 8
    m, ngroups = idx0.shape
    if ngroups % per:
        raise RuntimeError(f"k={4 * ngroups} is not a multiple of {4 * per}")
    nib = (idx0 | (idx1 << 2)).reshape(m, ngroups // per, per)
    shifts = torch.arange(per, dtype=torch.int64) * 4
    word = (nib << shifts).sum(-1)  # disjoint bit fields: sum == or
    if mdt == torch.int16:
        word = torch.where(word >= 1 << 15, word - (1 << 16), word)
    else:
        word = torch.where(word >= 1 << 31, word - (1 << 32), word)
    return word.to(mdt)


def compress24(dense, mask=None, out_dtype=torch.float16, source=None):
    """Prune (magnitude unless `mask` is given) and compress.

    Returns (values [m, k/2] in out_dtype, canonical meta [m, k/16] int16 | [m, k/32] int32).
    `source` (default: dense) is the tensor the kept values are gathered from -- the MVUE
    path passes the rescaled fp32 values there.  The gathered value is cast to out_dtype by a
    plain round-to-nearest-even conversion, like the store at
    _semi_structured_conversions.py:614-621.
    """
    if mask is None:
        mask = prune24_mask(dense)
    idx0, idx1 = encode24(mask)
    src = _groups(dense if source is None else source)
    v0 = src.gather(-1, idx0.unsqueeze(-1))
    v1 = src.gather(-1, idx1.unsqueeze(-1))
    values = torch.cat((v0, v1), dim=-1).reshape(dense.shape[0], dense.shape[1] // 2)
    return values.to(out_dtype), pack_meta(idx0, idx1, out_dtype)


def _reorder_dest(m, ncols, mdt):
    """Scatter rule of the reference: reorder_meta (csrc .cu:826-851) followed by
    ColumnMajorInterleaved<2> (_semi_structured_conversions.py:639-654 / :1047-1062)."""
    group, inter = (32, 4) if mdt == torch.int16 else (16, 2)
    r = torch.arange(m).view(-1, 1).expand(m, ncols)
    c = torch.arange(ncols).view(1, -1).expand(m, ncols)
    dr = r // group * group + (r % 8) * inter + (r % group) // 8
    top_right = ((dr % 2 == 0) & (c % 2 == 1)).long()
    bottom_left = ((dr % 2 == 1) & (c % 2 == 0)).long()
    dr = dr + top_right - bottom_left
    dc = c - top_right + bottom_left
    return (dc // 2) * m * 2 + dr * 2 + dc % 2


def cutlass_reorder_meta(meta):
    """Canonical meta -> the CUTLASS-reordered meta the reference stores (same shape)."""
    m, ncols = meta.shape
    out = torch.empty(m * ncols, dtype=meta.dtype)
    out[_reorder_dest(m, ncols, meta.dtype).reshape(-1)] = meta.reshape(-1)
    return out.view(m, ncols)


def cutlass_unreorder_meta(meta_reordered):
    """Inverse of cutlass_reorder_meta."""
    m, ncols = meta_reordered.shape
    return meta_reordered.reshape(-1)[_reorder_dest(m, ncols, meta_reordered.dtype).reshape(-1)].view(m, ncols)


def decompress24(values, meta):
    """Scatter the kept values back to their positions, zeros elsewhere.

    Inverse of compress24 on canonical meta (_semi_structured_conversions.py:291-328).
    """
    m, half_k = values.shape
    per = 4 if meta.dtype == torch.int16 else 8
    word = meta.long()
    shifts = torch.arange(2 * per, dtype=torch.int64) * 2
    pos = ((word.unsqueeze(-1) >> shifts) & 3).reshape(m, half_k)  # position of each kept value
    base = (torch.arange(half_k) // 2 * 4).view(1, -1)
    raw = values.view(torch.int16 if values.element_size() == 2 else torch.int8)
    dense = torch.zeros(m, 2 * half_k, dtype=raw.dtype)
    dense.scatter_(1, pos + base, raw)
    return dense.view(values.dtype)


def sparse24_dense(dense):
    """Dense-shaped magnitude pruning: (dense*mask, mask in the dense dtype).

    triton_ops.py:84-154 (`sparse24_triton`).
    """
    mask = prune24_mask(dense)
    return torch.where(mask, dense, torch.zeros_like(dense)), mask.to(dense.dtype)
