"""Oracle: the counter-based uniforms of the seeded MVUE24 path.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

The reference draws the two uniforms of a group from Triton's in-kernel Philox, seeded from Python's
`random` (sparse/_semi_structured_conversions.py:536-542, :1076) -- not reproducible, so there is
nothing of the reference to match bit for bit.  The replacement is Philox4x32-10 as published
(Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11; the Random123
library): multipliers 0xD2511F53 / 0xCD9E8D57, Weyl key increments 0x9E3779B9 / 0xBB67AE85, ten
rounds.  Convention of this build: key = seed, counter = {index lo, index hi, offset lo, offset hi}
with index = row * (k/8) + (8-column unit); words 0,1 serve the unit's even group, 2,3 the odd one;
uniform = (word & 0xffffff) * 2^-24.

Pinned by the known-answer vectors of the Random123 distribution (kat_vectors, philox4x32 10 rounds).
"""
import numpy as np
import torch

_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter, key):
    """counter [..., 4], key [..., 2] (arrays of 32-bit words held in uint64) -> [..., 4] words."""
    c = np.asarray(counter, dtype=np.uint64).copy()
    k = np.broadcast_to(np.asarray(key, dtype=np.uint64), c.shape[:-1] + (2,)).copy()
    for _ in range(10):
        p0, p1 = _M0 * c[..., 0], _M1 * c[..., 2]
        n0 = (p1 >> np.uint64(32)) ^ c[..., 1] ^ k[..., 0]
        n2 = (p0 >> np.uint64(32)) ^ c[..., 3] ^ k[..., 1]
        c = np.stack((n0 & _MASK, p1 & _MASK, n2 & _MASK, p0 & _MASK), axis=-1)
        k = np.stack(((k[..., 0] + np.uint64(_W0)) & _MASK, (k[..., 1] + np.uint64(_W1)) & _MASK), axis=-1)
    return c


def mvue_uniforms(seed, offset, m, k):
    """The packed uniforms [m, k/2] (float32) of the seeded MVUE24 path."""
    index = np.arange(m * (k // 8), dtype=np.uint64)
    counter = np.stack((index & _MASK, index >> np.uint64(32),
                        np.full_like(index, offset & 0xFFFFFFFF), np.full_like(index, (offset >> 32) & 0xFFFFFFFF)), axis=-1)
    words = philox4x32_10(counter, np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint64))
    u = (words & np.uint64(0xFFFFFF)).astype(np.float32) * np.float32(2.0 ** -24)
    return torch.from_numpy(u.reshape(m, k // 2))
