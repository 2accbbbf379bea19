"""Writes the golden vectors under tests/golden/.

    python tests/golden/make_fixtures.py

Two kinds of data:
  * reference_known_answers.json -- the vectors the reference's own files hold for this path: the
    16-row mask -> nibble table (sparse/_semi_structured_conversions.py:46-71), the docstring example
    (sparse/semi_structured.py:604-627) and the masked_add_ smoke vector (sparse/decay.py:40-46).
    Typed in from those lines; nothing is imported from the reference.
  * conversion_64x128.npz -- seeded inputs of a 64 x 128 case with the expected outputs of every
    conversion, computed by the CPU oracle (oracle/) once it had passed the known answers above and
    its closed-form checks.  They pin the oracle against drift and give the GPU path fixed bytes to hit.
16-bit and 8-bit floats are stored as their bit patterns (uint16 / uint8).
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def bits(t):
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return t.contiguous().view(torch.uint8).numpy()
    if t.dtype == torch.bool:
        return t.numpy().astype(np.uint8)
    return t.contiguous().numpy()


def known_answers():
    # [m0, m1, m2, m3] -> nibble idx0 | idx1 << 2, the 16 rows listed at _semi_structured_conversions.py:47-71
    table = [
        [[1, 1, 0, 0], 0b0100], [[1, 0, 1, 0], 0b1000], [[0, 1, 1, 0], 0b1001], [[1, 0, 0, 1], 0b1100],
        [[0, 1, 0, 1], 0b1101], [[0, 0, 1, 1], 0b1110],
        [[0, 0, 0, 0], 0b1110], [[0, 0, 0, 1], 0b1110], [[0, 0, 1, 0], 0b1110], [[0, 1, 0, 0], 0b1101],
        [[0, 1, 1, 1], 0b1001], [[1, 0, 0, 0], 0b1100], [[1, 0, 1, 1], 0b1000], [[1, 1, 0, 1], 0b0100],
        [[1, 1, 1, 0], 0b1000], [[1, 1, 1, 1], 0b1000],
    ]
    return {
        "nibble_table": {"source": "sparse/_semi_structured_conversions.py:46-71", "mask_to_nibble": table},
        "docstring_example": {"source": "sparse/semi_structured.py:604-627", "row_pattern": [0, 0, 1, 1], "shape": [128, 128],
                              "dtype": "float16", "values": 1.0, "metadata_int16": -4370},
        "masked_add_smoke": {"source": "sparse/decay.py:40-46", "grad": [1, 1, 1, 1], "p": [1, 2, 3, 4], "mask": [1, 0, 1, 0],
                             "alpha": 0.03, "result": [1.0, 1.06, 1.0, 1.12]},
    }


def conversion_case():
    g = torch.Generator().manual_seed(0)
    w32 = 0.02 * torch.randn(64, 128, generator=g)
    w = w32.half()
    wb = torch.randn(64, 128, generator=g).bfloat16()
    u = torch.rand(64, 128, generator=g)
    x = torch.randn(32, 128, generator=g).half()
    grad = 1e-3 * torch.randn(64, 128, generator=g)
    out = {"w_f16": bits(w), "w_bf16": bits(wb), "u_f32": bits(u), "x_f16": bits(x), "grad_f32": bits(grad)}
    mask = oracle.prune24_mask(w)
    v, m = oracle.compress24(w)
    out.update(magnitude_mask=bits(mask), magnitude_values_f16=bits(v), magnitude_meta_i16=bits(m))
    v8, m8 = oracle.compress24(wb, out_dtype=torch.float8_e4m3fn)
    out.update(magnitude_bf16_values_e4m3=bits(v8), magnitude_bf16_meta_i32=bits(m8))
    out["cutlass_reordered_meta_i16"] = bits(oracle.cutlass_reorder_meta(m))
    mv, mm, mmask = oracle.mvue24(wb, u)
    out.update(mvue_values_f16=bits(mv), mvue_meta_i16=bits(mm), mvue_mask=bits(mmask))
    sp, smask = oracle.soft_threshold24(wb)
    out.update(soft_sparse_bf16=bits(sp), soft_mask_bf16=bits(smask))
    tsp, tmask = oracle.transposable_mask(wb)
    out.update(transposable_sparse_bf16=bits(tsp), transposable_mask=bits(tmask))
    tv, tm = oracle.compress24(wb.t().contiguous(), mask=tmask.t().contiguous())
    out.update(transposed_mask_values_f16=bits(tv), transposed_mask_meta_i16=bits(tm))
    out["masked_add_f32"] = bits(oracle.masked_add(grad, w.float(), tmask, 2e-4))
    out["spmm_f32"] = bits(oracle.spmm_ref(x, torch.where(mask, w, torch.zeros_like(w))))
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "reference_known_answers.json"), "w") as f:
        json.dump(known_answers(), f, indent=1)
    np.savez_compressed(os.path.join(HERE, "conversion_64x128.npz"), **conversion_case())
    print("written:", sorted(os.listdir(HERE)))
