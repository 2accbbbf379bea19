"""CPU oracle for the 2:4 sparse hot path.  TEST INFRASTRUCTURE ONLY.

Every function here restates, in plain CPU PyTorch, the semantics of one piece of
huyz2023/2by4-pretrain's 2:4 path, citing the reference file:line it follows.  It is the
checker the HIP kernels are compared against; nothing in the shipped package imports it.
Only the tests, the smoke entry point and the benchmark's CPU-baseline leg may use it.

Pinning status (what fixes each function independently of this file):
  prune24_mask           brute force over tie shapes vs the closed form "top-2 by (|x|, index)"
  encode24 / compress24  16-row truth table and the -4370 docstring vector of the reference
  cutlass_reorder_meta   PyTorch's own torch.sparse._semi_structured_conversions on pre-pruned input
  decompress24           round trip with compress24
  mvue24                 sum(p)=2, analytic inclusion probabilities, Monte-Carlo unbiasedness
  soft_threshold24       closed form (2nd smallest |a|), sort-based restatement on tie-free data
  transposable_mask      90-way fp64 brute force on exactly-summable data, row/column-sum invariants
  philox4x32_10          Random123's known-answer vectors
  masked_add             the reference's smoke vector [1, 1.06, 1, 1.12]
  adamw_masked_decay     step-1 closed forms, torch.optim.AdamW over several steps
  adamw_step_update      torch.optim.AdamW (amsgrad on/off) in phase 1, phase 1 at eps = 0 in phase 2, step-1 closed forms of Z
  gelu_glu_forward/_backward  torch's gelu(approximate='tanh') * x and autograd's gradient of it
  spmm_ref               dense masked fp32 product (definition); parity of the reference's CUTLASS
                         GEMM itself is unpinned (CUTLASS is an un-vendored, unpinned submodule)
"""
from .semi_structured import (  # noqa: F401
    prune24_mask, encode24, compress24, pack_meta, meta_dtype_for, cutlass_reorder_meta,
    cutlass_unreorder_meta, decompress24, sparse24_dense,
)
from .mvue import mvue24, mvue24_probabilities, mvue24_dense  # noqa: F401
from .soft_threshold import soft_threshold24  # noqa: F401
from .transposable import (  # noqa: F401
    transposable_patterns, transposable_mask, transposable_mask_bruteforce,
)
from .decay import masked_add  # noqa: F401
from .philox import philox4x32_10, mvue_uniforms  # noqa: F401
from .adamw import adamw_masked_decay  # noqa: F401
from .adamw_step import adamw_step_update, variance_change_statistic  # noqa: F401
from .gelu_glu import gelu_glu_forward, gelu_glu_backward  # noqa: F401
from .spmm import spmm_ref, spmm_ref_int, linear_ref  # noqa: F401
