"""CPU oracle for the fused attention-variant path.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the product: it may be imported by
`tests/`, by `__graft_entry__.smoke()` and by the `cpu_baseline` leg of `bench.py`, and only as the
checker / the baseline being timed.  The product path (`flashtensor_amd`) never imports it and fails
loudly when its HIP library is missing.

Each function restates, op for op and dtype for dtype, the eager PyTorch definition of one workload of
the reference (`cases/kernels/*.py`, `bench/{ea,sima}.mlir`) on CPU tensors; the docstrings cite the
lines they follow.  How each function is pinned (closed forms, library routines, fp64 brute force) is
listed in `oracle/cases.py`'s header and exercised by `tests/test_oracle_*.py`.
"""
from .cases import (  # noqa: F401
    attn_forward, h2o_forward, keyformer_forward, roco_forward, ea_forward, sima_forward,
    snapkv_forward, corm_forward, corm_mask_rule, corm_margin, gemma2_forward, attn2d_forward, attn_h2o2d_forward,
    ea_block_forward, sima_block_forward, prepare_block_inputs,
    prepare_inputs, prepare_exp_rand, heavy_hitters, roco_mean_var, chunked_over_heads,
)
from .noise import seeded_exp_rand, seeded_exp_rand_pairs, noise_u32, lowbias32  # noqa: F401
from .metrics import loss, topk_agreement  # noqa: F401
