"""Writes the committed fixtures under tests/golden/.

    python tests/golden/make_golden.py

Inputs are seeded and rebuilt by the tests from ``CASES``; expected outputs come from the scalar C
restatement (``oracle/hstu_bruteforce.c``, double accumulation).  The reference has no stored
vectors for this path and none of its code is imported here; the one case with reference
provenance is the closed-form input pattern of its C example
(hstu_forward_v1/examples/aclnn/test_aclnn_hstu_forward_jagged.cpp:52-63).
"""

import os
import sys

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(os.path.dirname(_HERE))
for _p in (os.path.join(_ROOT, "ops-rec_amd"), _ROOT, os.path.dirname(_HERE)):
    if _p not in sys.path:
        sys.path.insert(0, _p)

from ops_rec import workloads  # noqa: E402


def _c1():
    return workloads.config("C1")


def _ctx_tgt():
    return workloads.make("g", batch=3, heads=2, dim=32, lo=20, hi=70, dtype=torch.bfloat16, std=0.5, rab_std=0.2,
                          num_context=4, max_target=9, target_group_size=2, alpha=0.5, seed=21)  # fmt: skip


def _delta_gqa():
    from helpers import small_case

    return small_case(seed=22, batch=3, heads=4, heads_k=2, dim=32, dim_v=16, lo=5, hi=40, dtype=torch.float16,
                      std=0.5, delta=True, rab=True)  # fmt: skip


CASES = {"c1_fp32": _c1, "small_ctx_tgt_rab_bf16": _ctx_tgt, "small_delta_gqa_f16": _delta_gqa}


def main():
    from oracle import bruteforce

    for name, build in CASES.items():
        w = build()
        out = bruteforce.forward(w.q, w.k, w.v, **w.oracle_kwargs())
        np.savez_compressed(os.path.join(_HERE, f"{name}.npz"), out=out.numpy())
        print(name, tuple(out.shape))
    n, d = 4, 32
    q = (torch.arange(10 * n * d) % 3).float().div(3.0).view(10, n, d)
    k = (torch.arange(14 * n * d) % 5).float().div(5.0).view(14, n, d)
    v = (torch.arange(14 * n * d) % 7).float().div(7.0).view(14, n, d)
    out = bruteforce.forward(q, k, v, None, None, 0, 6, 8, 1.0 / 6, [0, 4, 10], [0, 6, 14], None, None, 0, 1.0)
    np.savez_compressed(os.path.join(_HERE, "aclnn_example_forward.npz"), out=out.numpy())
    print("aclnn_example_forward", tuple(out.shape), out[0, 0, :4].tolist())


if __name__ == "__main__":
    main()
