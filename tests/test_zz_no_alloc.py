"""The entry point that allocates nothing, ``hstu_jagged_fwd_noalloc``: its workspace is a device array of the library.
Called through the C ABI, two calls in a row on one stream, the second with a smaller input, each compared bit for
bit with ``hstu_jagged_fwd`` given a workspace from torch's allocator (the split variant adds its fp32 partial outputs
in a fixed order, so the two agree to the bit, which is well inside the stated bf16 tolerance of 1e-2)."""

import ctypes

import pytest
import torch

from ops_rec import _native, _ops, workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def prepared(w):
    return _ops.prepare_forward(w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, w.max_seq_len,
                                w.silu_scale, w.seq_offset, w.seq_offset, w.num_context, w.num_target,
                                w.target_group_size, w.alpha)  # fmt: skip


def noalloc(p):
    lib = _native.load()
    stream = torch.cuda.current_stream(DEV).cuda_stream
    rc = lib.hstu_jagged_fwd_noalloc(ctypes.byref(p.params), ctypes.c_void_p(stream))
    assert rc == _native.HSTU_OK, _native.last_error()


@pytest.mark.parametrize(
    "first,second,variant",
    [
        # split items: counters and partial outputs in the scratch array; then a shorter sequence
        (dict(batch=2, heads=2, dim=128, lo=2800, hi=3000), dict(batch=1, heads=2, dim=128, lo=1500, hi=1500), "split"),
        # the same at the head-dim slot 64 (three workgroups per CU resident: more parts than at 128)
        (dict(batch=2, heads=2, dim=64, lo=2800, hi=3000), dict(batch=1, heads=2, dim=64, lo=1500, hi=1500), "split"),
        # per-XCD queues: counters in the scratch array; then a short plain list that needs none of it
        (dict(batch=48, heads=4, dim=128, lo=200, hi=2000), dict(batch=8, heads=4, dim=128, lo=100, hi=600), "queues"),
    ],
)
def test_noalloc_entry_point_matches_the_workspace_one(first, second, variant):
    for i, shape in enumerate((first, second)):
        w = workloads.make("x", dtype=torch.bfloat16, device=DEV, seed=5 + i, **shape)
        p = prepared(w)
        if i == 0:
            assert variant in p.kernel_name() and p.workspace_bytes > 0
            assert p.workspace_bytes <= _native.load().hstu_jagged_fwd_noalloc_max_workspace()
        want = p.launch().clone()
        torch.cuda.synchronize()
        p.out.fill_(float("nan"))
        noalloc(p)
        torch.cuda.synchronize()
        assert torch.equal(p.out, want), f"{variant}, call {i}: the two entry points differ"


def test_noalloc_entry_point_limits():
    """The scratch array is sized for the largest request a description can make today (the counter block plus one
    fp32 partial output of 128 x 128 per resident workgroup at two workgroups per CU), so the refusal with
    HSTU_ERR_WORKSPACE guards variants to come and cannot be provoked from here; what can be checked from the host is
    that a description is validated first and that the limit is what the header says."""
    lib = _native.load()
    assert lib.hstu_jagged_fwd_noalloc(None, None) == 161001
    assert lib.hstu_jagged_fwd_noalloc_max_workspace() == (32 << 20) + 16384
    # the largest workspace any forward description asks for fits: long single sequences at every slot with split items
    asked = []
    for dim in (32, 64, 128, 256):
        w = workloads.make("x", dtype=torch.bfloat16, device=DEV, batch=1, heads=1, dim=dim, lo=20480, hi=20480)
        asked.append(prepared(w).workspace_bytes)
    assert max(asked) == lib.hstu_jagged_fwd_noalloc_max_workspace(), asked
