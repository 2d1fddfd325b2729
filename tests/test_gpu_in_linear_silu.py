"""in_linear_silu on the GPU against the CPU oracle, through the registered operator (``in_linear_silu_fwd`` of the
C ABI underneath).

Shapes, inputs (integers in [-100, 100] for x, Xavier-uniform weights, bias of ones) and tolerances (fp16 1e-3, bf16
5e-3, absolute and relative) are those of the reference's test
(ascendc/activation/in_linear_silu/in_linear_silu_forward/test/pytest/test_in_linear_silu.py:62-135).  On top of
them, every case is compared with the oracle's statement of the kernel's rounding points (one rounding of mixed, SiLU
of the rounded value): there the only freedom left is the fp32 summation, so all but a few elements must agree bit for
bit and none may be more than one rounding step away.
"""

import ctypes

import pytest
import torch

import ops_rec
from ops_rec import _native
from oracle import in_linear_silu_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float16: 1e-3, torch.bfloat16: 5e-3}
ULP = {torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}
op = ops_rec.ascendc.activation.distance_in_linear_silu


def reference_inputs(m, n, k, dtype, seed, bias_value=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randint(-100, 101, (m, k), generator=g).to(dtype)
    bound = (6.0 / (n + k)) ** 0.5  # xavier_uniform_ of an [n, k] matrix
    w = ((torch.rand(n, k, generator=g) * 2 - 1) * bound).to(dtype)
    bias = torch.full((n,), bias_value, dtype=torch.float32)
    return x, w, bias


def check(x, w, bias, split):
    dtype = x.dtype
    got = op(x.to(DEV), w.to(DEV), bias.to(DEV) if bias is not None else None, split)
    assert [tuple(t.shape) for t in got] == [(x.shape[0], s) for s in split] + [(x.shape[0], w.shape[0])]
    assert all(t.dtype == dtype and t.is_contiguous() for t in got)
    exact = O.in_linear_silu(x, w, bias, split)
    stated = O.in_linear_silu(x, w, bias, split, round_to=dtype)
    names = ("user", "value", "query", "key", "linear_output")
    for name, g, e, st in zip(names, got, exact, stated):
        g64 = g.double().cpu()
        assert torch.isfinite(g64).all(), name
        # the reference's tolerance, against a golden with the reference golden's rounding points (its addmm and silu
        # run in the 16-bit type: one rounding each, test_in_linear_silu.py:36-39)
        # An element whose exact value sits on a rounding boundary can fall to the other side under another fp32
        # summation order, and one step of the type exceeds this tolerance for values in [2, 5): such flips are
        # bounded to one step below and may be at most 1 element in 100 000 (or 2 elements) here.
        outside = (g64 - st).abs() > TOL[dtype] + TOL[dtype] * st.abs()
        assert int(outside.sum()) <= max(2, outside.numel() // 100000), (name, int(outside.sum()))
        # and against the exact value: the two roundings together stay within a step and a half of the type
        torch.testing.assert_close(g64, e, rtol=1.5 * ULP[dtype], atol=TOL[dtype], msg=lambda m_: f"{name} (exact): {m_}")

    def one_step(name, g64, want, slack=0.0):
        # at most one step of the 16-bit type away (plus `slack`), and almost always equal
        step = ULP[dtype] * torch.clamp(want.abs(), min=2.0**-14)
        assert ((g64 - want).abs() <= 1.001 * step + slack).all(), name
        assert (g64 != want).double().mean().item() < 0.02, (name, (g64 != want).double().mean().item())

    # the kernel's rounding points.  linear_output: the exact sum rounded once (the fp32 summation is the only freedom).  The splits: SiLU of the kernel's own rounded linear_output, rounded once.
    # Where the terms cancel, the fp32 sum is off by more than a step of the small result: the classic bound
    # (k + 1) * 2^-24 * (|x| @ |w|^T + |bias|) on the sum is allowed on top of the step.
    lin = got[4].double().cpu()
    mass = x.double().abs() @ w.double().abs().t() + (bias.double().abs() if bias is not None else 0.0)
    one_step("linear_output", lin, O.in_linear_silu(x, w, bias, split, round_to=dtype)[4],
             slack=mass * (x.shape[1] + 1) * 2.0**-24)  # fmt: skip
    act = (lin / (1.0 + torch.exp(-lin))).float().to(dtype).double()
    one_step("splits", torch.cat([g.double().cpu() for g in got[:4]], dim=1), act)
    return got


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [
    (2789, 9216, 64), (3677, 9216, 64),                      # test_in_linear_silu (ci)
    (256, 1024, 16), (512, 1024, 32), (2048, 1024, 64),      # test_in_linear_silu_normal
    (256, 4096, 64), (512, 9216, 16), (256, 16384, 32),
    (2561, 1024, 64), (2561, 1024, 128), (2561, 1024, 256),  # test_in_linear_silu_diff_dim
    (1204, 4096, 128),
])  # fmt: skip
def test_reference_shapes(dtype, m, n, k):
    quarter = n // 4
    split = [quarter] * 4 if (m % 2 == 0) else [quarter - 16, quarter - 16, quarter + 16, quarter + 16]
    check(*reference_inputs(m, n, k, dtype, seed=m + n + k), split)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_common_input(dtype):
    # get_common_input: m = 100, n = 64, k = 16, the smallest legal problem (one partial tile in every direction)
    check(*reference_inputs(100, 64, 16, dtype, seed=1), [16, 16, 16, 16])


@pytest.mark.parametrize("m,n,k,split", [
    (1, 64, 16, [16, 16, 16, 16]),
    (127, 192, 48, [16, 64, 32, 80]),       # k not a multiple of the k step: the last step is half empty
    (129, 320, 80, [64, 64, 64, 128]),      # k = 2.5 steps, n = 2.5 tiles
    (300, 2048, 512, [512, 512, 512, 512]),  # the layer shape of the headline workload (embedding 512, 4 x 512 out)
    (77, 3072, 768, [768, 768, 768, 768]),
    (40, 8192, 2048, [2048] * 4),
    (33, 32768, 8192, [8192] * 4),           # the largest legal k and n
    (200, 1024, 240 + 16, [256] * 4),
    (333, 4096, 1024, [1024, 1008, 1040, 1024]),  # 128 x 256 tiles: partial tiles in m, split edges inside a tile
    (130, 4096 + 64, 1040, [1040, 1040, 1040, 1040]),  # ... and a last n tile of 64 columns, k = 32.5 steps
    (4100, 1024, 256, [256] * 4),  # m tiles dealt to the XCDs in groups of 8 (small weights, m >= 4096): 33 m tiles
    (4230, 2048, 128, [512, 496, 528, 512]),
])  # fmt: skip
def test_edges_and_long_k(m, n, k, split):
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / k**0.5).to(torch.bfloat16)
    bias = torch.randn(n, generator=g)
    check(x, w, bias, split)


def test_every_output_column_names_its_weight_row():
    # one-hot x rows and weight[j, i] = (j % 64) + i / 16 (exact in fp16): each output element tells which weight row,
    # which k and which split made it; covers the permuted placement of weight rows in LDS and the split boundaries
    k, split = 64, [16, 112, 64, 64]
    n = sum(split)
    x = torch.eye(k).repeat(3, 1)[:150].to(torch.float16)
    w = ((torch.arange(n) % 64)[:, None] + torch.arange(k)[None, :] / 16.0).to(torch.float16)
    assert torch.equal(w.float(), (torch.arange(n) % 64)[:, None] + torch.arange(k)[None, :] / 16.0)
    got = check(x, w, torch.zeros(n), split)
    lin = got[4].float().cpu()
    rows = torch.arange(150) % k
    want = (torch.arange(n) % 64)[None, :] + rows[:, None] / 16.0
    assert torch.equal(lin, want)


def test_no_bias_through_the_c_abi_on_a_side_stream():
    m, n, k, split = 500, 1024, 64, [256] * 4
    x, w, _ = reference_inputs(m, n, k, torch.float16, seed=9)
    xd, wd = x.to(DEV), w.to(DEV)
    outs = [torch.full((m, s), float("nan"), dtype=x.dtype, device=DEV) for s in split + [n]]
    p = _native.new_in_linear_silu_params()
    p.x, p.weight, p.bias = xd.data_ptr(), wd.data_ptr(), None
    p.user, p.value, p.query, p.key, p.linear_output = (t.data_ptr() for t in outs)
    p.m, p.n, p.k = m, n, k
    for i, s in enumerate(split):
        p.split[i] = s
    p.dtype = _native.DT_FP16
    s_ = torch.cuda.Stream(device=DEV)
    s_.wait_stream(torch.cuda.current_stream())
    lib = _native.load()
    assert lib.in_linear_silu_fwd_kernel_name(ctypes.byref(p)).decode() == "in_linear_silu_f16_stages2_tile128"
    assert lib.in_linear_silu_fwd(ctypes.byref(p), ctypes.c_void_p(s_.cuda_stream)) == 0
    s_.synchronize()
    want = O.in_linear_silu(x, w, None, split, round_to=torch.float16)
    for g, t in zip(outs, want):
        # the reference's fp16 tolerance (the fp32 summation error where terms of size 7 cancel is a few 1e-4)
        torch.testing.assert_close(g.double().cpu(), t, rtol=1e-3, atol=1e-3)


def test_repeated_launches_give_the_same_bits():
    x, w, b = (t.to(DEV) for t in reference_inputs(3001, 4096, 128, torch.bfloat16, seed=2))
    a1 = op(x, w, b, [1024] * 4)
    a2 = op(x, w, b, [1024] * 4)
    assert all(torch.equal(p, q) for p, q in zip(a1, a2))


def test_full_size_properties():
    # m = the headline workload's token count, embedding 512 -> 4 x 512: checked through properties and a row slice
    m, n, k, split = 20292, 2048, 512, [512] * 4
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn(m, k, generator=g, device=DEV).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g, device=DEV) / k**0.5).to(torch.bfloat16)
    b = torch.randn(n, generator=g, device=DEV)
    user, value, query, key, lin = op(x, w, b, split)
    # the four outputs are SiLU of the matching columns of linear_output, bit for bit
    z = lin.float()
    act = (z / (1.0 + torch.exp(-z))).to(torch.bfloat16)
    cat = torch.cat([user, value, query, key], dim=1)
    assert (cat != act).float().mean().item() < 1e-3  # __expf against exp: a last-bit difference now and then
    torch.testing.assert_close(cat.float(), act.float(), rtol=2.0**-7, atol=1e-6)
    # rows are independent: a slice run alone gives the same bits, and matches the oracle
    rows = slice(m - 200, m)
    part = op(x[rows], w, b, split)
    assert torch.equal(part[4], lin[rows]) and torch.equal(part[2], query[rows])
    want = O.in_linear_silu(x[rows].cpu(), w.cpu(), b.cpu(), split, round_to=torch.bfloat16)
    step = 2.0**-7 * torch.clamp(want[4].abs(), min=2.0**-14)
    assert ((part[4].double().cpu() - want[4]).abs() <= 1.001 * step).all()


def test_adapter_rejects_bad_arguments():
    x, w, b = (t.to(DEV) for t in reference_inputs(100, 64, 16, torch.float16, seed=1))
    for args, msg in [
        ((x, w, b, [16, 17, 15, 16]), "multiples of 16"),     # test_invalid_split_args
        ((x, w, b, [16, 16, 32, 32]), "sum\\(splitList\\)"),
        ((x, w, b, [16, 16, 32]), "4 elements"),
        ((x, w, x.clone(), [16] * 4), "bias must be 1D"),      # test_invalid_bias
        ((x, w, b[:32], [16] * 4), "bias dim\\[0\\]"),
        ((x[0], w, b, [16] * 4), "x must be 2D"),
        ((x, w[:, :8], b, [16] * 4), "weight dim\\[1\\]"),
        ((x.float(), w.float(), b, [16] * 4), "float16 or bfloat16"),
        ((x, w.bfloat16(), b, [16] * 4), "dtype of x"),
        ((x, w, b.half(), [16] * 4), "bias must be float32"),
        ((x[:0], w, b, [16] * 4), "x tensor must be non-empty"),
    ]:
        with pytest.raises(RuntimeError, match=msg):
            op(*args)
    # n must be a multiple of 4 k (in_linear_silu_plugin.cpp:59)
    x2 = torch.zeros(4, 32, dtype=torch.float16, device=DEV)
    w2 = torch.zeros(64, 32, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 4 x dim"):
        op(x2, w2, b, [16] * 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_autograd_through_the_operator(dtype):
    # loss.backward() through distance_in_linear_silu -> in_linear_silu_backward, against the oracle's backward
    m, n, k, split = 257, 512, 128, [64, 192, 128, 128]
    g = torch.Generator().manual_seed(4)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = (torch.randn(n, k, generator=g) / k**0.5).to(dtype)
    b = torch.randn(n, generator=g)
    xd, wd, bd = (t.to(DEV).requires_grad_() for t in (x, w, b))
    outs = ops_rec.ascendc.activation.in_linear_silu(xd, wd, bd, split)
    grads = [torch.randn(m, s, generator=g).to(dtype) for s in split]
    loss = sum((o.float() * gr.to(DEV).float()).sum() for o, gr in zip(outs[:4], grads))
    loss.backward()
    dx, dw, db = O.in_linear_silu_backward(x, w, grads, outs[4].detach().cpu())
    tol = 2e-2 if dtype == torch.bfloat16 else 4e-3
    for got, want in ((xd.grad, dx), (wd.grad, dw), (bd.grad, db)):
        scale = want.abs().max().item()
        torch.testing.assert_close(got.double().cpu(), want, rtol=tol, atol=tol * scale)
    assert xd.grad.dtype == dtype and wd.grad.dtype == dtype and bd.grad.dtype == torch.float32


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,split", [(1, [16, 16, 16, 16]), (63, [16, 48, 32, 32]), (200, [512, 496, 528, 512]),
                                     (1000, [2304] * 4), (4097, [256, 128, 64, 64])])  # fmt: skip
def test_backward_silu_stage_through_the_c_abi(dtype, m, split):
    # in_linear_silu_bwd_dmixed: d_mixed = cat(grads) * silu'(linear_output) and its column sums, against the oracle;
    # d_mixed within one rounding step of the type, the sums within the fp32 summation error of m terms
    from ops_rec import _activation

    n = sum(split)
    g = torch.Generator().manual_seed(m + n)
    lin = (torch.randn(m, n, generator=g) * 2).to(dtype)
    grads = [torch.randn(m, s, generator=g).to(dtype) for s in split]
    lin_d, grads_d = lin.to(DEV), [t.to(DEV) for t in grads]
    d_mixed, sums = _activation.silu_backward_stage(lin_d, grads_d, split)
    want = O.silu_backward_stage(grads, lin)
    got = d_mixed.double().cpu()
    step = ULP[dtype] * torch.clamp(want.abs(), min=2.0**-14)
    assert ((got - want).abs() <= 0.51 * step + 1e-7).all()
    want_sums = want.sum(dim=0)
    mass = want.abs().sum(dim=0)
    assert ((sums.double().cpu() - want_sums).abs() <= mass * 2.0**-20 + 1e-6).all()
    # the same bits on a second launch (no atomics), and no bias gradient when none is wanted
    d2, s2 = _activation.silu_backward_stage(lin_d, grads_d, split)
    assert torch.equal(d2, d_mixed) and torch.equal(s2, sums)
    d3, s3 = _activation.silu_backward_stage(lin_d, grads_d, split, want_bias_grad=False)
    assert s3 is None and torch.equal(d3, d_mixed)
