"""ln_mul on the GPU against the CPU oracle, through the registered operator (which calls ``ln_mul_fwd`` of the C ABI).

The shape matrix, the random inputs and the fp32 tolerance (rtol = atol = 1e-4) are those of the reference's test
(ascendc/activation/ln_mul/test/pytest/test_ln_mul.py:52-66); bf16 / fp16 inputs (not in the reference) are held to
one rounding step of the output type around the fp64 oracle value: rtol 2^-8 (bf16) / 2^-11 (fp16) plus the same
absolute floor.
"""

import ctypes

import numpy as np
import pytest
import torch

import ops_rec
from ops_rec import _native
from oracle import ln_mul_oracle as L

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: dict(rtol=1e-4, atol=1e-4), torch.bfloat16: dict(rtol=2.0**-8, atol=2e-3),
       torch.float16: dict(rtol=2.0**-11, atol=3e-4)}  # fmt: skip
ln_mul = ops_rec.ascendc.activation.ln_mul


def inputs(a, r, dtype, seed, affine_dtype=None):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(a, r, generator=g).to(dtype)
    u = torch.randn(a, r, generator=g).to(dtype)
    gamma = torch.randn(r, generator=g).to(affine_dtype or dtype)
    beta = torch.randn(r, generator=g).to(affine_dtype or dtype)
    return x, u, gamma, beta


def oracle(x, u, gamma, beta):
    f = lambda t: t.double().numpy()  # noqa: E731
    return L.ln_mul(f(x), f(u), f(gamma), f(beta))


def check(x, u, gamma, beta, expect_kernel=None):
    dev = [t.to(DEV) for t in (x, u, gamma, beta)]
    got = ln_mul(*dev)
    assert got.dtype == x.dtype and got.shape == x.shape and got.is_contiguous()
    np.testing.assert_allclose(got.double().cpu().numpy(), oracle(x, u, gamma, beta), **TOL[x.dtype])
    return got


@pytest.mark.parametrize("r", [1, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048])
def test_reference_shape_matrix_fp32(r):
    # test_ln_mul.py:52-54: a in 1..2048 by powers of two for every r
    for a in [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048]:
        check(*inputs(a, r, torch.float32, seed=a * 4096 + r))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("affine_f32", [False, True])
@pytest.mark.parametrize("r", [8, 16, 64, 104, 192, 384, 512, 768, 1000, 1024, 1536, 2048, 3072, 4096, 6144, 8192, 12288,
                               16384, 24576, 32768])
def test_sixteen_bit_rows(dtype, affine_f32, r):
    for a in (1, 3, 130):
        check(*inputs(a, r, dtype, seed=a + r, affine_dtype=torch.float32 if affine_f32 else None))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r", [1, 2, 3, 7, 100, 1001, 1022, 3001, 5002, 20000, 40004])
def test_rows_that_are_not_whole_chunks(dtype, r):
    # element-wise form of the kernel: any row length
    for a in (1, 5, 67):
        check(*inputs(a, r, dtype, seed=7 * a + r, affine_dtype=torch.float32))


@pytest.mark.parametrize("r", [96, 384, 768, 1536, 3072, 4096, 6144, 8192, 12288, 16384, 16388, 50000])
def test_more_row_lengths_fp32(r):
    check(*inputs(9, r, torch.float32, seed=r))


def test_many_short_rows():
    # more rows than one launch dimension of 65535 workgroups would hold
    x, u, gamma, beta = inputs(1 << 20, 32, torch.float32, seed=1)
    check(x, u, gamma, beta)
    x, u, gamma, beta = inputs((1 << 19) + 3, 64, torch.bfloat16, seed=2, affine_dtype=torch.float32)
    check(x, u, gamma, beta)


def test_pointers_that_are_only_element_aligned():
    # contiguous views that start 4 bytes into an allocation: no 16-byte chunks, the element-wise form must be taken
    a, r = 33, 512
    x, u, gamma, beta = inputs(a, r, torch.float32, seed=5)
    want = oracle(x, u, gamma, beta)
    store = torch.zeros(a * r + 1, device=DEV)
    store[1:] = x.to(DEV).flatten()
    x_dev = store[1:].view(a, r)
    assert x_dev.is_contiguous() and x_dev.data_ptr() % 16 == 4
    got = ln_mul(x_dev, u.to(DEV), gamma.to(DEV), beta.to(DEV))
    np.testing.assert_allclose(got.double().cpu().numpy(), want, rtol=1e-4, atol=1e-4)
    gstore = torch.zeros(r + 2, device=DEV)
    gstore[2:] = gamma.to(DEV)
    got = ln_mul(x.to(DEV), u.to(DEV), gstore[2:], beta.to(DEV))
    np.testing.assert_allclose(got.double().cpu().numpy(), want, rtol=1e-4, atol=1e-4)


def test_non_contiguous_inputs_are_made_contiguous():
    x, u, gamma, beta = inputs(40, 256, torch.float32, seed=6)
    xt = x.t().contiguous().to(DEV).t()  # same values, column-major storage
    ug = torch.zeros(40, 512)
    ug[:, ::2] = u
    got = ln_mul(xt, ug.to(DEV)[:, ::2], gamma.to(DEV), beta.to(DEV))
    np.testing.assert_allclose(got.double().cpu().numpy(), oracle(x, u, gamma, beta), rtol=1e-4, atol=1e-4)


def test_constant_rows_and_large_offsets():
    # a row of equal values has variance 0: out = beta * u exactly as far as fp32 carries it; a large common offset
    # must not leak into the variance (two-pass form, not E[x^2] - E[x]^2)
    r = 512
    _, u, gamma, beta = inputs(4, r, torch.float32, seed=8)
    x = torch.tensor([[0.0], [1.0], [-3.5], [1000.0]]).repeat(1, r)
    got = check(x, u, gamma, beta)
    np.testing.assert_allclose(got.cpu().numpy(), (beta * u).numpy(), rtol=1e-6, atol=1e-6)
    x2, u2, g2, b2 = inputs(16, r, torch.float32, seed=9)
    check(x2 + 4096.0, u2, g2, b2)


def test_full_size_layer_shape_properties():
    # the shape the attention output of the headline workload has as [tokens, heads * dim]: 20480 x 512 in bf16, and
    # 16 times as many tokens; checked through properties that need no CPU pass over the whole matrix, and a slice
    for a in (20480, 327680):
        x, u, gamma, beta = (t.to(DEV) for t in inputs(a, 512, torch.bfloat16, seed=a, affine_dtype=torch.float32))
        y = ln_mul(x, u, gamma, beta)
        assert torch.equal(ln_mul(x, u, gamma, beta), y)  # same bits every launch
        one, zero = torch.ones_like(gamma), torch.zeros_like(beta)
        n = ln_mul(x, torch.ones_like(u), one, zero).float()
        assert n.mean(dim=1).abs().max() < 2e-3 and ((n * n).mean(dim=1) - 1).abs().max() < 1e-2
        assert torch.count_nonzero(ln_mul(x, torch.zeros_like(u), gamma, beta)) == 0
        # rows are independent: a slice run alone gives the same bits, and matches the oracle
        rows = slice(a - 77, a)
        part = ln_mul(x[rows], u[rows], gamma, beta)
        assert torch.equal(part, y[rows])
        want = oracle(x[rows].cpu(), u[rows].cpu(), gamma.cpu(), beta.cpu())
        np.testing.assert_allclose(part.double().cpu().numpy(), want, **TOL[torch.bfloat16])


def test_adapter_rejects_bad_arguments():
    x, u, gamma, beta = (t.to(DEV) for t in inputs(4, 8, torch.float32, seed=3))
    for args, msg in [
        ((x[0], u, gamma, beta), "x should be 2D"),
        ((x, u[0], gamma, beta), "u should be 2D"),
        ((x, u, gamma[None], beta), "gamma should be 1D"),
        ((x, u, gamma, beta[None]), "beta should be 1D"),
        ((x, u[:2], gamma, beta), "identical shape"),
        ((x[:0], u[:0], gamma, beta), "x tensor must be non-empty"),
        ((x, u, gamma[:4], beta), "x.size\\(1\\) elements"),
        ((x, u.half(), gamma, beta), "same dtype"),
        ((x, u, gamma.half(), beta.half()), "float32 or both of the dtype of x"),
        ((x.double(), u.double(), gamma, beta), "unsupported dtype"),
        ((x, u, gamma.cpu(), beta), "gamma tensor must be on the GPU"),
    ]:
        with pytest.raises(RuntimeError, match=msg):
            ln_mul(*args)


def test_raw_c_abi_call_on_a_side_stream():
    # the entry point as a non-torch caller would use it: plain pointers, an explicit stream
    x, u, gamma, beta = (t.to(DEV) for t in inputs(300, 768, torch.float32, seed=4))
    out = torch.full_like(x, float("nan"))
    p = _native.new_ln_mul_params()
    p.x, p.u, p.gamma, p.beta, p.out = (t.data_ptr() for t in (x, u, gamma, beta, out))
    p.rows, p.cols = 300, 768
    p.dtype = p.affine_dtype = _native.DT_FP32
    p.epsilon = 1e-5
    s = torch.cuda.Stream(device=DEV)
    s.wait_stream(torch.cuda.current_stream())
    lib = _native.load()
    assert lib.ln_mul_fwd_kernel_name(ctypes.byref(p)).decode() == "ln_mul_f32_g64_v3"
    assert lib.ln_mul_fwd(ctypes.byref(p), ctypes.c_void_p(s.cuda_stream)) == 0
    s.synchronize()
    np.testing.assert_allclose(out.double().cpu().numpy(), oracle(x.cpu(), u.cpu(), gamma.cpu(), beta.cpu()),
                               rtol=1e-4, atol=1e-4)  # fmt: skip
    # another epsilon than the reference's is honoured
    p.epsilon = 0.5
    assert lib.ln_mul_fwd(ctypes.byref(p), ctypes.c_void_p(s.cuda_stream)) == 0
    s.synchronize()
    f = lambda t: t.double().cpu().numpy()  # noqa: E731
    np.testing.assert_allclose(f(out), L.ln_mul(f(x), f(u), f(gamma), f(beta), eps=0.5), rtol=1e-4, atol=1e-4)
