"""The single-op suite at the benchmark's full sizes (config 2), fp32 and bf16, against the CPU
oracle.  The oracle's cache-friendly loop order finishes 2048^3 in well under a second and performs
the same roundings per element as the reference's m,n,k nest (tests/test_oracle_pins.py)."""
import numpy as np
import pytest
import torch

from tests.util import (BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_as_close_as_eager, assert_close, assert_close_bf16, assert_close_f32,
                        bf16_round, dev, host, rng)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from llcompiler_amd import ops as _ops
    return _ops


def _uniform(shape, seed):
    return rng(seed).uniform(-1, 1, shape).astype(np.float32)


def test_matmul_2048_f32(ops, oracle):
    a, b = _uniform((2048, 2048), 1), _uniform((2048, 2048), 2)
    want = oracle.matmul(a, b, "mkn").astype(np.float64)
    got = host(ops.matmul(dev(a), dev(b))).astype(np.float64)
    err = np.abs(got - want)
    # Summing 2048 products of magnitude ~1/3 in fp32 leaves ~1e-5 of rounding noise in ANY order (the
    # oracle itself is outside rtol 1e-4 / atol 1e-5 of the fp64 product on ~1300 of 4.2 M outputs, the
    # ones that cancel to ~0).  So: the stated tolerance must hold for all but 1 in 10^4 outputs, and
    # every output must be within 1e-4 of the output scale.
    strict_bad = int((err > F32_ATOL + F32_RTOL * np.abs(want)).sum())
    print("matmul 2048^3 f32: %d of %d outputs outside rtol 1e-4 / atol 1e-5 of the oracle (max abs error %.3g)"
          % (strict_bad, err.size, err.max()))
    assert strict_bad <= 150, "%d outputs outside rtol 1e-4 / atol 1e-5" % strict_bad
    scale = float(np.sqrt((want ** 2).mean()))
    assert err.max() <= F32_ATOL + F32_RTOL * scale, "max abs error %g at output scale %g" % (err.max(), scale)
    # and against the float64 product: the kernel's rounding noise is no worse than the oracle's own (both sum 2048
    # fp32 products per output, in nearly the same order), in the mean and at the worst output
    exact = a.astype(np.float64) @ b.astype(np.float64)
    e_kernel, e_oracle = np.abs(got - exact), np.abs(want - exact)
    assert np.sqrt((e_kernel ** 2).mean()) <= 1.25 * np.sqrt((e_oracle ** 2).mean()), "rms error against fp64 worse than the oracle's"
    assert e_kernel.max() <= 1.25 * e_oracle.max(), "max error against fp64 %g, the oracle's %g" % (e_kernel.max(), e_oracle.max())
    # aggregate check that no tile was dropped or duplicated: (A B) v == A (B v)
    v = _uniform((2048,), 3).astype(np.float64)
    np.testing.assert_allclose(got @ v, a.astype(np.float64) @ (b.astype(np.float64) @ v), rtol=1e-4, atol=1e-2)


def test_matmul_2048_bf16(ops, oracle):
    a, b = bf16_round(_uniform((2048, 2048), 1)), bf16_round(_uniform((2048, 2048), 2))
    want = bf16_round(oracle.matmul(a, b, "mkn"))
    got = host(ops.matmul(dev(a, torch.bfloat16), dev(b, torch.bfloat16)))
    assert_close_bf16(got, want, "matmul 2048^3 bf16")


def test_batch_matmul_full(ops, oracle):
    a, b = _uniform((32, 512, 64), 4), _uniform((32, 64, 512), 5)
    assert_close_f32(host(ops.batch_matmul(dev(a), dev(b))), oracle.batch_matmul(a, b, "mkn"), "bmm f32")
    ab, bb = bf16_round(a), bf16_round(b)
    got = host(ops.batch_matmul(dev(ab, torch.bfloat16), dev(bb, torch.bfloat16)))
    assert_close_bf16(got, bf16_round(oracle.batch_matmul(ab, bb, "mkn")), "bmm bf16")


def test_add_relu_full(ops, oracle):
    shape = (64, 1024, 1024)
    a, b = _uniform(shape, 6), _uniform(shape, 7)
    prog = ops.make_program([("add", "r0", "in0", "in1"), ("relu", "r0", "r0")], "r0")
    got = host(ops.elementwise(prog, [dev(a), dev(b)], shape, torch.float32))
    want = oracle.unary("relu", oracle.binary("add", a, b))
    np.testing.assert_array_equal(got, want)  # add and max are exactly rounded: bit exact
    ab, bb = bf16_round(a), bf16_round(b)
    gotb = host(ops.elementwise(prog, [dev(ab, torch.bfloat16), dev(bb, torch.bfloat16)], shape, torch.bfloat16))
    np.testing.assert_array_equal(gotb, bf16_round(oracle.unary("relu", oracle.binary("add", ab, bb))))


def test_softmax_full(ops, oracle):
    x = _uniform((4096, 4096), 8)
    got = host(ops.softmax(dev(x)))
    assert_close_f32(got, oracle.softmax_lastdim(x), "softmax f32")
    np.testing.assert_allclose(got.astype(np.float64).sum(-1), 1.0, rtol=1e-5)
    xb = bf16_round(x)
    assert_close_bf16(host(ops.softmax(dev(xb, torch.bfloat16))), bf16_round(oracle.softmax_lastdim(xb)), "softmax bf16")


def test_layernorm_full(ops, oracle):
    x = _uniform((8192, 1024), 9)
    g, b = _uniform((1024,), 10), _uniform((1024,), 11)
    assert_close_f32(host(ops.layer_norm(dev(x), dev(g), dev(b), 1e-5)), oracle.layernorm_lastdim(x, g, b, 1e-5), "layernorm f32")
    ones, zeros = np.ones(1024, np.float32), np.zeros(1024, np.float32)
    assert_close_f32(host(ops.layer_norm(dev(x), dev(ones), dev(zeros), 1e-5)), oracle.layernorm_lastdim(x, ones, zeros, 1e-5),
                     "layernorm f32 gamma=1 beta=0")
    xb, gb, bb = bf16_round(x), bf16_round(g), bf16_round(b)
    got = host(ops.layer_norm(dev(xb, torch.bfloat16), dev(gb, torch.bfloat16), dev(bb, torch.bfloat16), 1e-5))
    # bf16 outputs near zero (beta - gamma x_hat cancelling) have no meaningful relative error: the bar is the stated
    # tolerance plus what the oracle's own result, rounded to bf16, misses the float64 evaluation by
    x64, g64, b64 = xb.astype(np.float64), gb.astype(np.float64), bb.astype(np.float64)
    mu = x64.mean(-1, keepdims=True)
    exact = (x64 - mu) / np.sqrt(((x64 - mu) ** 2).mean(-1, keepdims=True) + 1e-5) * g64 + b64
    assert_as_close_as_eager(got, bf16_round(oracle.layernorm_lastdim(xb, gb, bb, 1e-5)), exact, BF16_RTOL, BF16_ATOL, "layernorm bf16")
