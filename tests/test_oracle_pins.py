"""Pins the CPU oracle: the reference's own known answers, torch eager (the comparator the
reference's python tests use, llcompiler/test_models/utility.py:18-28), closed forms and brute
force.  Each check is chosen so that a plausible slip (transposed operand, wrong pad order, wrong
reduce init, dropped term) fails it."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

RTOL = ATOL = 1e-5  # the reference's own bar (utility.py:18-21)


def rng(seed):
    return np.random.default_rng(seed)


# ---- the two numeric goldens in the reference's runner tests ----
def test_golden_abs(oracle):
    # test/RunnerTest/abs.mlir:5-10
    np.testing.assert_array_equal(oracle.golden_abs(), np.array([1.0, 1.0], np.float32))


def test_golden_i64_mul_to_f32(oracle):
    # test/RunnerTest/mlir-runner.mlir:11-25
    np.testing.assert_array_equal(oracle.golden_i64_mul_to_f32(), np.array([4.0], np.float32))


# ---- shape known answers from test/Dialect/LLH/symbol_infer/infer_symbol_shape.mlir ----
def test_shape_goldens_conv_static(oracle):
    # :181-186  2x3x224x224 (*) 64x3x7x7, dil (2,3), pad (3,2,3,2), stride (2,1) -> 2x64x109x210
    x = np.zeros((2, 3, 224, 224), np.float32)[:, :, :, :]
    oh = oracle.window_out(224, 3, 3, 2, 7, 2)
    ow = oracle.window_out(224, 2, 2, 3, 7, 1)
    assert (oh, ow) == (109, 210)
    y = oracle.conv2d(x[:1, :, :40, :40], np.zeros((4, 3, 7, 7), np.float32), pad=(3, 2, 3, 2), stride=(2, 1),
                      dilation=(2, 3))
    assert y.shape == (1, 4, oracle.window_out(40, 3, 3, 2, 7, 2), oracle.window_out(40, 2, 2, 3, 7, 1))


def test_shape_goldens_maxpool_static(oracle):
    # :73-78  2x64x9x17, k7, dil (2,1), pad (3,1,3,1), stride 2 -> 2x64x2x7
    y = oracle.maxpool2d(np.zeros((2, 64, 9, 17), np.float32), (7, 7), pad=(3, 1, 3, 1), stride=(2, 2),
                         dilation=(2, 1))
    assert y.shape == (2, 64, 2, 7)


def test_shape_golden_dynamic_conv_map(oracle):
    # :166 annotates the dynamic k7 p3 s2 d1 case with (s0 - 1) ceildiv 2 + 1, while the static rule
    # (LLHinfersymbolShape.cpp:265-266) and torch divide with floor.  The two agree where s0 - 1 is
    # even; run-time extents come from torch (out_put_call.py:154-170), so floor is the semantics.
    for s in (7, 31, 225):
        assert oracle.window_out(s, 3, 3, 1, 7, 2) == -(-(s - 1) // 2) + 1
    for s in (8, 224):
        assert oracle.window_out(s, 3, 3, 1, 7, 2) == (s - 1) // 2 + 1
        assert F.conv2d(torch.zeros(1, 1, s, s), torch.zeros(1, 1, 7, 7), stride=2, padding=3).shape[-1] == (s - 1) // 2 + 1


def test_shape_goldens_matmul_bmm_reduce(oracle):
    # :133-135, :212-214, :266-268
    assert oracle.matmul(np.zeros((5, 512), np.float32), np.zeros((512, 10), np.float32)).shape == (5, 10)
    assert oracle.batch_matmul(np.zeros((12, 5, 512), np.float32), np.zeros((12, 512, 10), np.float32)).shape == (12, 5, 10)
    assert oracle.reduce("sum", np.zeros((3, 3, 4, 5), np.float32), [1, 2]).shape == (3, 5)


# ---- contractions ----
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 3, 3), (7, 5, 11), (33, 65, 129)])
def test_matmul_vs_torch_and_orders(oracle, M, N, K):
    r = rng(M * 100 + N * 10 + K)
    a = r.uniform(-1, 1, (M, K)).astype(np.float32)
    b = r.uniform(-1, 1, (K, N)).astype(np.float32)
    c = oracle.matmul(a, b)
    ref64 = (a.astype(np.float64) @ b.astype(np.float64))
    np.testing.assert_allclose(c, ref64, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(c, torch.mm(torch.from_numpy(a), torch.from_numpy(b)).numpy(), rtol=RTOL, atol=ATOL)
    # the cache-friendly loop order performs the same roundings per element
    np.testing.assert_array_equal(c, oracle.matmul(a, b, "mkn"))
    np.testing.assert_allclose(oracle.matmul(a, b, "f64"), ref64.astype(np.float32), rtol=0, atol=0)


def test_matmul_non_symmetric_catches_transpose(oracle):
    a = np.array([[1, 2, 3], [4, 5, 6]], np.float32)  # 2x3
    b = np.array([[1, 0], [0, 1], [2, 3]], np.float32)  # 3x2
    np.testing.assert_array_equal(oracle.matmul(a, b), np.array([[7, 11], [16, 23]], np.float32))


def test_matmul_is_sequential_fp32_sum(oracle):
    # 2^24 + 1 + 1 ... in fp32 stays 2^24 when summed in k order; a pairwise or fp64 sum would not
    K = 9
    a = np.ones((1, K), np.float32)
    b = np.ones((K, 1), np.float32)
    a[0, 0] = 2.0 ** 24
    assert oracle.matmul(a, b)[0, 0] == np.float32(2.0 ** 24)
    assert oracle.matmul(a, b, "f64")[0, 0] == np.float32(2.0 ** 24 + 8)


def test_batch_matmul_vs_torch(oracle):
    r = rng(5)
    a = r.uniform(-1, 1, (3, 9, 6)).astype(np.float32)
    b = r.uniform(-1, 1, (3, 6, 4)).astype(np.float32)
    want = torch.bmm(torch.from_numpy(a), torch.from_numpy(b)).numpy()
    np.testing.assert_allclose(oracle.batch_matmul(a, b), want, rtol=RTOL, atol=ATOL)
    np.testing.assert_array_equal(oracle.batch_matmul(a, b), oracle.batch_matmul(a, b, "mkn"))


CONV_CASES = [
    # N, C, H, W, F, KH, KW, pad(h,w), stride, dil, group
    (2, 3, 9, 11, 4, 3, 3, (1, 1), (1, 1), (1, 1), 1),
    (1, 3, 17, 13, 5, 7, 7, (3, 3), (2, 2), (1, 1), 1),
    (2, 4, 10, 12, 6, 3, 2, (2, 0), (2, 1), (1, 2), 2),
    (1, 6, 8, 8, 6, 3, 3, (1, 2), (1, 3), (2, 1), 6),
    (1, 8, 5, 7, 3, 1, 1, (0, 0), (2, 2), (1, 1), 1),
    (3, 3, 12, 12, 2, 5, 5, (2, 2), (1, 1), (1, 1), 1),  # test_models/ops/conv.py:6-24 shape class
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_vs_torch(oracle, case):
    N, C, H, W, Fo, KH, KW, p, s, d, g = case
    r = rng(hash(case) % 1000)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = r.standard_normal((Fo, C // g, KH, KW)).astype(np.float32)
    b = r.standard_normal(Fo).astype(np.float32)
    want = F.conv2d(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b), stride=s, padding=p,
                    dilation=d, groups=g).numpy()
    got = oracle.conv2d(x, w, b, pad=(p[0], p[1], p[0], p[1]), stride=s, dilation=d, group=g)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
    want_nb = F.conv2d(torch.from_numpy(x), torch.from_numpy(w), None, stride=s, padding=p, dilation=d,
                       groups=g).numpy()
    np.testing.assert_allclose(oracle.conv2d(x, w, None, pad=(p[0], p[1], p[0], p[1]), stride=s, dilation=d,
                                             group=g), want_nb, rtol=1e-4, atol=1e-5)


def test_conv2d_asymmetric_pad_order(oracle):
    # pad = (h_lo, w_lo, h_hi, w_hi): compare with explicit zero padding
    r = rng(11)
    x = r.standard_normal((1, 2, 6, 7)).astype(np.float32)
    w = r.standard_normal((3, 2, 3, 3)).astype(np.float32)
    pad = (2, 0, 1, 3)
    xp = F.pad(torch.from_numpy(x), (pad[1], pad[3], pad[0], pad[2]))
    want = F.conv2d(xp, torch.from_numpy(w)).numpy()
    np.testing.assert_allclose(oracle.conv2d(x, w, None, pad=pad), want, rtol=1e-4, atol=1e-5)


def test_conv2d_delta_kernel_is_shift(oracle):
    # a one-hot kernel at (kh,kw) picks x[oh+kh-ph, ow+kw-pw]: catches correlation/convolution flips
    x = np.arange(1 * 1 * 5 * 6, dtype=np.float32).reshape(1, 1, 5, 6)
    w = np.zeros((1, 1, 3, 3), np.float32)
    w[0, 0, 0, 2] = 1.0
    y = oracle.conv2d(x, w, None, pad=(1, 1, 1, 1))
    want = np.zeros_like(x)
    want[0, 0, 1:, :-1] = x[0, 0, :-1, 1:]
    np.testing.assert_array_equal(y, want)


# ---- elementwise ----
def test_unary_vs_torch(oracle):
    r = rng(3)
    x = r.uniform(-4, 4, 4099).astype(np.float32)
    t = torch.from_numpy(x)
    exact = {"abs": torch.abs(t), "relu": torch.relu(t), "neg": -t}
    for k, v in exact.items():
        np.testing.assert_array_equal(oracle.unary(k, x), v.numpy())
    pos = np.abs(x) + 0.1
    tp = torch.from_numpy(pos)
    np.testing.assert_array_equal(oracle.unary("sqrt", pos), np.sqrt(pos))  # IEEE correctly rounded
    np.testing.assert_allclose(oracle.unary("sqrt", pos), torch.sqrt(tp).numpy(), rtol=RTOL, atol=ATOL)
    close = {"exp": (x, torch.exp(t)), "rsqrt": (pos, torch.rsqrt(tp)), "gelu": (x, F.gelu(t)),
             "tanh": (x, torch.tanh(t)), "erf": (x, torch.erf(t)), "sigmoid": (x, torch.sigmoid(t)),
             "log": (pos, torch.log(tp)), "recip": (pos, 1.0 / tp)}
    for k, (inp, v) in close.items():
        np.testing.assert_allclose(oracle.unary(k, inp), v.numpy(), rtol=RTOL, atol=ATOL, err_msg=k)


def test_gelu_closed_form(oracle):
    # 0.5 x (1 + erf(x/sqrt2)): gelu(0)=0, gelu(x)-gelu(-x)=x
    x = np.linspace(-5, 5, 101).astype(np.float32)
    g = oracle.unary("gelu", x)
    assert g[50] == 0.0
    np.testing.assert_allclose(g - g[::-1], x, rtol=1e-6, atol=1e-6)


def test_relu_edge_cases(oracle):
    x = np.array([-0.0, 0.0, -1.0, np.inf, -np.inf, np.nan], np.float32)
    y = oracle.unary("relu", x)
    np.testing.assert_array_equal(y[:5], np.array([0, 0, 0, np.inf, 0], np.float32))
    assert np.isnan(y[5])


def test_binary_vs_torch(oracle):
    r = rng(4)
    a = r.uniform(-2, 2, 2051).astype(np.float32)
    b = r.uniform(0.5, 2, 2051).astype(np.float32)
    ta, tb = torch.from_numpy(a), torch.from_numpy(b)
    for k, v in {"add": ta + tb, "sub": ta - tb, "mul": ta * tb, "div": ta / tb, "max": torch.maximum(ta, tb),
                 "min": torch.minimum(ta, tb)}.items():
        np.testing.assert_array_equal(oracle.binary(k, a, b), v.numpy(), err_msg=k)
    np.testing.assert_allclose(oracle.binary("pow", np.abs(a) + 0.1, b), torch.pow(ta.abs() + 0.1, tb).numpy(),
                               rtol=RTOL, atol=ATOL)
    ia = r.integers(0, 1000, 100).astype(np.int64)
    ib = r.integers(1, 50, 100).astype(np.int64)
    for k, v in {"add": ia + ib, "sub": ia - ib, "mul": ia * ib, "div": ia // ib, "max": np.maximum(ia, ib),
                 "min": np.minimum(ia, ib)}.items():
        np.testing.assert_array_equal(oracle.binary(k, ia, ib), v, err_msg=k)


def test_compare_where_convert(oracle):
    r = rng(6)
    a = r.integers(-3, 4, 500).astype(np.float32)
    b = r.integers(-3, 4, 500).astype(np.float32)
    for k, fn in {"EQ": np.equal, "NE": np.not_equal, "GE": np.greater_equal, "GT": np.greater,
                  "LE": np.less_equal, "LT": np.less}.items():
        np.testing.assert_array_equal(oracle.compare(k, a, b), fn(a, b), err_msg=k)
        np.testing.assert_array_equal(oracle.compare(k, a.astype(np.int64), b.astype(np.int64)), fn(a, b))
    pred = a > b  # a mixed predicate (the reference's own test only uses all-true, where.py:25-29)
    np.testing.assert_array_equal(oracle.where(pred, a, b), np.where(pred, a, b))
    np.testing.assert_array_equal(oracle.convert(np.array([1.9, -1.9, 3.0], np.float32), np.int64), [1, -1, 3])
    np.testing.assert_array_equal(oracle.convert(np.array([3, -4], np.int64), np.float32), np.array([3, -4], np.float32))


# ---- data movement: bit-exact vs numpy ----
def test_broadcast_transpose_slice_extract_gather(oracle):
    r = rng(7)
    x = r.standard_normal((3, 1, 5, 1)).astype(np.float32)
    np.testing.assert_array_equal(oracle.broadcast_to(x, (3, 4, 5, 6)), np.broadcast_to(x, (3, 4, 5, 6)))
    z = r.integers(0, 255, (2, 3, 4, 5)).astype(np.int64)
    for perms in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 2, 3), (0, 1, 3, 2)]:
        np.testing.assert_array_equal(oracle.transpose(z, perms), np.transpose(z, perms))
    h = r.standard_normal((7, 9)).astype(np.float16)
    np.testing.assert_array_equal(oracle.transpose(h, (1, 0)), h.T)
    got = oracle.stride_slice(z, (0, 1, 0, 1), (2, 3, 4, 5), (1, 1, 2, 3))
    np.testing.assert_array_equal(got, z[0:2, 1:3, 0:4:2, 1:5:3])
    assert got.shape == (2, 2, 2, 2)  # ceildiv(5-1, 3) = 2
    np.testing.assert_array_equal(oracle.extract(z, 1), z[1])
    np.testing.assert_array_equal(oracle.extract(z, -1), z[-1])  # LLHCanonicalize.cpp:337-354
    table = r.standard_normal((11, 6)).astype(np.float32)
    idx = np.array([[0, 10, 3], [3, 3, 7]], np.int64)
    np.testing.assert_array_equal(oracle.gather_rows(table, idx), table[idx])


# ---- reductions and normalisations ----
def test_reduce_vs_numpy_and_inits(oracle):
    r = rng(8)
    x = r.standard_normal((3, 4, 5, 6)).astype(np.float32)
    for axes in ([3], [1, 2], [0], [2, 3], [0, 1, 2, 3]):
        np.testing.assert_allclose(oracle.reduce("sum", x, axes), x.astype(np.float64).sum(tuple(axes)), rtol=RTOL, atol=ATOL)
        np.testing.assert_array_equal(oracle.reduce("max", x, axes), x.max(tuple(axes)))
        np.testing.assert_array_equal(oracle.reduce("min", x, axes), x.min(tuple(axes)))
    # init values (LLHToHLO.cpp:81-133): max over all-negative input must not be clamped at 0
    neg = -np.abs(x) - 1
    assert oracle.reduce("max", neg, [3]).max() < 0
    np.testing.assert_array_equal(oracle.reduce("sum", x, [-1]), oracle.reduce("sum", x, [3]))


def test_softmax_vs_torch_and_invariants(oracle):
    r = rng(9)
    x = (r.standard_normal((37, 129)) * 5).astype(np.float32)
    y = oracle.softmax_lastdim(x)
    np.testing.assert_allclose(y, torch.softmax(torch.from_numpy(x), -1).numpy(), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(y.sum(-1), 1.0, rtol=1e-5)
    np.testing.assert_allclose(oracle.softmax_lastdim(x + 100.0), y, rtol=1e-4, atol=1e-6)  # shift invariance
    big = np.array([[1e4, -1e4, 0.0]], np.float32)  # stable: no overflow
    np.testing.assert_array_equal(oracle.softmax_lastdim(big), np.array([[1, 0, 0]], np.float32))
    # the five-pass decomposition spelt with the oracle's own primitives
    mx = oracle.reduce("max", x, [1])[:, None]
    e = oracle.unary("exp", oracle.binary("sub", x, oracle.broadcast_to(mx, x.shape)))
    s = oracle.reduce("sum", e, [1])[:, None]
    np.testing.assert_array_equal(oracle.binary("div", e, oracle.broadcast_to(s, x.shape)), y)


def test_layernorm_vs_torch_and_invariants(oracle):
    r = rng(10)
    x = (r.standard_normal((19, 96)) * 3 + 2).astype(np.float32)
    g = r.uniform(-1, 1, 96).astype(np.float32)
    b = r.uniform(-1, 1, 96).astype(np.float32)
    want = F.layer_norm(torch.from_numpy(x), (96,), torch.from_numpy(g), torch.from_numpy(b), 1e-5).numpy()
    np.testing.assert_allclose(oracle.layernorm_lastdim(x, g, b, 1e-5), want, rtol=1e-4, atol=1e-5)
    y = oracle.layernorm_lastdim(x, None, None, 1e-5)
    np.testing.assert_allclose(y.mean(-1), 0, atol=1e-5)
    np.testing.assert_allclose(y.var(-1), 1, rtol=1e-3)  # biased variance, eps small


def test_batch_norm_inference_and_fold(oracle):
    r = rng(12)
    x = r.standard_normal((2, 5, 4, 3)).astype(np.float32)
    s, b, m = (r.standard_normal(5).astype(np.float32) for _ in range(3))
    v = r.uniform(0.5, 2, 5).astype(np.float32)
    want = F.batch_norm(torch.from_numpy(x), torch.from_numpy(m), torch.from_numpy(v), torch.from_numpy(s),
                        torch.from_numpy(b), training=False, eps=1e-5).numpy()
    np.testing.assert_allclose(oracle.batch_norm_inference(x, s, b, m, v, 1e-5), want, rtol=1e-4, atol=1e-5)
    # folding BN into the conv before it gives the same function
    xin = r.standard_normal((2, 3, 6, 6)).astype(np.float32)
    w = r.standard_normal((5, 3, 3, 3)).astype(np.float32)
    cb = r.standard_normal(5).astype(np.float32)
    y = oracle.conv2d(xin, w, cb, pad=(1, 1, 1, 1))
    want2 = oracle.batch_norm_inference(y, s, b, m, v, 1e-5)
    w2, b2 = oracle.fold_bn_into_conv(w, cb, s, b, m, v, 1e-5)
    np.testing.assert_allclose(oracle.conv2d(xin, w2, b2, pad=(1, 1, 1, 1)), want2, rtol=1e-4, atol=1e-4)


def test_maxpool_vs_torch_and_init_quirk(oracle):
    r = rng(13)
    x = r.standard_normal((2, 3, 11, 13)).astype(np.float32)
    for k, p, s, d in [((3, 3), (1, 1), (2, 2), (1, 1)), ((5, 5), (2, 2), (1, 1), (1, 1)), ((2, 3), (1, 0), (2, 1), (2, 1))]:
        if 2 * p[0] > d[0] * (k[0] - 1) + 1 or 2 * p[1] > d[1] * (k[1] - 1) + 1:
            continue
        want = F.max_pool2d(torch.from_numpy(x), k, s, p, d).numpy()
        got = oracle.maxpool2d(x, k, pad=(p[0], p[1], p[0], p[1]), stride=s, dilation=d)
        np.testing.assert_array_equal(got, want)
    # reference quirk (LLHToHLO.cpp:313-314): init 0 means result = max(0, torch result)
    q = oracle.maxpool2d(x, (3, 3), pad=(1, 1, 1, 1), stride=(2, 2), init_zero=True)
    t = F.max_pool2d(torch.from_numpy(x), 3, 2, 1).numpy()
    np.testing.assert_array_equal(q, np.maximum(t, 0))


def test_global_avgpool(oracle):
    r = rng(14)
    x = r.standard_normal((4, 6, 7, 7)).astype(np.float32)
    want = F.adaptive_avg_pool2d(torch.from_numpy(x), 1).numpy().reshape(4, 6)
    np.testing.assert_allclose(oracle.global_avgpool(x), want, rtol=RTOL, atol=ATOL)


def test_bf16_rounding(oracle):
    x = np.array([1.0, 1.00390625, 1.005859375, -3.1415927, 65504.0, 1e-40, np.inf], np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(oracle.round_bf16(x), want)
    r = rng(15)
    y = r.standard_normal(10000).astype(np.float32)
    np.testing.assert_array_equal(oracle.round_bf16(y), torch.from_numpy(y).to(torch.bfloat16).float().numpy())
