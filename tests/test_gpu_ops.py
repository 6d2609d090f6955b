"""GPU parity of every kernel entry point against the CPU oracle, called through the C-ABI.

Tolerances are the north star's: fp32 rtol 1e-4 / atol 1e-5, bf16 rtol 2e-2, data movement bit
exact.  Inputs are seeded numpy arrays copied to the device, so oracle and kernel see the same bits.
"""
import numpy as np
import pytest
import torch

from tests.util import (assert_close, assert_close_bf16, assert_close_f32, bf16_round, dev, host, rng)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from llcompiler_amd import ops as _ops
    return _ops


# --------------------------------------------------------------------------- elementwise
def test_add_relu_f32_and_bf16(ops, oracle):
    r = rng(1)
    for shape in [(4, 1024, 256), (7, 33), (5,), (3, 1, 17)]:
        a = r.uniform(-1, 1, shape).astype(np.float32)
        b = r.uniform(-1, 1, shape).astype(np.float32)
        prog = ops.make_program([("add", "r0", "in0", "in1"), ("relu", "r0", "r0")], "r0")
        want = oracle.unary("relu", oracle.binary("add", a, b))
        got = ops.elementwise(prog, [dev(a), dev(b)], shape, torch.float32)
        np.testing.assert_array_equal(host(got), want, err_msg=str(shape))  # add and max are exactly rounded
        ab, bb = bf16_round(a), bf16_round(b)
        wantb = bf16_round(oracle.unary("relu", oracle.binary("add", ab, bb)))
        gotb = ops.elementwise(prog, [dev(a, torch.bfloat16), dev(b, torch.bfloat16)], shape, torch.bfloat16)
        np.testing.assert_array_equal(host(gotb), wantb, err_msg=str(shape))


def test_fused_chain_with_immediates(ops, oracle):
    # ElewiseFusion1 of the reference's notes: x+x; -3; /2; relu; * y
    r = rng(2)
    x = r.standard_normal((3, 3, 56, 56)).astype(np.float32)
    y = r.standard_normal((3, 3, 56, 56)).astype(np.float32)
    prog = ops.make_program([("add", "r0", "in0", "in0"), ("sub", "r0", "r0", 3.0), ("div", "r0", "r0", 2.0),
                             ("relu", "r0", "r0"), ("mul", "r1", "r0", "in1")], "r1")
    t = oracle.binary("add", x, x)
    t = oracle.binary("sub", t, np.full_like(t, 3.0))
    t = oracle.binary("div", t, np.full_like(t, 2.0))
    want = oracle.binary("mul", oracle.unary("relu", t), y)
    got = ops.elementwise(prog, [dev(x), dev(y)], x.shape, torch.float32)
    np.testing.assert_array_equal(host(got), want)


def test_straight_line_and_dag_programs(ops, oracle):
    """Straight-line chains are rewritten to accumulator form by the library (operands swapped, seed input moved
    first); a program that keeps two values alive runs on the register-file interpreter.  Same results either way."""
    r = rng(31)
    shape = (5, 130)
    x = r.uniform(0.5, 1.5, shape).astype(np.float32)
    y = r.uniform(0.5, 1.5, shape).astype(np.float32)
    z = r.standard_normal(shape).astype(np.float32)
    B, U, F = oracle.binary, oracle.unary, np.full_like
    cases = [
        # immediate or input on the left of a non-commutative op
        ([("sub", "r0", 2.0, "in0"), ("div", "r0", "in1", "r0"), ("pow", "r0", 1.5, "r0")], "r0", [x, y],
         lambda: B("pow", F(x, 1.5), B("div", y, B("sub", F(x, 2.0), x)))),
        # the running value on the right of a compare
        ([("mul", "r1", "in0", 0.5), ("gt", "r1", "in1", "r1")], "r1", [x, y],
         lambda: oracle.compare("GT", y, B("mul", x, F(x, 0.5))).astype(np.float32)),
        # seed input used again later, three other inputs, input order unlike slot order
        ([("add", "r0", "in2", "in0"), ("mul", "r0", "r0", "in2"), ("sub", "r0", "r0", "in1"), ("max", "r0", "in3", "r0")],
         "r0", [x, y, z, x * 0.25], lambda: B("max", x * np.float32(0.25), B("sub", B("mul", B("add", z, x), z), y))),
        # x op x on the seed and on the running value
        ([("mul", "r0", "in0", "in0"), ("add", "r0", "r0", "r0"), ("sqrt", "r0", "r0")], "r0", [x],
         lambda: U("sqrt", B("add", B("mul", x, x), B("mul", x, x)))),
        # two live values: not a straight line
        ([("add", "r0", "in0", "in1"), ("mul", "r1", "in0", "in1"), ("sub", "r2", "r0", "r1")], "r2", [x, y],
         lambda: B("sub", B("add", x, y), B("mul", x, y))),
        # result is not the last value written
        ([("add", "r0", "in0", "in1"), ("neg", "r1", "r0")], "r0", [x, y], lambda: B("add", x, y)),
    ]
    for insts, result, inputs, want in cases:
        prog = ops.make_program(insts, result)
        got = ops.elementwise(prog, [dev(t) for t in inputs], shape, torch.float32)
        assert_close_f32(host(got), want(), str(insts))


@pytest.mark.parametrize("name", ["abs", "sqrt", "exp", "relu", "rsqrt", "neg", "gelu", "tanh", "erf", "sigmoid", "log", "recip"])
def test_unary_ops(ops, oracle, name):
    r = rng(3)
    x = r.uniform(-4, 4, (63, 130)).astype(np.float32)
    if name in ("sqrt", "rsqrt", "log", "recip"):
        x = np.abs(x) + 0.1
    prog = ops.make_program([(name, "r0", "in0")], "r0")
    got = ops.elementwise(prog, [dev(x)], x.shape, torch.float32)
    assert_close_f32(host(got), oracle.unary(name, x), name)


@pytest.mark.parametrize("name", ["add", "sub", "mul", "div", "max", "min", "pow"])
def test_binary_ops(ops, oracle, name):
    r = rng(4)
    a = r.uniform(0.1, 2, (17, 257)).astype(np.float32) * (1 if name == "pow" else r.choice([-1, 1], (17, 257)))
    a = a.astype(np.float32)
    b = r.uniform(0.5, 2, (17, 257)).astype(np.float32)
    prog = ops.make_program([(name, "r0", "in0", "in1")], "r0")
    got = ops.elementwise(prog, [dev(a), dev(b)], a.shape, torch.float32)
    assert_close_f32(host(got), oracle.binary(name, a, b), name)


def test_nan_propagation_in_relu_and_max(ops):
    x = np.array([np.nan, -1.0, 2.0, -0.0], np.float32)
    prog = ops.make_program([("relu", "r0", "in0")], "r0")
    got = host(ops.elementwise(prog, [dev(x)], x.shape, torch.float32))
    assert np.isnan(got[0]) and list(got[1:]) == [0.0, 2.0, 0.0]


def test_broadcast_patterns(ops, oracle):
    r = rng(5)
    # bias over the last dim, per-channel NCHW, attention mask [B,1,1,S] -> [B,H,S,S], scalar tensor<1>
    cases = [((6, 40), (40,)), ((2, 5, 7, 8), (1, 5, 1, 1)), ((2, 3, 8, 8), (2, 1, 1, 8)), ((4, 9), (1,)),
             ((3, 4, 5), (3, 1, 5)), ((3, 4, 6), (4, 1))]
    for full, small in cases:
        a = r.standard_normal(full).astype(np.float32)
        b = r.standard_normal(small).astype(np.float32)
        prog = ops.make_program([("add", "r0", "in0", "in1")], "r0")
        got = ops.elementwise(prog, [dev(a), dev(b)], full, torch.float32)
        np.testing.assert_array_equal(host(got), a + b, err_msg=str((full, small)))
        # the same through the oracle's explicit broadcast_to
        bb = b.reshape((1,) * (len(full) - b.ndim) + b.shape)
        np.testing.assert_array_equal(host(got), oracle.binary("add", a, oracle.broadcast_to(bb, full)))


def test_compare_where_convert(ops, oracle):
    r = rng(6)
    a = r.integers(-3, 4, (11, 50)).astype(np.float32)
    b = r.integers(-3, 4, (11, 50)).astype(np.float32)
    for name, kind in [("eq", "EQ"), ("ne", "NE"), ("ge", "GE"), ("gt", "GT"), ("le", "LE"), ("lt", "LT")]:
        prog = ops.make_program([(name, "r0", "in0", "in1")], "r0")
        got = ops.elementwise(prog, [dev(a), dev(b)], a.shape, torch.bool)
        np.testing.assert_array_equal(host(got), oracle.compare(kind, a, b), err_msg=name)
    pred = a > b
    prog = ops.make_program([("where", "r0", "in0", "in1", "in2")], "r0")
    got = ops.elementwise(prog, [dev(pred), dev(a), dev(b)], a.shape, torch.float32)
    np.testing.assert_array_equal(host(got), oracle.where(pred, a, b))
    f = np.array([1.9, -1.9, 3.0, 100.5], np.float32)
    np.testing.assert_array_equal(host(ops.convert(dev(f), torch.int64)), oracle.convert(f, np.int64))
    i = np.array([3, -4, 1 << 20], np.int64)
    np.testing.assert_array_equal(host(ops.convert(dev(i), torch.float32)), oracle.convert(i, np.float32))
    np.testing.assert_array_equal(host(ops.convert(dev(f), torch.bfloat16)), bf16_round(f))
    big = np.array([(1 << 40) + 3, -(1 << 35)], np.int64)
    np.testing.assert_array_equal(host(ops.convert(dev(big), torch.int32)), big.astype(np.int32))


def test_int64_elementwise(ops, oracle):
    r = rng(7)
    a = r.integers(0, 1 << 40, (5, 33)).astype(np.int64)
    b = r.integers(1, 1000, (5, 33)).astype(np.int64)
    for name in ["add", "sub", "mul", "div", "max", "min"]:
        prog = ops.make_program([(name, "r0", "in0", "in1")], "r0", integer=True)
        got = ops.elementwise(prog, [dev(a), dev(b)], a.shape, torch.int64)
        np.testing.assert_array_equal(host(got), oracle.binary(name, a, b), err_msg=name)


@pytest.mark.parametrize("seed", range(6))
def test_random_programs_bit_exact(ops, oracle, seed):
    """Randomly drawn straight-line and branching programs over exactly rounded ops (add, sub, mul, max, min, relu,
    abs, neg, with immediates on either side and inputs broadcast along leading, inner or all dims), in fp32, bf16
    storage and int64: every rewrite the library applies (accumulator form, swapped operands of sub, seed input moved
    to slot 0) must leave the bits the oracle computes op by op."""
    r = rng(100 + seed)
    shape = [(5, 7, 33), (130, 66), (3, 1, 257), (2, 3, 4, 40), (1, 513), (64, 64)][seed]
    binary, unary = ["add", "sub", "mul", "max", "min"], ["relu", "abs", "neg"]
    for trial in range(12):
        integer = trial % 4 == 3
        n_in = int(r.integers(1, 5))
        in_shapes, inputs = [], []
        for _ in range(n_in):
            kind = int(r.integers(0, 4))
            shp = list(shape)
            if kind == 1:
                shp = [1] * (len(shape) - 1) + [shape[-1]]            # a row broadcast over the leading dims
            elif kind == 2 and len(shape) > 1:
                shp[-1] = 1                                             # a column broadcast along the last dim
            elif kind == 3:
                shp = [1] * len(shape)                                  # a scalar tensor
            in_shapes.append(tuple(shp))
            if integer:
                inputs.append(r.integers(-50, 50, shp).astype(np.int64))
            else:
                inputs.append((r.integers(-64, 64, shp) / 8.0).astype(np.float32))   # exact in bf16 too
        in_shapes[0], inputs[0] = tuple(shape), (r.integers(-50, 50, shape).astype(np.int64) if integer else
                                                 (r.integers(-64, 64, shape) / 8.0).astype(np.float32))
        n_regs = int(r.integers(1, 4))
        insts, env, written = [], {}, []

        def operand(allow_imm=True):
            c = int(r.integers(0, 3 if allow_imm else 2))
            if c == 0 or not written:
                k = int(r.integers(0, n_in))
                return "in%d" % k, np.broadcast_to(inputs[k], shape)
            if c == 1:
                k = written[int(r.integers(0, len(written)))]
                return k, env[k]
            v = float(r.integers(-4, 5)) if integer else float(r.integers(-16, 17)) / 4.0
            return v, np.full(shape, v, np.int64 if integer else np.float32)
        for _ in range(int(r.integers(1, 9))):
            dst = "r%d" % int(r.integers(0, n_regs))
            if r.random() < 0.3 and not integer:
                name = unary[int(r.integers(0, len(unary)))]
                a, av = operand(allow_imm=False)
                insts.append((name, dst, a))
                val = oracle.unary(name, np.ascontiguousarray(av))
            else:
                name = binary[int(r.integers(0, len(binary)))]
                a, av = operand()
                b, bv = operand(allow_imm=not isinstance(a, float))
                insts.append((name, dst, a, b))
                val = oracle.binary(name, np.ascontiguousarray(av), np.ascontiguousarray(bv))
                if not integer:
                    # keep magnitudes small so that products stay exactly representable in fp32 and bf16
                    val = np.clip(val, -16.0, 16.0).astype(np.float32)
                    insts.append(("min", dst, dst, 16.0))
                    insts.append(("max", dst, dst, -16.0))
            env[dst] = val
            if dst not in written:
                written.append(dst)
        result = written[int(r.integers(0, len(written)))]
        prog = ops.make_program(insts, result, integer=integer)
        if integer:
            got = ops.elementwise(prog, [dev(t) for t in inputs], tuple(shape), torch.int64)
            np.testing.assert_array_equal(host(got), env[result], err_msg="int64 %s -> %s" % (insts, result))
        else:
            got = ops.elementwise(prog, [dev(t) for t in inputs], tuple(shape), torch.float32)
            np.testing.assert_array_equal(host(got), env[result], err_msg="f32 %s -> %s" % (insts, result))
            # bf16 storage: the inputs are exact in bf16, the arithmetic is fp32, the result is rounded once
            gotb = ops.elementwise(prog, [dev(t, torch.bfloat16) for t in inputs], tuple(shape), torch.bfloat16)
            np.testing.assert_array_equal(host(gotb), bf16_round(env[result]), err_msg="bf16 %s -> %s" % (insts, result))


def test_elementwise_empty_and_errors(ops):
    prog = ops.make_program([("relu", "r0", "in0")], "r0")
    out = ops.elementwise(prog, [torch.empty(0, 4, device="cuda")], (0, 4), torch.float32)
    assert out.shape == (0, 4)
    from llcompiler_amd._capi import LlcHipError
    with pytest.raises(LlcHipError):
        ops.elementwise(prog, [torch.zeros(3, 4, device="cuda")], (3, 5), torch.float32)


# --------------------------------------------------------------------------- row kernels
# 768 and 1536 columns: the exact-fit tiles of three and six vectors per lane (16 lanes per row from 8192 rows on)
@pytest.mark.parametrize("shape", [(37, 129), (64, 128), (9, 512), (5, 4096), (3, 5000), (2, 20000), (4, 12, 64, 64), (1, 1),
                                   (9, 768), (8, 1536), (8200, 768)])
def test_softmax(ops, oracle, shape):
    r = rng(8)
    x = (r.standard_normal(shape) * 3).astype(np.float32)
    got = ops.softmax(dev(x))
    assert_close_f32(host(got), oracle.softmax_lastdim(x), "softmax f32 %s" % (shape,))
    xb = bf16_round(x)
    gotb = ops.softmax(dev(x, torch.bfloat16))
    assert_close_bf16(host(gotb), bf16_round(oracle.softmax_lastdim(xb)), "softmax bf16 %s" % (shape,))


def test_softmax_masked_rows(ops, oracle):
    # additive -1e4 padding tails as in the BERT config; plus a row of equal values
    x = np.zeros((3, 64), np.float32)
    x[0, 40:] = -1e4
    x[1, :] = 7.0
    x[2, 1:] = -1e4
    got = host(ops.softmax(dev(x)))
    assert_close_f32(got, oracle.softmax_lastdim(x))
    np.testing.assert_allclose(got.sum(-1), 1.0, rtol=1e-5)


@pytest.mark.parametrize("shape", [(19, 96), (32, 768), (8, 1024), (5, 100), (2, 9000), (3, 7, 64), (8, 1536), (8200, 768)])
def test_layer_norm(ops, oracle, shape):
    r = rng(9)
    x = (r.standard_normal(shape) * 2 + 1).astype(np.float32)
    g = r.uniform(-1, 1, shape[-1]).astype(np.float32)
    b = r.uniform(-1, 1, shape[-1]).astype(np.float32)
    got = ops.layer_norm(dev(x), dev(g), dev(b), 1e-5)
    assert_close_f32(host(got), oracle.layernorm_lastdim(x, g, b, 1e-5), "layernorm f32 %s" % (shape,))
    got = ops.layer_norm(dev(x), None, None, 1e-5)
    assert_close_f32(host(got), oracle.layernorm_lastdim(x, None, None, 1e-5), "layernorm plain %s" % (shape,))
    xb, gb, bb = bf16_round(x), bf16_round(g), bf16_round(b)
    gotb = ops.layer_norm(dev(x, torch.bfloat16), dev(g, torch.bfloat16), dev(b, torch.bfloat16), 1e-5)
    assert_close_bf16(host(gotb), bf16_round(oracle.layernorm_lastdim(xb, gb, bb, 1e-5)), "layernorm bf16 %s" % (shape,))


@pytest.mark.parametrize("shape,axes", [((3, 4, 5, 6), [3]), ((3, 4, 5, 6), [1, 2]), ((3, 4, 5, 6), [0]), ((3, 4, 5, 6), [2, 3]),
                                        ((3, 4, 5, 6), [0, 1, 2, 3]), ((16, 4096), [1]), ((7, 300, 9), [1]), ((2, 3000), [-1]),
                                        ((8, 1536), [1]), ((5, 49, 130), [1]), ((16, 49, 512), [1]), ((40, 9, 4096), [1])])
def test_reduce(ops, oracle, shape, axes):
    r = rng(10)
    x = r.standard_normal(shape).astype(np.float32)
    for kind in ["sum", "max", "min"]:
        got = ops.reduce(kind, dev(x), axes)
        want = oracle.reduce(kind, x, axes)
        if kind == "sum":
            assert_close_f32(host(got), want, "reduce_sum %s %s" % (shape, axes))
        else:
            np.testing.assert_array_equal(host(got), want)
    neg = -np.abs(x) - 1  # init is -inf, not 0 (LLHToHLO.cpp:81-133)
    assert host(ops.reduce("max", dev(neg), axes)).max() < 0


def test_reduce_many_rows_of_768(ops, oracle):
    """8192 rows and more of 768 elements: 16 lanes per row, six vectors each in bf16 (three on 64 lanes in fp32).
    Sums of positive values, so that the comparison is not one of rounding order on sums that cancel."""
    r = rng(12)
    x = r.uniform(0.0, 1.0, (8200, 768)).astype(np.float32)
    assert_close_f32(host(ops.reduce("sum", dev(x), [1])), oracle.reduce("sum", x, [1]), "reduce_sum (8200, 768)")
    for kind in ["max", "min"]:
        np.testing.assert_array_equal(host(ops.reduce(kind, dev(x), [1])), oracle.reduce(kind, x, [1]))
    xb = bf16_round(x)
    np.testing.assert_array_equal(host(ops.reduce("max", dev(xb, torch.bfloat16), [1])), oracle.reduce("max", xb, [1]))
    assert_close_bf16(host(ops.reduce("sum", dev(xb, torch.bfloat16), [1])), bf16_round(oracle.reduce("sum", xb, [1])), "reduce_sum bf16 (8200, 768)")


@pytest.mark.parametrize("seed", range(3))
def test_random_rowwise_and_shape_cases(ops, oracle, seed):
    """Randomly drawn softmax / layer_norm / reduce shapes (rows from one element to tens of thousands, any number
    of rows) and random transposes, strided slices and copies of permuted or sliced views, the data movement bit
    exact against numpy indexing."""
    r = rng(900 + seed)
    for _ in range(10):
        cols = int(r.choice([1, 2, 7, 64, 100, 257, 768, 1000, 4096, 5003, 33000]))
        rows = int(r.integers(1, max(2, min(70, 200000 // cols))))
        lead = (rows,) if r.random() < 0.6 else (int(r.integers(1, 4)), rows)
        shape = lead + (cols,)
        x = (r.standard_normal(shape) * 2).astype(np.float32)
        assert_close_f32(host(ops.softmax(dev(x))), oracle.softmax_lastdim(x), "softmax %s" % (shape,))
        g, b = r.uniform(-1, 1, cols).astype(np.float32), r.uniform(-1, 1, cols).astype(np.float32)
        if cols > 1:
            assert_close_f32(host(ops.layer_norm(dev(x), dev(g), dev(b), 1e-5)), oracle.layernorm_lastdim(x, g, b, 1e-5),
                             "layer_norm %s" % (shape,))
        xb = bf16_round(x)
        assert_close_bf16(host(ops.softmax(dev(xb, torch.bfloat16))), bf16_round(oracle.softmax_lastdim(xb)), "softmax bf16 %s" % (shape,))
        axes = [len(shape) - 1] if r.random() < 0.5 else [0] if len(shape) == 2 else [0, 1]
        np.testing.assert_array_equal(host(ops.reduce("max", dev(x), axes)), oracle.reduce("max", x, axes))
        assert_close_f32(host(ops.reduce("sum", dev(x), axes)), oracle.reduce("sum", x, axes), "reduce_sum %s %s" % (shape, axes))
    for _ in range(12):
        rank = int(r.integers(2, 5))
        shape = tuple(int(v) for v in r.choice([1, 2, 3, 5, 8, 17, 33, 64, 70], rank))
        dtype = [np.float32, np.int64, np.float16, np.int8][int(r.integers(0, 4))]
        x = r.integers(-100, 100, shape).astype(dtype)
        perms = tuple(int(v) for v in r.permutation(rank))
        np.testing.assert_array_equal(host(ops.transpose(dev(x), perms)), np.ascontiguousarray(x.transpose(perms)),
                                      err_msg="transpose %s %s %s" % (shape, perms, dtype))
        start = tuple(int(r.integers(0, n)) for n in shape)
        end = tuple(int(r.integers(st, n + 1)) for st, n in zip(start, shape))
        step = tuple(int(r.integers(1, 4)) for _ in shape)
        want = x[tuple(slice(a, b, c) for a, b, c in zip(start, end, step))]
        got = ops.stride_slice(dev(x), start, end, step)
        assert tuple(got.shape) == want.shape, "slice %s %s %s %s" % (shape, start, end, step)
        np.testing.assert_array_equal(host(got), want, err_msg="slice %s %s %s %s" % (shape, start, end, step))
        view = dev(x).permute(*perms)[tuple(slice(None, None, int(r.integers(1, 3))) for _ in shape)]
        np.testing.assert_array_equal(host(ops.copy(view)), view.cpu().numpy(), err_msg="copy of a strided view %s %s" % (shape, perms))


@pytest.mark.parametrize("shape,axes", [((2, 3, 4, 5), [0, 2]), ((6, 1, 7, 33), [0, 3]), ((4, 5, 6, 7, 8), [0, 2, 4]),
                                        ((3, 64, 2, 70), [-1, 1]), ((5, 1, 1, 9), [1, 2]), ((8, 17, 3), [0, 1, 2]),
                                        ])
def test_reduce_over_split_axes(ops, oracle, shape, axes):
    """Axis sets that are not one run of adjacent dims: the library reduces run by run, innermost first."""
    r = rng(len(shape) * 100 + sum(shape))
    x = r.uniform(-1, 1, shape).astype(np.float32)
    for kind in ("sum", "max", "min"):
        want = oracle.reduce(kind, x, axes)
        got = ops.reduce(kind, dev(x), axes)
        assert tuple(got.shape) == want.shape
        if kind == "sum":
            assert_close_f32(host(got), want, "reduce %s %s %s" % (kind, shape, axes))
        else:
            np.testing.assert_array_equal(host(got), want)
    # 16-bit storage: the partial results between two runs are stored in that type too
    norm = sorted(a % len(shape) for a in axes)
    runs = []
    for a in norm:
        if runs and runs[-1][-1] == a - 1:
            runs[-1].append(a)
        else:
            runs.append([a])
    want = bf16_round(x)
    for run in reversed(runs):
        want = bf16_round(oracle.reduce("sum", want, run))
    gotb = host(ops.reduce("sum", dev(bf16_round(x), torch.bfloat16), axes))
    assert_close_bf16(gotb.reshape(-1), np.asarray(want).reshape(-1), "bf16")


def test_reduce_over_split_axes_with_an_empty_run(ops):
    """An empty reduced run yields the init value whatever the other runs hold."""
    x = torch.zeros(2, 0, 3, 4, device="cuda")
    np.testing.assert_array_equal(host(ops.reduce("sum", x, [1, 3])), np.zeros((2, 3), np.float32))
    np.testing.assert_array_equal(host(ops.reduce("max", x, [1, 3])), np.full((2, 3), -np.inf, np.float32))
    # the empty run innermost, a non-empty reduced run further out: still the init value in every output
    y = torch.zeros(2, 3, 4, 0, device="cuda")
    np.testing.assert_array_equal(host(ops.reduce("sum", y, [1, 3])), np.zeros((2, 4), np.float32))
    np.testing.assert_array_equal(host(ops.reduce("min", y, [1, 3])), np.full((2, 4), np.inf, np.float32))
    # one empty run over the last dim: the output is written, not left as allocated
    z = torch.zeros(5, 0, device="cuda")
    np.testing.assert_array_equal(host(ops.reduce("sum", z, [1])), np.zeros(5, np.float32))
    np.testing.assert_array_equal(host(ops.reduce("max", z, [1])), np.full(5, -np.inf, np.float32))
    np.testing.assert_array_equal(host(ops.reduce("max", torch.zeros(5, 0, 3, device="cuda"), [1])),
                                  np.full((5, 3), -np.inf, np.float32))


# --------------------------------------------------------------------------- data movement (bit exact)
@pytest.mark.parametrize("dtype", [np.float32, np.int64, np.float16, np.int8])
def test_transpose_bit_exact(ops, oracle, dtype):
    r = rng(11)
    x = r.integers(0, 127, (4, 6, 70, 66)).astype(dtype)
    for perms in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 2, 3), (0, 1, 3, 2), (2, 3, 0, 1), (0, 1, 2, 3)]:
        got = ops.transpose(dev(x), perms)
        np.testing.assert_array_equal(host(got), oracle.transpose(x, perms), err_msg=str(perms))
    m = r.integers(0, 127, (129, 257)).astype(dtype)
    np.testing.assert_array_equal(host(ops.transpose(dev(m), (1, 0))), m.T)


def test_attention_head_split_and_merge(ops, oracle):
    r = rng(12)
    x = r.standard_normal((2, 16, 4, 64)).astype(np.float32)  # [B,S,heads,64]
    t = ops.transpose(dev(x), (0, 2, 1, 3))
    np.testing.assert_array_equal(host(t), oracle.transpose(x, (0, 2, 1, 3)))
    back = ops.transpose(t, (0, 2, 1, 3))
    np.testing.assert_array_equal(host(back), x)
    xb = dev(x, torch.bfloat16)
    np.testing.assert_array_equal(host(ops.transpose(ops.transpose(xb, (0, 2, 1, 3)), (0, 2, 1, 3))), host(xb))


def test_slice_extract_broadcast_copy_gather(ops, oracle):
    r = rng(13)
    z = r.integers(0, 1 << 30, (6, 5, 8, 12)).astype(np.int64)
    got = ops.stride_slice(dev(z), (0, 1, 0, 1), (6, 3, 8, 11), (1, 1, 2, 3))
    np.testing.assert_array_equal(host(got), oracle.stride_slice(z, (0, 1, 0, 1), (6, 3, 8, 11), (1, 1, 2, 3)))
    assert got.shape == (6, 2, 4, 4)
    f = r.standard_normal((7, 3, 16)).astype(np.float32)
    np.testing.assert_array_equal(host(ops.stride_slice(dev(f), (2, 0, 4), (5, 3, 12), (1, 1, 1))), f[2:5, :, 4:12])
    np.testing.assert_array_equal(host(ops.extract(dev(f), 2)), oracle.extract(f, 2))
    np.testing.assert_array_equal(host(ops.extract(dev(f), -1)), oracle.extract(f, -1))
    b = r.standard_normal((3, 1, 5, 1)).astype(np.float32)
    np.testing.assert_array_equal(host(ops.broadcast_to(dev(b), (3, 4, 5, 6))), oracle.broadcast_to(b, (3, 4, 5, 6)))
    view = dev(f).permute(2, 0, 1)[::2]
    np.testing.assert_array_equal(host(ops.copy(view)), np.ascontiguousarray(f.transpose(2, 0, 1)[::2]))
    table = r.standard_normal((11, 6)).astype(np.float32)
    table8 = r.standard_normal((50, 768)).astype(np.float32)
    idx = np.array([[0, 10, 3], [3, 3, 7]], np.int64)
    np.testing.assert_array_equal(host(ops.gather_rows(dev(table), dev(idx))), oracle.gather_rows(table, idx))
    idx2 = r.integers(0, 50, (4, 9)).astype(np.int64)
    np.testing.assert_array_equal(host(ops.gather_rows(dev(table8), dev(idx2))), oracle.gather_rows(table8, idx2))
    # empty and ragged
    assert ops.stride_slice(dev(f), (3, 0, 0), (3, 3, 16), (1, 1, 1)).shape == (0, 3, 16)


# --------------------------------------------------------------------------- contractions
MM_SHAPES = [(1, 1, 1), (3, 3, 3), (4, 512, 784), (4, 10, 512), (33, 65, 129), (128, 128, 128), (256, 384, 96),
             (200, 72, 264), (130, 250, 36)]


@pytest.mark.parametrize("M,N,K", MM_SHAPES)
def test_matmul_f32(ops, oracle, M, N, K):
    r = rng(M * 7 + N * 3 + K)
    a = r.uniform(-1, 1, (M, K)).astype(np.float32)
    b = r.uniform(-1, 1, (K, N)).astype(np.float32)
    want = oracle.matmul(a, b, "mkn")
    assert_close_f32(host(ops.matmul(dev(a), dev(b))), want, "NN %s" % ((M, N, K),))
    # rhs as a transposed view of an [N,K] weight (llh.transpose folded into the operand)
    bt = dev(np.ascontiguousarray(b.T))
    assert_close_f32(host(ops.matmul(dev(a), bt.t())), want, "NT %s" % ((M, N, K),))
    at = dev(np.ascontiguousarray(a.T))
    assert_close_f32(host(ops.matmul(at.t(), dev(b))), want, "TN %s" % ((M, N, K),))


@pytest.mark.parametrize("M,N,K", MM_SHAPES)
def test_matmul_bf16(ops, oracle, M, N, K):
    r = rng(M * 7 + N * 3 + K + 1)
    a = bf16_round(r.uniform(-1, 1, (M, K)))
    b = bf16_round(r.uniform(-1, 1, (K, N)))
    want = bf16_round(oracle.matmul(a, b, "mkn"))
    got = ops.matmul(dev(a, torch.bfloat16), dev(b, torch.bfloat16))
    assert_close_bf16(host(got), want, "NN bf16 %s" % ((M, N, K),))
    bt = dev(np.ascontiguousarray(b.T), torch.bfloat16)
    assert_close_bf16(host(ops.matmul(dev(a, torch.bfloat16), bt.t())), want, "NT bf16 %s" % ((M, N, K),))
    goth = ops.matmul(dev(a, torch.float16), dev(b, torch.float16))
    assert_close_bf16(host(goth), oracle.matmul(a, b, "mkn"), "NN f16 %s" % ((M, N, K),))


@pytest.mark.parametrize("M,N,K", [(1024, 2048, 256), (1536, 1408, 448), (4096, 2048, 256)])
def test_matmul_16bit_complete_tiles(ops, oracle, M, N, K):
    """Shapes that take the direct-to-LDS kernels (complete 128x128x64 tiles, >= 128 of them; the last shape
    has enough tiles and a short enough reduction for the two-workgroups-per-CU form): row-major and
    transposed-view rhs, bf16 and f16, with and without the fused epilogue."""
    r = rng(M + N + K)
    a = bf16_round(r.uniform(-1, 1, (M, K)))
    b = bf16_round(r.uniform(-1, 1, (K, N)))
    base = oracle.matmul(a, b, "mkn")
    want = bf16_round(base)
    da = dev(a, torch.bfloat16)
    assert_close_bf16(host(ops.matmul(da, dev(b, torch.bfloat16))), want, "NN bf16")
    bt = dev(np.ascontiguousarray(b.T), torch.bfloat16)
    assert_close_bf16(host(ops.matmul(da, bt.t())), want, "NT bf16")
    assert_close_bf16(host(ops.matmul(dev(a, torch.float16), dev(b, torch.float16))), base, "NN f16")
    bth = dev(np.ascontiguousarray(b.T), torch.float16)
    assert_close_bf16(host(ops.matmul(dev(a, torch.float16), bth.t())), base, "NT f16")
    bias = bf16_round(r.standard_normal(N))
    res = bf16_round(r.standard_normal((M, N)))
    for act, alpha in [("none", 1.0), ("relu", 0.5), ("gelu", 0.125)]:
        w = base * np.float32(alpha) + bias[None, :] + res
        if act != "none":
            w = oracle.unary(act, w)
        epi = ops.Epilogue(alpha=alpha, bias=dev(bias, torch.bfloat16), residual=dev(res, torch.bfloat16), act=act)
        assert_close_bf16(host(ops.matmul(da, dev(b, torch.bfloat16), epi)), bf16_round(w), "NN epilogue " + act)
        assert_close_bf16(host(ops.matmul(da, bt.t(), epi)), bf16_round(w), "NT epilogue " + act)


@pytest.mark.parametrize("M,N,K", [(3584, 3584, 128), (3584, 3584, 192), (3584, 2688, 256), (2048, 3200, 320),
                                   (3584, 3584, 448)])
def test_matmul_16bit_wide_tiles(ops, oracle, M, N, K):
    """Shapes that take the 256 x BN tile kernel (complete tiles, at least 192 of them): BN = 256, 192 (N = 2688 =
    14 x 192) and 128 (N = 3200 = 25 x 128); reductions of 2, 3, 4, 5 and 7 k-tiles (the pipeline's prologue, paired
    main loop and two- or three-tile tail); row-major and transposed-view rhs, bf16 and f16, every fused epilogue."""
    r = rng(M + 3 * N + 7 * K)
    a = bf16_round(r.uniform(-1, 1, (M, K)))
    b = bf16_round(r.uniform(-1, 1, (K, N)))
    base = oracle.matmul(a, b, "mkn")
    want = bf16_round(base)
    da = dev(a, torch.bfloat16)
    assert_close_bf16(host(ops.matmul(da, dev(b, torch.bfloat16))), want, "NN bf16")
    bt = dev(np.ascontiguousarray(b.T), torch.bfloat16)
    assert_close_bf16(host(ops.matmul(da, bt.t())), want, "NT bf16")
    assert_close_bf16(host(ops.matmul(dev(a, torch.float16), dev(b, torch.float16))), base, "NN f16")
    bth = dev(np.ascontiguousarray(b.T), torch.float16)
    assert_close_bf16(host(ops.matmul(dev(a, torch.float16), bth.t())), base, "NT f16")
    bias = bf16_round(r.standard_normal(N))
    res = bf16_round(r.standard_normal((M, N)))
    for act, alpha, with_res in [("none", 1.0, True), ("relu", 0.5, False), ("gelu", 0.125, True)]:
        w = base * np.float32(alpha) + bias[None, :]
        if with_res:
            w = w + res
        if act != "none":
            w = oracle.unary(act, w)
        epi = ops.Epilogue(alpha=alpha, bias=dev(bias, torch.bfloat16), residual=dev(res, torch.bfloat16) if with_res else None, act=act)
        assert_close_bf16(host(ops.matmul(da, dev(b, torch.bfloat16), epi)), bf16_round(w), "NN epilogue " + act)
        assert_close_bf16(host(ops.matmul(da, bt.t(), epi)), bf16_round(w), "NT epilogue " + act)


def test_batch_matmul_16bit_wide_tiles(ops, oracle):
    """Batches of complete 256-row tiles: the batch index rides in the grid's z dimension of the wide-tile kernel."""
    r = rng(77)
    B, M, N, K = 4, 1792, 1792, 192
    a = bf16_round(r.uniform(-1, 1, (B, M, K)))
    b = bf16_round(r.uniform(-1, 1, (B, K, N)))
    want = bf16_round(oracle.batch_matmul(a, b, "mkn"))
    got = ops.batch_matmul(dev(a, torch.bfloat16), dev(b, torch.bfloat16))
    assert_close_bf16(host(got), want, "wide batch_matmul NN")
    bt = dev(np.ascontiguousarray(b.transpose(0, 2, 1)), torch.bfloat16)
    assert_close_bf16(host(ops.batch_matmul(dev(a, torch.bfloat16), bt.transpose(1, 2))), want, "wide batch_matmul NT")


def f16_round(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


def assert_close_f16(got, want, what=""):
    # half precision keeps 11 significant bits; the absolute floor covers sums that cancel to ~0
    assert_close(got, want, 2e-3, 4e-3, what)


@pytest.mark.parametrize("M,N,K", [(64, 64, 256), (128, 192, 320), (512, 768, 768), (192, 1088, 704), (512, 2304, 512)])
def test_matmul_16bit_small_rows_deep_ring(ops, oracle, M, N, K):
    """A few hundred rows times a linear layer's weight [N, K] (k-contiguous): the 64 x 64 tile kernel with a ring of
    direct-to-LDS stages.  Reductions of 4 and 5 k-tiles (shorter than the ring of 8), 12, 11 (odd) and 8; up to 256
    tiles (8 stages, one workgroup per CU) and more (4 stages, two per CU); bf16 and f16, every fused epilogue."""
    r = rng(5 * M + 3 * N + K)
    a = bf16_round(r.uniform(-1, 1, (M, K)))
    wt = bf16_round(r.uniform(-1, 1, (N, K)) * 0.25)
    base = oracle.matmul(a, np.ascontiguousarray(wt.T), "mkn")
    da, dw = dev(a, torch.bfloat16), dev(wt, torch.bfloat16)
    assert_close_bf16(host(ops.matmul(da, dw.t())), bf16_round(base), "NT bf16 %s" % ((M, N, K),))
    assert_close_f16(host(ops.matmul(dev(a, torch.float16), dev(wt, torch.float16).t())), f16_round(base), "NT f16 %s" % ((M, N, K),))
    bias = bf16_round(r.standard_normal(N))
    res = bf16_round(r.standard_normal((M, N)))
    for act, alpha, with_res in [("none", 1.0, True), ("relu", 0.5, False), ("gelu", 0.125, True)]:
        w = base * np.float32(alpha) + bias[None, :]
        if with_res:
            w = w + res
        if act != "none":
            w = oracle.unary(act, w)
        epi = ops.Epilogue(alpha=alpha, bias=dev(bias, torch.bfloat16), residual=dev(res, torch.bfloat16) if with_res else None, act=act)
        assert_close_bf16(host(ops.matmul(da, dw.t(), epi)), bf16_round(w), "NT epilogue %s %s" % (act, (M, N, K)))


def test_batch_matmul_16bit_small_rows_deep_ring(ops, oracle):
    """The same kernel over a batch (the batch index rides in the grid's z dimension), with a residual per entry."""
    r = rng(91)
    B, M, N, K = 5, 128, 192, 448
    a = bf16_round(r.uniform(-1, 1, (B, M, K)))
    wt = bf16_round(r.uniform(-1, 1, (B, N, K)) * 0.25)
    res = bf16_round(r.standard_normal((B, M, N)))
    base = oracle.batch_matmul(a, np.ascontiguousarray(wt.transpose(0, 2, 1)), "mkn")
    got = ops.batch_matmul(dev(a, torch.bfloat16), dev(wt, torch.bfloat16).transpose(1, 2),
                           ops.Epilogue(residual=dev(res, torch.bfloat16)))
    assert_close_bf16(host(got), bf16_round(base + res), "deep ring batch_matmul NT + residual")


@pytest.mark.parametrize("B,M,N", [(8, 1024, 384), (2, 4096, 128), (1, 8192, 256), (32, 512, 512)])
def test_batch_matmul_reduction_of_64_sweeps_the_columns(ops, oracle, B, M, N):
    """K = 64 with a row-major B goes to the kernel that keeps a 64-row panel of A in registers and sweeps B's
    columns in 256-byte tiles (odd and even tile counts, one tile, plain matmul as batch 1), in all three storage
    types, bare and with alpha, bias, residual and an activation in the epilogue."""
    r = rng(B * 31 + N)
    a = r.uniform(-1, 1, (B, M, 64)).astype(np.float32)
    b = r.uniform(-1, 1, (B, 64, N)).astype(np.float32)
    bias = r.uniform(-0.5, 0.5, (N,)).astype(np.float32)
    res = r.uniform(-0.5, 0.5, (B, M, N)).astype(np.float32)
    want = oracle.batch_matmul(a, b, "mkn")
    got = ops.batch_matmul(dev(a), dev(b)) if B > 1 else ops.matmul(dev(a[0]), dev(b[0]))[None]
    assert_close_f32(host(got), want, "f32")
    for act in ("relu", "gelu"):
        w2 = oracle.unary(act, (want * np.float32(0.5) + bias[None, None, :] + res).astype(np.float32))
        epi = ops.Epilogue(alpha=0.5, bias=dev(bias), residual=dev(res), act=act)
        assert_close_f32(host(ops.batch_matmul(dev(a), dev(b), epi)), w2, "f32 epilogue " + act)
    for dt, rnd, tol in ((torch.bfloat16, bf16_round, assert_close_bf16), (torch.float16, f16_round, assert_close_f16)):
        if N % 128:
            continue
        ar, br, biasr, resr = rnd(a), rnd(b), rnd(bias), rnd(res)
        w = oracle.batch_matmul(ar, br, "mkn")
        tol(host(ops.batch_matmul(dev(ar, dt), dev(br, dt))), rnd(w), "16-bit")
        w2 = oracle.unary("relu", (w * np.float32(0.5) + biasr[None, None, :] + resr).astype(np.float32))
        epi = ops.Epilogue(alpha=0.5, bias=dev(biasr, dt), residual=dev(resr, dt), act="relu")
        tol(host(ops.batch_matmul(dev(ar, dt), dev(br, dt), epi)), rnd(w2), "16-bit epilogue")


def _attention_oracle(oracle, q, k, v, mask, scale, rnd):
    """The unfused op group on the CPU oracle: batch_matmul, scale, mask add, softmax over the keys, the
    probabilities rounded to the storage type (the fused kernel feeds them to the matrix cores in it), batch_matmul."""
    B, H, Sq, D = q.shape
    Skv = k.shape[2]
    s = oracle.batch_matmul(q.reshape(B * H, Sq, D), np.ascontiguousarray(k.reshape(B * H, Skv, D).transpose(0, 2, 1)), "mkn")
    s = s.reshape(B, H, Sq, Skv) * np.float32(scale)
    if mask is not None:
        s = s + mask[:, None, None, :]
    p = rnd(oracle.softmax_lastdim(s.reshape(-1, Skv))).reshape(B * H, Sq, Skv)
    return oracle.batch_matmul(p, v.reshape(B * H, Skv, D), "mkn").reshape(B, H, Sq, D)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_attention_with_a_fully_masked_sample(ops, oracle, dt):
    """A batch entry whose every key carries the most negative finite number of the storage type (an all-padding
    sequence): the unfused group adds it to the scores, which it absorbs, and softmaxes to the uniform row, so the
    output is the mean of V; the fused kernel works in log2 units, where that value would overflow."""
    r = rng(5)
    B, H, S = 2, 2, 128
    rnd = bf16_round if dt == "bf16" else (lambda a: np.asarray(a, np.float32))
    tdt = torch.bfloat16 if dt == "bf16" else torch.float32
    q, k, v = (rnd(r.uniform(-1, 1, (B, H, S, 64))) for _ in range(3))
    lowest = float(torch.finfo(tdt).min)
    mask = np.zeros((B, S), np.float32)
    mask[0, :] = lowest
    mask[1, S // 2:] = lowest
    want = _attention_oracle(oracle, q, k, v, mask, 0.125, rnd)
    assert np.isfinite(want).all()
    np.testing.assert_allclose(want[0, 0, 0], v[0, 0].mean(axis=0), rtol=1e-4, atol=1e-5)
    got = ops.attention(dev(q, tdt), dev(k, tdt), dev(v, tdt), dev(mask, tdt), 0.125)
    (assert_close_bf16 if dt == "bf16" else assert_close_f32)(host(got), rnd(want), "fully masked sample " + dt)


@pytest.mark.parametrize("B,H,Sq,Skv,masked", [(1, 1, 128, 128, False), (2, 3, 100, 200, True), (1, 2, 64, 64, False),
                                             (3, 2, 33, 77, False), (1, 1, 1, 1, True), (2, 12, 256, 256, True),
                                             (1, 2, 130, 448, False)])
def test_attention(ops, oracle, B, H, Sq, Skv, masked):
    r = rng(B * 1000 + H * 100 + Sq + Skv)
    q = bf16_round(r.uniform(-1, 1, (B, H, Sq, 64)))
    k = bf16_round(r.uniform(-1, 1, (B, H, Skv, 64)))
    v = bf16_round(r.uniform(-1, 1, (B, H, Skv, 64)))
    mask = None
    if masked:  # per-sample valid length, the tail at -1e4, as a BERT attention mask
        mask = np.zeros((B, Skv), np.float32)
        for b in range(B):
            mask[b, int(r.integers(Skv // 2, Skv)) + 1:] = -1e4
        mask = bf16_round(mask)
    scale = 0.125
    for dt, rnd, close in ((torch.bfloat16, bf16_round, assert_close_bf16),
                           (torch.float16, lambda x: x.astype(np.float16).astype(np.float32), assert_close_bf16),
                           (torch.float32, lambda x: x, assert_close_f32)):
        want = _attention_oracle(oracle, q, k, v, mask, scale, rnd)
        dm = dev(mask, dt) if masked else None
        got = ops.attention(dev(q, dt), dev(k, dt), dev(v, dt), dm, scale)
        close(host(got), want, "attention %s" % dt)
    # head-split views of [B, S, H*64] activations in, the merged layout out (no copies on either side)
    qs = dev(np.ascontiguousarray(q.transpose(0, 2, 1, 3)).reshape(B, Sq, H * 64), torch.bfloat16)
    ks = dev(np.ascontiguousarray(k.transpose(0, 2, 1, 3)).reshape(B, Skv, H * 64), torch.bfloat16)
    vs = dev(np.ascontiguousarray(v.transpose(0, 2, 1, 3)).reshape(B, Skv, H * 64), torch.bfloat16)
    for dt, rnd, close in ((torch.bfloat16, bf16_round, assert_close_bf16), (torch.float32, lambda x: x, assert_close_f32)):
        merged = torch.zeros((B, Sq, H, 64), dtype=dt, device="cuda")
        ops.attention(qs.to(dt).view(B, Sq, H, 64).permute(0, 2, 1, 3), ks.to(dt).view(B, Skv, H, 64).permute(0, 2, 1, 3),
                      vs.to(dt).view(B, Skv, H, 64).permute(0, 2, 1, 3), dev(mask, dt) if masked else None, scale,
                      out=merged.permute(0, 2, 1, 3))
        want = _attention_oracle(oracle, q, k, v, mask, scale, rnd)
        close(host(merged).transpose(0, 2, 1, 3), want, "attention on head-split views %s" % dt)


@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("B,H,Sq,Skv,masked", [(1, 1, 128, 128, False), (2, 3, 100, 200, True), (3, 2, 33, 77, False),
                                             (1, 1, 1, 1, True), (2, 12, 256, 256, True), (1, 2, 130, 448, False)])
def test_attention_head_dims_32_and_128(ops, oracle, D, B, H, Sq, Skv, masked):
    """The fused kernel in the 16-bit types at the other two head dims it takes (half a 128-byte row per key, and two
    64-wide tiles side by side), contiguous operands and head-split views; fp32 operands of those head dims are refused."""
    r = rng(D * 7 + B * 1000 + H * 100 + Sq + Skv)
    q = bf16_round(r.uniform(-1, 1, (B, H, Sq, D)))
    k = bf16_round(r.uniform(-1, 1, (B, H, Skv, D)))
    v = bf16_round(r.uniform(-1, 1, (B, H, Skv, D)))
    mask = None
    if masked:
        mask = np.zeros((B, Skv), np.float32)
        for b in range(B):
            mask[b, int(r.integers(Skv // 2, Skv)) + 1:] = -1e4
        mask = bf16_round(mask)
    scale = float(D) ** -0.5
    for dt, rnd in ((torch.bfloat16, bf16_round), (torch.float16, lambda x: x.astype(np.float16).astype(np.float32))):
        want = _attention_oracle(oracle, q, k, v, mask, scale, rnd)
        got = ops.attention(dev(q, dt), dev(k, dt), dev(v, dt), dev(mask, dt) if masked else None, scale)
        assert_close_bf16(host(got), want, "attention head dim %d %s" % (D, dt))
    qs = dev(np.ascontiguousarray(q.transpose(0, 2, 1, 3)).reshape(B, Sq, H * D), torch.bfloat16)
    ks = dev(np.ascontiguousarray(k.transpose(0, 2, 1, 3)).reshape(B, Skv, H * D), torch.bfloat16)
    vs = dev(np.ascontiguousarray(v.transpose(0, 2, 1, 3)).reshape(B, Skv, H * D), torch.bfloat16)
    merged = torch.zeros((B, Sq, H, D), dtype=torch.bfloat16, device="cuda")
    ops.attention(qs.view(B, Sq, H, D).permute(0, 2, 1, 3), ks.view(B, Skv, H, D).permute(0, 2, 1, 3),
                  vs.view(B, Skv, H, D).permute(0, 2, 1, 3), dev(mask, torch.bfloat16) if masked else None, scale,
                  out=merged.permute(0, 2, 1, 3))
    assert_close_bf16(host(merged).transpose(0, 2, 1, 3), _attention_oracle(oracle, q, k, v, mask, scale, bf16_round),
                      "attention on head-split views, head dim %d" % D)
    from llcompiler_amd._capi import LlcHipError
    with pytest.raises(LlcHipError):
        ops.attention(dev(q), dev(k), dev(v), None, scale)


@pytest.mark.parametrize("seed", range(3))
def test_random_bmm_attention_pool_gather_cases(ops, oracle, seed):
    """Randomly drawn batched products (rank 3 and the rank-4 head-split form, either operand a transposed view,
    every storage type), attention shapes (ragged query and key counts, masks, any batch and head count), max-pool
    windows and row gathers."""
    r = rng(1100 + seed)
    types = [(torch.float32, assert_close_f32, lambda x: x), (torch.bfloat16, assert_close_bf16, bf16_round),
             (torch.float16, assert_close_bf16, lambda x: x)]
    for _ in range(10):
        B = int(r.choice([1, 2, 5, 12]))
        M, N, K = (int(r.choice(d)) for d in ([1, 7, 64, 128, 130, 256], [1, 8, 64, 72, 128, 256], [1, 8, 64, 96, 128, 200]))
        dt, close, rnd = types[int(r.integers(0, 3))]
        a = bf16_round(r.uniform(-1, 1, (B, M, K)))
        b = bf16_round(r.uniform(-1, 1, (B, K, N)))
        want = rnd(oracle.batch_matmul(a, b, "mkn"))
        da = dev(a, dt) if r.random() < 0.5 else dev(np.ascontiguousarray(a.transpose(0, 2, 1)), dt).transpose(1, 2)
        db = dev(b, dt) if r.random() < 0.5 else dev(np.ascontiguousarray(b.transpose(0, 2, 1)), dt).transpose(1, 2)
        close(host(ops.batch_matmul(da, db)), want, "bmm B%d %dx%dx%d %s" % (B, M, N, K, dt))
        if B % 2 == 0 or B == 12:                      # [B0, B1, rows, cols] operands cut out of [B0, rows, B1*cols]
            b1 = 2 if B % 2 == 0 and B != 12 else 3
            b0 = B // b1
            a4 = np.ascontiguousarray(a.reshape(b0, b1, M, K).transpose(0, 2, 1, 3))      # [b0, M, b1, K] in memory
            d4 = dev(a4, dt).permute(0, 2, 1, 3)                                            # logical [b0, b1, M, K]
            out = torch.empty((b0, M, b1, N), dtype=dt, device="cuda").permute(0, 2, 1, 3)  # merged layout written in place
            ops.batch_matmul(d4, db.reshape(b0, b1, K, N) if db.is_contiguous() else dev(b, dt).view(b0, b1, K, N), out=out)
            close(host(out).reshape(B, M, N), want, "bmm rank 4 B%d=%dx%d %dx%dx%d %s" % (B, b0, b1, M, N, K, dt))
    for _ in range(6):
        B, H = int(r.integers(1, 4)), int(r.integers(1, 5))
        Sq, Skv = int(r.choice([1, 5, 32, 100, 128, 129, 300])), int(r.choice([1, 17, 64, 65, 128, 200, 333]))
        q = bf16_round(r.uniform(-1, 1, (B, H, Sq, 64)))
        k = bf16_round(r.uniform(-1, 1, (B, H, Skv, 64)))
        v = bf16_round(r.uniform(-1, 1, (B, H, Skv, 64)))
        mask = None
        if r.random() < 0.5:
            mask = np.zeros((B, Skv), np.float32)
            for bb in range(B):
                mask[bb, int(r.integers(Skv // 2, Skv)) + 1:] = -1e4
            mask = bf16_round(mask)
        scale = float(r.choice([0.125, 0.25, 0.5]))   # (sharper distributions leave bf16 rounding noise of the
                                                      # probabilities above the absolute floor on outputs near 0)
        for dt, close, rnd in types:
            rr = rnd if dt != torch.float16 else (lambda x: x.astype(np.float16).astype(np.float32))
            want = _attention_oracle(oracle, q, k, v, mask, scale, rr)
            got = ops.attention(dev(q, dt), dev(k, dt), dev(v, dt), None if mask is None else dev(mask, dt), scale)
            close(host(got), want, "attention B%d H%d Sq%d Skv%d mask %s scale %g %s" % (B, H, Sq, Skv, mask is not None, scale, dt))
    for _ in range(8):
        N, Cc, H, W = int(r.integers(1, 4)), int(r.integers(1, 9)), int(r.integers(3, 30)), int(r.integers(3, 30))
        kern = (int(r.integers(1, 5)), int(r.integers(1, 5)))
        st = (int(r.integers(1, 4)), int(r.integers(1, 4)))
        dil = (int(r.integers(1, 3)), int(r.integers(1, 3)))
        pad = tuple(int(min(v, (kk - 1) * dd // 2)) for v, kk, dd in zip(r.integers(0, 3, 4), kern + kern, dil + dil))
        if (H + pad[0] + pad[2] - dil[0] * (kern[0] - 1) - 1) < 0 or (W + pad[1] + pad[3] - dil[1] * (kern[1] - 1) - 1) < 0:
            continue
        x = r.standard_normal((N, Cc, H, W)).astype(np.float32)
        for iz in (False, True):
            np.testing.assert_array_equal(host(ops.max_pool(dev(x), kern, pad=pad, stride=st, dilation=dil, init_zero=iz)),
                                          oracle.maxpool2d(x, kern, pad=pad, stride=st, dilation=dil, init_zero=iz),
                                          err_msg="max_pool %s k%s s%s d%s pad%s init_zero=%s" % (x.shape, kern, st, dil, pad, iz))
    for _ in range(6):
        rows, width = int(r.integers(1, 200)), int(r.choice([1, 3, 8, 64, 100, 768]))
        table = r.standard_normal((rows, width)).astype(np.float32)
        idx = r.integers(0, rows, tuple(int(v) for v in r.integers(1, 9, int(r.integers(1, 3))))).astype(np.int64)
        np.testing.assert_array_equal(host(ops.gather_rows(dev(table), dev(idx))), oracle.gather_rows(table, idx))
        tb = bf16_round(table)
        np.testing.assert_array_equal(host(ops.gather_rows(dev(tb, torch.bfloat16), dev(idx))), oracle.gather_rows(tb, idx))


@pytest.mark.parametrize("B,H,Sq,Skv", [(1, 12, 512, 512), (1, 3, 40, 257), (2, 2, 96, 320)])
def test_attention_few_workgroups_keys_split_over_the_waves(ops, oracle, B, H, Sq, Skv):
    """A sequence or two with a few heads: 32 queries per workgroup, every fourth key block to each of its waves, the
    four partial results combined at the end.  An encoder block's shape at a batch of one; key counts that leave the
    waves with two, one and one blocks (the last block one key long); a whole block of one wave masked with -inf
    (that wave's partial result then carries no weight) and a finite padding tail."""
    r = rng(B + 7 * H + Sq + Skv)
    q = bf16_round(r.uniform(-1, 1, (B, H, Sq, 64)))
    k = bf16_round(r.uniform(-1, 1, (B, H, Skv, 64)))
    v = bf16_round(r.uniform(-1, 1, (B, H, Skv, 64)))
    for dt, rnd in ((torch.bfloat16, bf16_round), (torch.float16, lambda x: x.astype(np.float16).astype(np.float32))):
        want = _attention_oracle(oracle, q, k, v, None, 0.125, rnd)
        got = ops.attention(dev(q, dt), dev(k, dt), dev(v, dt), None, 0.125)
        assert_close_bf16(host(got), want, "split attention %s %s" % (dt, (B, H, Sq, Skv)))
    mask = np.zeros((B, Skv), np.float32)
    mask[:, 64:128] = -np.inf              # the second wave's first block
    mask[0, Skv - Skv // 5:] = -1e4        # a padding tail
    keep = np.ones(Skv, bool)
    keep[64:128] = False
    tail = bf16_round(mask[:, keep])
    want = _attention_oracle(oracle, q, k[:, :, keep], v[:, :, keep], tail, 0.125, bf16_round)
    got = ops.attention(dev(q, torch.bfloat16), dev(k, torch.bfloat16), dev(v, torch.bfloat16), dev(mask, torch.bfloat16), 0.125)
    assert_close_bf16(host(got), want, "split attention, one block at -inf %s" % ((B, H, Sq, Skv),))


def test_attention_fully_masked_leading_block_and_errors(ops, oracle):
    # -inf on the whole first block of keys: the running maximum stays -inf there and must not turn into NaN
    r = rng(5)
    q = bf16_round(r.uniform(-1, 1, (1, 1, 32, 64)))
    k = bf16_round(r.uniform(-1, 1, (1, 1, 192, 64)))
    v = bf16_round(r.uniform(-1, 1, (1, 1, 192, 64)))
    mask = np.zeros((1, 192), np.float32)
    mask[0, :70] = -np.inf
    got = host(ops.attention(dev(q, torch.bfloat16), dev(k, torch.bfloat16), dev(v, torch.bfloat16), dev(mask, torch.bfloat16), 0.125))
    want = _attention_oracle(oracle, q[:, :, :, :], k[:, :, 70:], v[:, :, 70:], None, 0.125, bf16_round)
    assert_close_bf16(got, want, "attention with -inf on the first 70 keys")
    from llcompiler_amd._capi import LlcHipError
    x = dev(q, torch.bfloat16)
    got32 = host(ops.attention(dev(q), dev(k), dev(v), dev(mask), 0.125))
    assert_close_f32(got32, _attention_oracle(oracle, q, k[:, :, 70:], v[:, :, 70:], None, 0.125, lambda x: x), "fp32, -inf on 70 keys")
    with pytest.raises(LlcHipError):  # fp64 operands are not implemented: an error, not another path
        ops.attention(dev(q).double(), dev(k).double(), dev(v).double())
    with pytest.raises(LlcHipError):
        ops.attention(x, dev(k, torch.bfloat16)[..., :32], dev(v, torch.bfloat16))  # head dim 32
    with pytest.raises(LlcHipError):
        ops.attention(x, dev(k, torch.bfloat16), dev(v, torch.bfloat16)[:, :, :100])  # k and v lengths differ


@pytest.mark.parametrize("M,N,K", [(1, 100, 256), (4, 512, 784), (4, 10, 512), (3, 33, 1032), (5, 33, 1032), (16, 64, 2048),
                                   (13, 7, 40), (2, 1, 8)])
def test_matmul_skinny(ops, oracle, M, N, K):
    """At most 16 rows times a [N,K] weight read as its transpose (a linear layer on a small batch) takes the
    single-pass kernel: every dtype, the fused epilogue, rows taken from a wider buffer."""
    r = rng(M * 5 + N * 11 + K)
    a = bf16_round(r.uniform(-1, 1, (M, K)))
    w = bf16_round(r.uniform(-1, 1, (N, K)))
    bias = bf16_round(r.standard_normal(N))
    res = bf16_round(r.standard_normal((M, N)))
    base = oracle.matmul(a, np.ascontiguousarray(w.T), "mkn")
    wide = np.zeros((M, K + 24), np.float32)
    wide[:, 8:8 + K] = a
    for dt, close, rnd in ((torch.float32, assert_close_f32, lambda x: x), (torch.bfloat16, assert_close_bf16, bf16_round),
                           (torch.float16, assert_close_bf16, lambda x: x)):
        da, dw = dev(a, dt), dev(w, dt)
        close(host(ops.matmul(da, dw.t())), rnd(base), "skinny %s" % dt)
        close(host(ops.matmul(dev(wide, dt)[:, 8:8 + K], dw.t())), rnd(base), "skinny strided rows %s" % dt)
        for act, alpha in [("none", 1.0), ("relu", 0.5), ("gelu", 0.125)]:
            want = base * np.float32(alpha) + bias[None, :] + res
            if act != "none":
                want = oracle.unary(act, want)
            epi = ops.Epilogue(alpha=alpha, bias=dev(bias, dt), residual=dev(res, dt), act=act)
            close(host(ops.matmul(da, dw.t(), epi)), rnd(want), "skinny epilogue %s %s" % (act, dt))


def test_batch_matmul_16bit_complete_tiles(ops, oracle):
    r = rng(77)
    a = bf16_round(r.uniform(-1, 1, (8, 512, 256)))
    b = bf16_round(r.uniform(-1, 1, (8, 256, 512)))
    want = bf16_round(oracle.batch_matmul(a, b, "mkn"))
    assert_close_bf16(host(ops.batch_matmul(dev(a, torch.bfloat16), dev(b, torch.bfloat16))), want, "bmm bf16")
    bt = dev(np.ascontiguousarray(b.transpose(0, 2, 1)), torch.bfloat16)
    assert_close_bf16(host(ops.batch_matmul(dev(a, torch.bfloat16), bt.transpose(1, 2))), want, "bmm bf16 NT")


def _gelu_16bit_restated(x):
    """The GELU that the epilogues of the 16-bit products apply, restated in numpy fp32: x / (1 + 2^(-x p(x^2)))."""
    f = np.float32
    x = x.astype(f)
    u = x * x
    p = f(2.2971660592200047) + u * (f(0.1095363857595901) + u * (f(-0.0014344055324419125) + u * f(1.327634682739151e-05)))
    with np.errstate(over="ignore"):
        e = np.exp2((-x * p).astype(f)).astype(f)
    return (x / (f(1) + e)).astype(f)


def test_gelu_of_the_16bit_epilogues_against_the_oracle(ops, oracle):
    """The epilogues of the 16-bit products replace the erf form of GELU by a cheaper one (their results are rounded to
    bf16 / f16 anyway).  Its formula in fp32, against the oracle's erf form on 65536 points of [-8, 8): absolute error
    below 2.5e-4, relative error below 1.5e-3 on [-5, 5].  Then the kernels themselves: a product spelt so that output
    (i, j) is gelu(r_i + c_j) with r_i + c_j exact in fp32, against the oracle's gelu rounded to the storage type, at
    the stated tolerance and at one unit of the storage type's precision."""
    r_vals = (np.arange(256, dtype=np.float32) - 128) / 16          # -8 .. 8 in steps of 1/16: exact in bf16 and f16
    c_vals = np.arange(256, dtype=np.float32) / 4096                # 0 .. 1/16 in steps of 2^-12: exact in both
    x = (r_vals[:, None] + c_vals[None, :]).astype(np.float32)
    want = oracle.unary("gelu", x)
    formula = _gelu_16bit_restated(x)
    err = np.abs(formula.astype(np.float64) - want.astype(np.float64))
    inside = np.abs(x) <= 5
    rel = err[inside] / np.maximum(np.abs(want[inside]).astype(np.float64), 1e-30)
    print("16-bit epilogue GELU, formula in fp32 vs the oracle: max abs error %.3g, max relative error on [-5, 5] %.3g"
          % (err.max(), rel[np.abs(x[inside]) > 1e-3].max()))
    assert err.max() <= 2.5e-4 and rel[np.abs(x[inside]) > 1e-3].max() <= 1.5e-3
    a = np.zeros((256, 64), np.float32)
    a[:, 0] = r_vals
    b = np.zeros((64, 256), np.float32)
    b[0, :] = 1.0
    for dt, unit in ((torch.bfloat16, 2.0 ** -8), (torch.float16, 2.0 ** -9)):
        got = host(ops.matmul(dev(a, dt), dev(b, dt), ops.Epilogue(bias=dev(c_vals, dt), act="gelu")))
        rounded = host(dev(want, dt))
        assert_close_bf16(got, rounded, "gelu epilogue %s" % dt)
        off = np.abs(got.astype(np.float64) - want.astype(np.float64))
        assert (off <= unit * np.abs(want) + 2.5e-4).all(), "gelu epilogue %s: %g" % (dt, (off - unit * np.abs(want)).max())


def test_matmul_epilogue(ops, oracle):
    r = rng(21)
    M, N, K = 70, 136, 200
    a = r.standard_normal((M, K)).astype(np.float32) * 0.2
    b = r.standard_normal((K, N)).astype(np.float32) * 0.2
    bias = r.standard_normal(N).astype(np.float32)
    res = r.standard_normal((M, N)).astype(np.float32)
    base = oracle.matmul(a, b, "mkn")
    for act, alpha in [("none", 1.0), ("relu", 1.0), ("gelu", 0.125)]:
        want = base * np.float32(alpha) + bias[None, :] + res
        if act != "none":
            want = oracle.unary(act, want)
        epi = ops.Epilogue(alpha=alpha, bias=dev(bias), residual=dev(res), act=act)
        assert_close_f32(host(ops.matmul(dev(a), dev(b), epi)), want, "epilogue " + act)


@pytest.mark.parametrize("M,N,K,dt", [(70, 136, 200, torch.float32), (256, 256, 64, torch.float32), (384, 256, 128, torch.bfloat16),
                                      (128, 192, 128, torch.bfloat16), (1024, 768, 256, torch.bfloat16), (448, 768, 3072, torch.float32),
                                      (4096, 3072, 128, torch.bfloat16)])
def test_matmul_residual_may_be_the_output(ops, oracle, M, N, K, dt):
    """An in-place residual add (the residual operand is the result tensor): every kernel family reads a lane's residual
    values before it stores that lane's results, so the product is the same as with a separate result."""
    r = rng(77 + M + K)
    a = bf16_round(r.uniform(-1, 1, (M, K)) * 0.25)  # sums of 3072 products stay near the residual's size
    b = bf16_round(r.uniform(-1, 1, (K, N)) * 0.25)
    res = bf16_round(r.standard_normal((M, N)))
    bias = bf16_round(r.standard_normal(N))
    want = oracle.matmul(a, b, "mkn") + bias[None, :] + res
    inout = dev(res, dt)
    got = ops.matmul(dev(a, dt), dev(b, dt), ops.Epilogue(bias=dev(bias, dt), residual=inout), out=inout)
    assert got.data_ptr() == inout.data_ptr()
    if dt == torch.float32:
        assert_close_f32(host(got), want, "in-place residual f32 %dx%dx%d" % (M, N, K))
    else:
        assert_close_bf16(host(got), bf16_round(want.astype(np.float32)), "in-place residual bf16 %dx%dx%d" % (M, N, K))


def test_batch_matmul_residual_may_be_the_output(ops, oracle):
    """The same for the batched product with K = 64 (its kernel transposes a tile through LDS between reading the residual
    and storing the result)."""
    r = rng(91)
    B, M, K, N = 16, 512, 64, 512
    a = bf16_round(r.uniform(-1, 1, (B, M, K)) * 0.25)
    b = bf16_round(r.uniform(-1, 1, (B, K, N)) * 0.25)
    res = bf16_round(r.standard_normal((B, M, N)))
    want = np.stack([oracle.matmul(a[i], b[i], "mkn") for i in range(B)]) + res
    for dt, close in ((torch.float32, assert_close_f32), (torch.bfloat16, assert_close_bf16)):
        inout = dev(res, dt)
        got = ops.batch_matmul(dev(a, dt), dev(b, dt), ops.Epilogue(residual=inout), out=inout)
        assert got.data_ptr() == inout.data_ptr()
        close(host(got), want if dt == torch.float32 else bf16_round(want.astype(np.float32)), "in-place residual bmm %s" % dt)


@pytest.mark.parametrize("seed", range(4))
def test_random_matmul_cases(ops, oracle, seed):
    """Randomly drawn products: extents on both sides of every dispatch threshold (16 rows, complete 128-tiles,
    K of 1536 and more with few tiles), each operand plain or a transposed view, rows taken from a wider buffer,
    every storage type, random epilogues."""
    r = rng(500 + seed)
    dims_m = [1, 3, 16, 17, 64, 100, 128, 200, 256, 384]
    dims_n = [1, 8, 24, 64, 72, 128, 136, 256, 384]
    dims_k = [1, 8, 40, 64, 96, 256, 320, 1536, 2048]
    for trial in range(14):
        M, N, K = (int(d[r.integers(0, len(d))]) for d in (dims_m, dims_n, dims_k))
        if M * N * K > 60e6:
            K = 256
        dt, close, rnd = [(torch.float32, assert_close_f32, lambda x: x), (torch.bfloat16, assert_close_bf16, bf16_round),
                          (torch.float16, assert_close_bf16, lambda x: x)][int(r.integers(0, 3))]
        a = bf16_round(r.uniform(-1, 1, (M, K)))
        b = bf16_round(r.uniform(-1, 1, (K, N)))
        base = oracle.matmul(a, b, "mkn")
        lay_a, lay_b = int(r.integers(0, 3)), int(r.integers(0, 2))
        if lay_a == 0:
            da = dev(a, dt)
        elif lay_a == 1:
            da = dev(np.ascontiguousarray(a.T), dt).t()
        else:                                        # rows of a wider buffer: row pitch K + 16, 16-byte aligned start
            wide = np.zeros((M, K + 16), np.float32)
            wide[:, 8:8 + K] = a
            da = dev(wide, dt)[:, 8:8 + K]
        db = dev(b, dt) if lay_b == 0 else dev(np.ascontiguousarray(b.T), dt).t()
        epi, want = None, base
        if r.random() < 0.6:
            alpha = float(r.choice([1.0, 0.5, 0.125]))
            bias = bf16_round(r.standard_normal(N)) if r.random() < 0.7 else None
            res = bf16_round(r.standard_normal((M, N))) if r.random() < 0.5 else None
            act = str(r.choice(["none", "relu", "gelu"]))
            want = base * np.float32(alpha)
            if bias is not None:
                want = want + bias[None, :]
            if res is not None:
                want = want + res
            if act != "none":
                want = oracle.unary(act, want.astype(np.float32))
            epi = ops.Epilogue(alpha=alpha, bias=None if bias is None else dev(bias, dt),
                               residual=None if res is None else dev(res, dt), act=act)
        got = ops.matmul(da, db, epi)
        close(host(got), rnd(want.astype(np.float32)), "M=%d N=%d K=%d %s A-layout %d B-layout %d epilogue %s" % (
            M, N, K, dt, lay_a, lay_b, None if epi is None else (alpha, bias is not None, res is not None, act)))


@pytest.mark.parametrize("M,N,K", [(256, 192, 2048), (200, 132, 1536), (448, 768, 3072)])
def test_matmul_f32_long_reduction_few_tiles(ops, oracle, M, N, K):
    """Products whose reduction is cut into chunks (few output tiles, K >= 1536): the chunk sums (fp32 whatever the
    storage type) are added in a fixed order and the epilogue runs once, after the sum.  Both weight layouts, with
    and without epilogue, every storage type."""
    r = rng(M + N + K)
    a = r.uniform(-1, 1, (M, K)).astype(np.float32) * 0.25
    b = r.uniform(-1, 1, (K, N)).astype(np.float32) * 0.25
    bias = r.standard_normal(N).astype(np.float32)
    res = r.standard_normal((M, N)).astype(np.float32)
    base = oracle.matmul(a, b, "mkn")
    bt = dev(np.ascontiguousarray(b.T))
    assert_close_f32(host(ops.matmul(dev(a), dev(b))), base, "NN %s" % ((M, N, K),))
    first = host(ops.matmul(dev(a), bt.t()))
    assert_close_f32(first, base, "NT %s" % ((M, N, K),))
    np.testing.assert_array_equal(host(ops.matmul(dev(a), bt.t())), first)  # the same bits on every run
    for act, alpha in [("none", 1.0), ("relu", 0.5), ("gelu", 0.125)]:
        want = base * np.float32(alpha) + bias[None, :] + res
        if act != "none":
            want = oracle.unary(act, want)
        epi = ops.Epilogue(alpha=alpha, bias=dev(bias), residual=dev(res), act=act)
        assert_close_f32(host(ops.matmul(dev(a), bt.t(), epi)), want, "NT epilogue %s %s" % (act, (M, N, K)))
    # the 16-bit types split the same way (fp32 partial sums, one rounding at the end)
    ab, bb, biasb, resb = bf16_round(a), bf16_round(b), bf16_round(bias), bf16_round(res)
    baseb = oracle.matmul(ab, bb, "mkn")
    for dt, rnd in ((torch.bfloat16, bf16_round), (torch.float16, lambda x: x)):
        btd = dev(np.ascontiguousarray(bb.T), dt)
        firstb = host(ops.matmul(dev(ab, dt), btd.t()))
        assert_close_bf16(firstb, rnd(baseb), "NT %s %s" % (dt, (M, N, K)))
        np.testing.assert_array_equal(host(ops.matmul(dev(ab, dt), btd.t())), firstb)
        assert_close_bf16(host(ops.matmul(dev(ab, dt), dev(bb, dt))), rnd(baseb), "NN %s %s" % (dt, (M, N, K)))
        want = oracle.unary("gelu", baseb * np.float32(0.125) + biasb[None, :] + resb)
        epi = ops.Epilogue(alpha=0.125, bias=dev(biasb, dt), residual=dev(resb, dt), act="gelu")
        assert_close_bf16(host(ops.matmul(dev(ab, dt), btd.t(), epi)), rnd(want), "NT epilogue %s %s" % (dt, (M, N, K)))


@pytest.mark.parametrize("B,M,N,K", [(3, 9, 4, 6), (4, 64, 64, 64), (6, 128, 128, 64), (5, 100, 64, 100), (2, 130, 70, 36)])
def test_batch_matmul(ops, oracle, B, M, N, K):
    r = rng(B + M + N + K)
    a = r.uniform(-1, 1, (B, M, K)).astype(np.float32)
    b = r.uniform(-1, 1, (B, K, N)).astype(np.float32)
    want = oracle.batch_matmul(a, b, "mkn")
    assert_close_f32(host(ops.batch_matmul(dev(a), dev(b))), want, "bmm f32")
    # QK^T form: rhs is the transposed view of [B,N,K]
    bt = dev(np.ascontiguousarray(b.transpose(0, 2, 1)))
    assert_close_f32(host(ops.batch_matmul(dev(a), bt.transpose(1, 2))), want, "bmm f32 NT")
    ab, bb = bf16_round(a), bf16_round(b)
    gotb = ops.batch_matmul(dev(ab, torch.bfloat16), dev(bb, torch.bfloat16))
    assert_close_bf16(host(gotb), bf16_round(oracle.batch_matmul(ab, bb, "mkn")), "bmm bf16")


def test_batch_matmul_two_level_batches(ops, oracle):
    """Rank-4 operands [B0, B1, M, K]: the attention head split read in place from a [B, S, H*D] activation
    (q and v as permuted views, k as the permuted and transposed view), against the oracle on materialised
    copies.  fp32 (register-staged kernel) and bf16 (direct-to-LDS kernel for the scores shape)."""
    r = rng(91)
    B, S, H, D = 4, 256, 8, 64
    q = r.uniform(-1, 1, (B, S, H * D)).astype(np.float32)
    k = r.uniform(-1, 1, (B, S, H * D)).astype(np.float32)
    v = r.uniform(-1, 1, (B, S, H * D)).astype(np.float32)
    heads = lambda x: np.ascontiguousarray(x.reshape(B, S, H, D).transpose(0, 2, 1, 3)).reshape(B * H, S, D)
    kt = np.ascontiguousarray(heads(k).transpose(0, 2, 1))
    for dt, close, rnd in ((torch.float32, assert_close_f32, lambda x: x), (torch.bfloat16, assert_close_bf16, bf16_round)):
        qd, kd, vd = (dev(rnd(x), dt) for x in (q, k, v))
        q4 = qd.view(B, S, H, D).permute(0, 2, 1, 3)
        k4 = kd.view(B, S, H, D).permute(0, 2, 3, 1)
        v4 = vd.view(B, S, H, D).permute(0, 2, 1, 3)
        scores = ops.batch_matmul(q4, k4, ops.Epilogue(alpha=0.125))
        want = oracle.batch_matmul(heads(rnd(q)), np.ascontiguousarray(heads(rnd(k)).transpose(0, 2, 1)), "mkn") * np.float32(0.125)
        assert tuple(scores.shape) == (B * H, S, S)
        close(host(scores), rnd(want), "scores %s" % dt)
        # an attention mask [B,1,1,S] as one bias row per outer batch
        mask = rnd(np.where(r.uniform(0, 1, (B, S)) < 0.2, -1e4, 0.0).astype(np.float32))
        masked = ops.batch_matmul(q4, k4, ops.Epilogue(alpha=0.125, bias=dev(mask, dt)))
        wantm = want.reshape(B, H, S, S) + mask[:, None, None, :]
        close(host(masked).reshape(B, H, S, S), rnd(wantm), "masked scores %s" % dt)
        # one-level lhs with a two-level rhs
        p = r.uniform(0, 1, (B * H, S, S)).astype(np.float32)
        ctx = ops.batch_matmul(dev(rnd(p), dt), v4)
        want_ctx = rnd(oracle.batch_matmul(rnd(p), heads(rnd(v)), "mkn"))
        close(host(ctx), want_ctx, "context %s" % dt)
        # the head merge written in place: out is the [B, H, S, D] view of a [B, S, H*D] buffer
        merged = torch.zeros(B, S, H * D, dtype=dt, device="cuda")
        ops.batch_matmul(dev(rnd(p), dt), v4, out=merged.view(B, S, H, D).permute(0, 2, 1, 3))
        close(host(merged), want_ctx.reshape(B, H, S, D).transpose(0, 2, 1, 3).reshape(B, S, H * D), "merged context %s" % dt)
    del kt


def test_matmul_shape_errors(ops):
    from llcompiler_amd._capi import LlcHipError
    with pytest.raises(LlcHipError, match="matmul"):
        ops.matmul(torch.zeros(3, 4, device="cuda"), torch.zeros(5, 6, device="cuda"), out=torch.zeros(3, 6, device="cuda"))
    with pytest.raises(LlcHipError):
        ops.matmul(torch.zeros(3, 4, device="cuda"), torch.zeros(4, 6, device="cuda", dtype=torch.bfloat16),
                   out=torch.zeros(3, 6, device="cuda"))


CONV_CASES = [
    # N, C, H, W, F, KH, KW, pad(h,w), stride, dil, group
    (2, 3, 9, 11, 4, 3, 3, (1, 1), (1, 1), (1, 1), 1),
    (1, 3, 33, 29, 64, 7, 7, (3, 3), (2, 2), (1, 1), 1),   # stem-like, K = 147
    (2, 4, 10, 12, 6, 3, 2, (2, 0), (2, 1), (1, 2), 2),
    (1, 6, 8, 8, 6, 3, 3, (1, 2), (1, 3), (2, 1), 6),
    (2, 64, 14, 14, 128, 1, 1, (0, 0), (2, 2), (1, 1), 1),  # 1x1 stride-2 downsample
    (3, 3, 12, 12, 2, 5, 5, (2, 2), (1, 1), (1, 1), 1),
    (2, 64, 14, 14, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1),   # basic-block conv
    (2, 128, 7, 7, 256, 3, 3, (1, 1), (2, 2), (1, 1), 1),
    (2, 8, 15, 13, 72, 3, 3, (1, 1), (1, 1), (1, 1), 1),    # rows of 13 pixels: 4-pixel gathers straddle row ends
    (1, 16, 20, 20, 32, 3, 3, (2, 2), (1, 1), (2, 2), 1),   # dilated, stride 1
    (2, 8, 12, 16, 16, 3, 3, (1, 1), (1, 1), (1, 1), 2),    # groups, stride 1
    (4, 256, 7, 7, 128, 3, 3, (1, 1), (1, 1), (1, 1), 1),   # few pixels, deep reduction: split over k
    (2, 3, 32, 224, 64, 7, 7, (3, 3), (2, 2), (1, 1), 1),   # an image network's first layer: 3 channels, 7x7 window, stride 2
    (3, 3, 8, 192, 64, 7, 7, (3, 3), (2, 2), (1, 1), 1),    # the same on images of 8 rows: mostly padding rows
    (1, 3, 20, 236, 64, 7, 7, (2, 2), (2, 2), (1, 1), 1),   # pad 2, rows of 117 outputs
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d(ops, oracle, case):
    N, C, H, W, Fo, KH, KW, p, s, d, g = case
    r = rng(sum(case[:7]))
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    fan = (C // g) * KH * KW
    w = (r.standard_normal((Fo, C // g, KH, KW)) / np.sqrt(fan)).astype(np.float32)
    b = r.standard_normal(Fo).astype(np.float32)
    pad = (p[0], p[1], p[0], p[1])
    want = oracle.conv2d(x, w, None, pad=pad, stride=s, dilation=d, group=g)
    got = ops.conv2d(dev(x), dev(w), pad=pad, stride=s, dilation=d, group=g)
    assert_close_f32(host(got), want, "conv %s" % (case,))
    # conv_bias + relu + residual epilogue (a ResNet basic block tail)
    res = r.standard_normal(want.shape).astype(np.float32)
    want2 = oracle.unary("relu", oracle.conv2d(x, w, b, pad=pad, stride=s, dilation=d, group=g) + res)
    epi = ops.Epilogue(bias=dev(b), residual=dev(res), act="relu")
    assert_close_f32(host(ops.conv2d(dev(x), dev(w), pad=pad, stride=s, dilation=d, group=g, epilogue=epi)), want2,
                     "conv+bias+res+relu %s" % (case,))
    xb, wb = bf16_round(x), bf16_round(w)
    gotb = ops.conv2d(dev(xb, torch.bfloat16), dev(wb, torch.bfloat16), pad=pad, stride=s, dilation=d, group=g)
    assert_close_bf16(host(gotb), bf16_round(oracle.conv2d(xb, wb, None, pad=pad, stride=s, dilation=d, group=g)),
                      "conv bf16 %s" % (case,))


NHWC_CASES = [
    # N, C, H, W, F, KH, KW, pad(h_lo, w_lo, h_hi, w_hi), stride, dil
    (2, 64, 14, 14, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # basic-block conv
    (2, 64, 15, 13, 128, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1)),     # stride 2, odd extents
    (2, 64, 14, 14, 128, 1, 1, (0, 0, 0, 0), (2, 2), (1, 1)),     # 1x1 stride-2 downsample
    (1, 32, 20, 20, 68, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),      # dilated; 68 filters: a partial filter tile
    (3, 32, 9, 11, 8, 5, 3, (2, 0, 1, 2), (1, 2), (1, 1)),        # asymmetric window, pad and stride
    (4, 256, 7, 7, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # few pixels, deep reduction: split over k
    (1, 96, 5, 5, 4, 7, 7, (3, 3, 3, 3), (1, 1), (1, 1)),         # 49 taps, windows larger than the image
    (2, 128, 28, 28, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),    # 1568 pixels: 64-pixel tiles, no split
    (1, 192, 6, 9, 36, 3, 3, (1, 0, 2, 1), (1, 1), (1, 1)),       # 16-bit k-tiles of 64 in 192 channels, partial filter tile
]


@pytest.mark.parametrize("case", [NHWC_CASES[0], NHWC_CASES[5], NHWC_CASES[7]])
def test_conv2d_channels_last_residual_may_be_the_output(ops, oracle, case):
    """A residual block's add done in place (the residual operand is the result tensor), on the tile kernel, the split
    reduction and, in bf16, the input-patch kernel: a lane reads its residual values before it stores its results."""
    N, C, H, W, Fo, KH, KW, pad, s, d = case
    r = rng(sum(case[:7]) + 5)
    x = bf16_round(r.standard_normal((N, C, H, W)))
    w = bf16_round(r.standard_normal((Fo, C, KH, KW)) / np.sqrt(C * KH * KW))
    b = bf16_round(r.standard_normal(Fo))
    conv = oracle.conv2d(x, w, b, pad=pad, stride=s, dilation=d)
    res = bf16_round(r.standard_normal(conv.shape))
    want = oracle.unary("relu", conv + res)
    cl = torch.channels_last
    for dt, close in ((torch.float32, assert_close_f32), (torch.bfloat16, assert_close_bf16)):
        inout = dev(res, dt).contiguous(memory_format=cl)
        got = ops.conv2d(dev(x, dt).contiguous(memory_format=cl), dev(w, dt).contiguous(memory_format=cl), pad=pad, stride=s,
                         dilation=d, epilogue=ops.Epilogue(bias=dev(b, dt), residual=inout, act="relu"), out=inout)
        assert got.data_ptr() == inout.data_ptr()
        close(host(got), want if dt == torch.float32 else bf16_round(want), "in-place residual conv %s %s" % (dt, case))


@pytest.mark.parametrize("case", NHWC_CASES)
def test_conv2d_channels_last(ops, oracle, case):
    """The same entry point with the layout in the strides: x, weight, output and residual channels-last (NHWC in
    memory, logical shape NCHW) take the kernel that reads the im2col rows as contiguous runs."""
    N, C, H, W, Fo, KH, KW, pad, s, d = case
    r = rng(sum(case[:7]) + 1)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = (r.standard_normal((Fo, C, KH, KW)) / np.sqrt(C * KH * KW)).astype(np.float32)
    b = r.standard_normal(Fo).astype(np.float32)
    want = oracle.conv2d(x, w, None, pad=pad, stride=s, dilation=d)
    cl = torch.channels_last
    dx, dw = dev(x).contiguous(memory_format=cl), dev(w).contiguous(memory_format=cl)
    out = torch.empty(want.shape, device="cuda").contiguous(memory_format=cl)
    got = ops.conv2d(dx, dw, pad=pad, stride=s, dilation=d, out=out)
    assert got.is_contiguous(memory_format=cl)
    assert_close_f32(host(got), want, "channels-last conv %s" % (case,))
    res = r.standard_normal(want.shape).astype(np.float32)
    want2 = oracle.unary("relu", oracle.conv2d(x, w, b, pad=pad, stride=s, dilation=d) * np.float32(1.0) + res)
    epi = ops.Epilogue(bias=dev(b), residual=dev(res).contiguous(memory_format=cl), act="relu")
    out2 = torch.empty(want.shape, device="cuda").contiguous(memory_format=cl)
    assert_close_f32(host(ops.conv2d(dx, dw, pad=pad, stride=s, dilation=d, epilogue=epi, out=out2)), want2,
                     "channels-last conv+bias+res+relu %s" % (case,))
    if C % 64:
        return
    # the 16-bit types: a k-tile is 64 channels of one tap; products of the rounded operands summed in fp32
    xb, wb, bb, rb = bf16_round(x), bf16_round(w), bf16_round(b), bf16_round(res)
    wantb = oracle.conv2d(xb, wb, None, pad=pad, stride=s, dilation=d)
    wantb2 = oracle.unary("relu", wantb * np.float32(1.0) + bb[None, :, None, None] + rb)
    for dt in (torch.bfloat16, torch.float16):
        tx, tw = dev(xb, dt).contiguous(memory_format=cl), dev(wb, dt).contiguous(memory_format=cl)
        o = torch.empty(want.shape, device="cuda", dtype=dt).contiguous(memory_format=cl)
        g = ops.conv2d(tx, tw, pad=pad, stride=s, dilation=d, out=o)
        assert g.is_contiguous(memory_format=cl)
        assert_close_bf16(host(g), wantb, "channels-last conv %s %s" % (dt, case))
        epi = ops.Epilogue(bias=dev(bb, dt), residual=dev(rb, dt).contiguous(memory_format=cl), act="relu")
        o2 = torch.empty(want.shape, device="cuda", dtype=dt).contiguous(memory_format=cl)
        assert_close_bf16(host(ops.conv2d(tx, tw, pad=pad, stride=s, dilation=d, epilogue=epi, out=o2)), wantb2,
                          "channels-last conv+bias+res+relu %s %s" % (dt, case))


ROW_CONV_CASES = [
    # N, C, H, W, KH, KW, pad(h_lo, w_lo, h_hi, w_hi), stride: fp32 NCHW, 64 filters, reduction <= 148, stride 2 along w
    (4, 3, 128, 128, 7, 7, (3, 3, 3, 3), (2, 2)),     # an image network's first layer
    (6, 3, 98, 200, 7, 7, (3, 3, 3, 3), (2, 2)),      # 100 output columns: the last pixel block is partly outside
    (2, 4, 130, 224, 5, 7, (2, 2, 1, 3), (1, 2)),     # 4 channels, 5 x 7 window, stride 1 along h, asymmetric pads
    (5, 2, 60, 64, 7, 5, (0, 2, 3, 2), (1, 2)),       # no padding on top, 32 output columns
]


@pytest.mark.parametrize("case", ROW_CONV_CASES)
def test_conv2d_first_layer_row_kernel(ops, oracle, case):
    """Few input channels, a large window, stride 2: the kernel that keeps the input rows under the window in LDS as
    they lie in memory and feeds the MFMAs from them (64 filters; zeros left, right, above and below come from the
    padding columns of the LDS rows and from a row of zeros)."""
    N, C, H, W, KH, KW, pad, s = case
    r = rng(sum(case[:6]) + 9)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = (r.standard_normal((64, C, KH, KW)) / np.sqrt(C * KH * KW)).astype(np.float32)
    b = r.standard_normal(64).astype(np.float32)
    want = oracle.conv2d(x, w, None, pad=pad, stride=s)
    assert want.shape[0] * want.shape[2] >= 256 and want.shape[3] % 4 == 0
    assert_close_f32(host(ops.conv2d(dev(x), dev(w), pad=pad, stride=s)), want, "first-layer conv %s" % (case,))
    want2 = oracle.unary("relu", (oracle.conv2d(x, w, b, pad=pad, stride=s) * np.float32(1.0)).astype(np.float32))
    epi = ops.Epilogue(bias=dev(b), act="relu")
    assert_close_f32(host(ops.conv2d(dev(x), dev(w), pad=pad, stride=s, epilogue=epi)), want2, "first-layer conv + bias + relu")
    want3 = oracle.conv2d(x, w, None, pad=pad, stride=s) * np.float32(0.25)
    assert_close_f32(host(ops.conv2d(dev(x), dev(w), pad=pad, stride=s, epilogue=ops.Epilogue(alpha=0.25))), want3, "alpha")
    # 16-bit storage: the same kernel on fp32 copies of the image and the filters, the result rounded on its way out
    xb, wb, bb = bf16_round(x), bf16_round(w), bf16_round(b)
    want16 = oracle.unary("relu", oracle.conv2d(xb, wb, bb, pad=pad, stride=s))
    for dt, rnd, close in ((torch.bfloat16, bf16_round, assert_close_bf16), (torch.float16, f16_round, assert_close_f16)):
        epi = ops.Epilogue(bias=dev(bb, dt), act="relu")
        got = ops.conv2d(dev(xb, dt), dev(wb, dt), pad=pad, stride=s, epilogue=epi)
        assert got.dtype == dt
        close(host(got), rnd(want16), "first-layer conv + bias + relu %s %s" % (dt, case))


@pytest.mark.parametrize("case", ROW_CONV_CASES)
def test_conv2d_first_layer_channels_last_result(ops, oracle, case):
    """The first-layer kernels with NCHW operands and a channels-last result (what the channels-last layers after
    them read), fp32 and 16-bit, with bias + relu; other shapes in that combination are refused."""
    N, C, H, W, KH, KW, pad, s = case
    r = rng(sum(case[:6]) + 10)
    x = bf16_round(r.standard_normal((N, C, H, W)))
    w = bf16_round(r.standard_normal((64, C, KH, KW)) / np.sqrt(C * KH * KW))
    b = bf16_round(r.standard_normal(64))
    plain = oracle.conv2d(x, w, None, pad=pad, stride=s)
    want = oracle.unary("relu", oracle.conv2d(x, w, b, pad=pad, stride=s))
    cl = torch.channels_last
    for dt, rnd, close in ((torch.float32, lambda v: v, assert_close_f32), (torch.bfloat16, bf16_round, assert_close_bf16),
                           (torch.float16, f16_round, assert_close_f16)):
        o = torch.empty(want.shape, device="cuda", dtype=dt).contiguous(memory_format=cl)
        got = ops.conv2d(dev(x, dt), dev(w, dt), pad=pad, stride=s, out=o)
        assert got.is_contiguous(memory_format=cl) and not got.is_contiguous()
        close(host(got), rnd(plain), "first-layer conv, channels-last result %s %s" % (dt, case))
        o2 = torch.empty(want.shape, device="cuda", dtype=dt).contiguous(memory_format=cl)
        got = ops.conv2d(dev(x, dt), dev(w, dt), pad=pad, stride=s, epilogue=ops.Epilogue(bias=dev(b, dt), act="relu"), out=o2)
        close(host(got), rnd(want), "first-layer conv + bias + relu, channels-last result %s %s" % (dt, case))
    # stride 1 along w is no first-layer shape: NCHW operands with a channels-last result have no kernel there
    o = torch.empty((N, 64, H, W), device="cuda").contiguous(memory_format=cl)
    with pytest.raises(RuntimeError):
        ops.conv2d(dev(x), dev(w), pad=(KH // 2, KW // 2, KH // 2, KW // 2), stride=(1, 1), out=o)


def test_conv2d_first_layer_16bit_infinite_pixel_stays_in_its_windows(ops, oracle):
    """The 16-bit first-layer kernel reads eight window columns per matrix-instruction operand for a 7-wide window
    (the eighth against a zero filter value): an infinite pixel in that extra column must not reach the sum."""
    r = rng(77)
    x = bf16_round(r.standard_normal((4, 3, 128, 128)))
    x[1, 2, 40, 51] = np.inf
    x[2, 0, 0, 0] = -np.inf
    w = bf16_round(r.standard_normal((64, 3, 7, 7)) / np.sqrt(147))
    pad, s = (3, 3, 3, 3), (2, 2)
    want = bf16_round(oracle.conv2d(x, w, None, pad=pad, stride=s))
    for out_cl in (False, True):
        o = torch.empty(want.shape, device="cuda", dtype=torch.bfloat16)
        if out_cl:
            o = o.contiguous(memory_format=torch.channels_last)
        got = host(ops.conv2d(dev(x, torch.bfloat16), dev(w, torch.bfloat16), pad=pad, stride=s, out=o))
        fin = np.isfinite(want)
        assert 0 < (~fin).sum() < want.size // 100
        np.testing.assert_array_equal(np.isfinite(got), fin)
        assert_close_bf16(got[fin], want[fin], "finite outputs beside an infinite pixel")


PATCH_CONV_CASES = [
    # N, H, W, F, KH, KW, pad(h_lo, w_lo, h_hi, w_hi): 64 channels in 16-bit storage, stride 1, at least 192 tiles
    (16, 56, 56, 64, 3, 3, (1, 1, 1, 1)),     # a ResNet's first stage: 24 whole tiles and one of 64 pixels per image
    (9, 30, 50, 128, 3, 3, (1, 1, 1, 1)),     # 1500 pixels per image (the last tile has 92), two filter tiles
    (20, 33, 41, 64, 3, 2, (0, 1, 2, 0)),     # 3 x 2 window, no padding above, two rows below, none on the right
    (12, 48, 48, 64, 5, 5, (2, 2, 2, 2)),     # 5 x 5 window: 25 taps, a patch of 7 rows of 52 pixels
]


@pytest.mark.parametrize("case", PATCH_CONV_CASES)
def test_conv2d_channels_last_16bit_input_patch_in_lds(ops, oracle, case):
    """Stride-1 windows over 64 channels in 16-bit storage: the kernel that parks the input patch of 128 output pixels
    in LDS once and reads every tap from it at a shifted address (zeros around the image come from a row of zeros);
    bf16 and f16, with and without bias + residual + relu."""
    N, H, W, F, KH, KW, pad = case
    r = rng(N + H + W + F + KH)
    x = bf16_round(r.standard_normal((N, 64, H, W)))
    w = bf16_round(r.standard_normal((F, 64, KH, KW)) / np.sqrt(64 * KH * KW))
    b = bf16_round(r.standard_normal(F))
    base = oracle.conv2d(x, w, None, pad=pad)
    res = bf16_round(r.standard_normal(base.shape))
    assert base.shape[0] * ((base.shape[2] * base.shape[3] + 127) // 128) * (F // 64) >= 192
    cl = torch.channels_last
    for dt, rnd, close in ((torch.bfloat16, bf16_round, assert_close_bf16), (torch.float16, f16_round, assert_close_f16)):
        dx, dw = dev(x, dt).contiguous(memory_format=cl), dev(w, dt).contiguous(memory_format=cl)
        o = torch.empty(base.shape, device="cuda", dtype=dt).contiguous(memory_format=cl)
        close(host(ops.conv2d(dx, dw, pad=pad, out=o)), rnd(base), "patch conv %s %s" % (dt, case))
        want = oracle.unary("relu", oracle.conv2d(x, w, b, pad=pad) + res)
        epi = ops.Epilogue(bias=dev(b, dt), residual=dev(res, dt).contiguous(memory_format=cl), act="relu")
        o2 = torch.empty(base.shape, device="cuda", dtype=dt).contiguous(memory_format=cl)
        close(host(ops.conv2d(dx, dw, pad=pad, epilogue=epi, out=o2)), rnd(want), "patch conv+bias+res+relu %s %s" % (dt, case))


WIDE_CONV_CASES = [
    # N, C, H, W, F, KH, KW, pad, stride, dil: reductions of 2048 and more, at least 192 tiles of 256 pixels x 128 (256) filters
    (17, 256, 54, 54, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # 49572 pixels: the last tile has 164 rows
    (16, 256, 112, 112, 128, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1)),   # stride 2
    (13, 128, 66, 66, 256, 4, 4, (1, 0, 2, 1), (1, 1), (2, 1)),     # 256-filter tiles, even window, dilation, asymmetric pads
]


@pytest.mark.parametrize("case", WIDE_CONV_CASES)
def test_conv2d_channels_last_16bit_on_wide_tiles(ops, oracle, case):
    """Channels-last 16-bit convolutions with work for the whole chip and a long reduction run on the wide-tile matmul
    kernel, the image as its row operand (windows gathered by the loads, taps outside the image read as zeros).  The
    oracle evaluates the first and the last image of the batch (samples are independent; the last one holds the
    incomplete tile)."""
    N, C, H, W, Fo, KH, KW, pad, s, d = case
    r = rng(sum(case[:7]) + 3)
    cl = torch.channels_last
    xb = bf16_round(r.standard_normal((N, C, H, W)))
    wb = bf16_round(r.standard_normal((Fo, C, KH, KW)) / np.sqrt(C * KH * KW))
    bb = bf16_round(r.standard_normal(Fo))
    pick = [0, N - 1]
    wantb = oracle.conv2d(xb[pick], wb, None, pad=pad, stride=s, dilation=d)
    full = (N,) + wantb.shape[1:]
    assert (N * full[2] * full[3] + 255) // 256 * (Fo // 128) >= 192 and C * KH * KW >= 2048
    rb = bf16_round(r.standard_normal(full))
    wantb2 = oracle.unary("relu", (wantb * np.float32(0.5) + bb[None, :, None, None] + rb[pick]).astype(np.float32))
    for dt in (torch.bfloat16, torch.float16):
        tx, tw = dev(xb, dt).contiguous(memory_format=cl), dev(wb, dt).contiguous(memory_format=cl)
        o = torch.empty(full, device="cuda", dtype=dt).contiguous(memory_format=cl)
        g = ops.conv2d(tx, tw, pad=pad, stride=s, dilation=d, out=o)
        assert_close_bf16(host(g)[pick], wantb, "wide channels-last conv %s %s" % (dt, case))
        epi = ops.Epilogue(alpha=0.5, bias=dev(bb, dt), residual=dev(rb, dt).contiguous(memory_format=cl), act="relu")
        o2 = torch.empty(full, device="cuda", dtype=dt).contiguous(memory_format=cl)
        assert_close_bf16(host(ops.conv2d(tx, tw, pad=pad, stride=s, dilation=d, epilogue=epi, out=o2))[pick], wantb2,
                          "wide channels-last conv with epilogue %s %s" % (dt, case))


@pytest.mark.parametrize("seed", range(4))
def test_random_conv_cases(ops, oracle, seed):
    """Randomly drawn convolutions: window, stride, dilation, asymmetric pads, groups, channel and filter counts on
    both sides of what each kernel takes (reduction a multiple of 4 or not, channels a multiple of 32 or not), NCHW
    and channels-last, fp32 and bf16, with and without the epilogue."""
    r = rng(700 + seed)
    cl = torch.channels_last
    done = 0
    while done < 10:
        g = int(r.choice([1, 1, 1, 2, 4]))
        C = g * int(r.choice([1, 2, 3, 8, 16, 32]))
        Fo = g * int(r.choice([1, 2, 4, 5, 16, 33, 64]))
        if g == 1 and r.random() < 0.4:
            C = int(r.choice([32, 64, 96, 128]))
        KH, KW = int(r.choice([1, 2, 3, 5])), int(r.choice([1, 2, 3, 5]))
        s = (int(r.integers(1, 3)), int(r.integers(1, 3)))
        d = (int(r.integers(1, 3)), int(r.integers(1, 3)))
        pad = tuple(int(v) for v in r.integers(0, 3, 4))
        N, H, W = int(r.integers(1, 4)), int(r.integers(4, 19)), int(r.integers(4, 19))
        oh = (H + pad[0] + pad[2] - d[0] * (KH - 1) - 1) // s[0] + 1
        ow = (W + pad[1] + pad[3] - d[1] * (KW - 1) - 1) // s[1] + 1
        if oh < 1 or ow < 1:
            continue
        done += 1
        x = r.standard_normal((N, C, H, W)).astype(np.float32)
        w = (r.standard_normal((Fo, C // g, KH, KW)) / np.sqrt((C // g) * KH * KW)).astype(np.float32)
        b = r.standard_normal(Fo).astype(np.float32)
        what = "N%d C%d %dx%d F%d k%dx%d s%s d%s pad%s g%d" % (N, C, H, W, Fo, KH, KW, s, d, pad, g)
        want = oracle.conv2d(x, w, None, pad=pad, stride=s, dilation=d, group=g)
        res = r.standard_normal(want.shape).astype(np.float32)
        kw = dict(pad=pad, stride=s, dilation=d, group=g)
        assert_close_f32(host(ops.conv2d(dev(x), dev(w), **kw)), want, what)
        # the epilogue is act(alpha * acc + bias + residual): bias is added after the scaling
        want3 = oracle.unary("relu", want * np.float32(0.5) + b[None, :, None, None] + res)
        epi = ops.Epilogue(alpha=0.5, bias=dev(b), residual=dev(res), act="relu")
        assert_close_f32(host(ops.conv2d(dev(x), dev(w), epilogue=epi, **kw)), want3, what + " with epilogue")
        xb, wb = bf16_round(x), bf16_round(w)
        gotb = ops.conv2d(dev(xb, torch.bfloat16), dev(wb, torch.bfloat16), **kw)
        assert_close_bf16(host(gotb), bf16_round(oracle.conv2d(xb, wb, None, pad=pad, stride=s, dilation=d, group=g)), what + " bf16")
        if g == 1 and C % 32 == 0 and Fo % 4 == 0 and KH * KW <= 64:
            dx, dw = dev(x).contiguous(memory_format=cl), dev(w).contiguous(memory_format=cl)
            out = torch.empty(want.shape, device="cuda").contiguous(memory_format=cl)
            epi = ops.Epilogue(alpha=0.5, bias=dev(b), residual=dev(res).contiguous(memory_format=cl), act="relu")
            assert_close_f32(host(ops.conv2d(dx, dw, epilogue=epi, out=out, **kw)), want3, what + " channels-last")
            if C % 64 == 0:
                tx, tw = dev(xb, torch.bfloat16).contiguous(memory_format=cl), dev(wb, torch.bfloat16).contiguous(memory_format=cl)
                o = torch.empty(want.shape, device="cuda", dtype=torch.bfloat16).contiguous(memory_format=cl)
                assert_close_bf16(host(ops.conv2d(tx, tw, out=o, **kw)),
                                  bf16_round(oracle.conv2d(xb, wb, None, pad=pad, stride=s, dilation=d, group=g)), what + " channels-last bf16")


def test_conv2d_layouts_must_agree(ops):
    from llcompiler_amd._capi import LlcHipError
    cl = torch.channels_last
    x = torch.zeros((1, 32, 6, 6), device="cuda")
    w = torch.zeros((8, 32, 3, 3), device="cuda")
    with pytest.raises(LlcHipError):  # channels-last input, NCHW weight and output
        ops.conv2d(x.contiguous(memory_format=cl), w, pad=(1, 1, 1, 1))
    x48 = torch.zeros((1, 48, 6, 6), device="cuda").contiguous(memory_format=cl)  # 48 channels: not a multiple of 32
    w48 = torch.zeros((8, 48, 3, 3), device="cuda").contiguous(memory_format=cl)
    with pytest.raises(LlcHipError):
        ops.conv2d(x48, w48, pad=(1, 1, 1, 1), out=torch.empty((1, 8, 6, 6), device="cuda").contiguous(memory_format=cl))
    # 32 channels of a 16-bit type are half a k-tile
    xh = torch.zeros((1, 32, 6, 6), device="cuda", dtype=torch.bfloat16).contiguous(memory_format=cl)
    wh = torch.zeros((8, 32, 3, 3), device="cuda", dtype=torch.bfloat16).contiguous(memory_format=cl)
    with pytest.raises(LlcHipError):
        ops.conv2d(xh, wh, pad=(1, 1, 1, 1), out=torch.empty((1, 8, 6, 6), device="cuda", dtype=torch.bfloat16).contiguous(memory_format=cl))


def test_conv2d_asymmetric_pad(ops, oracle):
    r = rng(31)
    x = r.standard_normal((1, 2, 6, 7)).astype(np.float32)
    w = r.standard_normal((3, 2, 3, 3)).astype(np.float32)
    pad = (2, 0, 1, 3)
    assert_close_f32(host(ops.conv2d(dev(x), dev(w), pad=pad)), oracle.conv2d(x, w, None, pad=pad))


def test_max_pool_and_avg_pool(ops, oracle):
    r = rng(32)
    x = r.standard_normal((2, 3, 23, 27)).astype(np.float32)
    for k, p, s, d in [((3, 3), (1, 1), (2, 2), (1, 1)), ((5, 5), (2, 2), (1, 1), (2, 2)), ((2, 3), (1, 0), (2, 1), (2, 1)),
                       ((7, 7), (3, 1), (2, 2), (2, 1))]:
        pad = (p[0], p[1], p[0], p[1])
        for iz in (False, True):
            got = ops.max_pool(dev(x), k, pad=pad, stride=s, dilation=d, init_zero=iz)
            np.testing.assert_array_equal(host(got), oracle.maxpool2d(x, k, pad=pad, stride=s, dilation=d, init_zero=iz))
    y = r.standard_normal((4, 6, 7, 7)).astype(np.float32)
    assert_close_f32(host(ops.global_avg_pool(dev(y))), oracle.global_avgpool(y))


def test_max_pool_and_avg_pool_channels_last(ops, oracle):
    """Channels-last tensors (NHWC in memory under NCHW shapes): the pooling kernels read and write them as they lie.
    The maximum is one of the inputs, so 16-bit results are exact too."""
    r = rng(33)
    cl = torch.channels_last
    for C in (8, 64, 72):
        x = bf16_round(r.standard_normal((3, C, 21, 26)))
        x[0, 1, 3, 4] = np.nan
        for k, p, s, d in [((3, 3), (1, 1), (2, 2), (1, 1)), ((2, 2), (0, 0), (2, 2), (1, 1)), ((5, 5), (2, 2), (1, 1), (2, 2)),
                           ((2, 3), (1, 0), (2, 1), (2, 1))]:
            pad = (p[0], p[1], p[0], p[1])
            for iz in (False, True):
                want = oracle.maxpool2d(x, k, pad=pad, stride=s, dilation=d, init_zero=iz)
                for dt in (torch.float32, torch.bfloat16, torch.float16):
                    xs = x if dt != torch.float16 else f16_round(x)
                    ws = want if dt != torch.float16 else oracle.maxpool2d(xs, k, pad=pad, stride=s, dilation=d, init_zero=iz)
                    o = torch.empty(want.shape, device="cuda", dtype=dt).contiguous(memory_format=cl)
                    got = ops.max_pool(dev(xs, dt).contiguous(memory_format=cl), k, pad=pad, stride=s, dilation=d, init_zero=iz, out=o)
                    assert got.is_contiguous(memory_format=cl)
                    np.testing.assert_array_equal(host(got), ws)
    # channel counts without 16-byte runs are refused, and so are mixed layouts
    x = dev(r.standard_normal((2, 6, 9, 9)).astype(np.float32)).contiguous(memory_format=cl)
    with pytest.raises(RuntimeError):
        ops.max_pool(x, (3, 3), out=torch.empty((2, 6, 7, 7), device="cuda").contiguous(memory_format=cl))
    with pytest.raises(RuntimeError):
        ops.max_pool(x, (3, 3), out=torch.empty((2, 6, 7, 7), device="cuda"))
    y = r.standard_normal((16, 512, 7, 7)).astype(np.float32)
    assert_close_f32(host(ops.global_avg_pool(dev(y).contiguous(memory_format=cl))), oracle.global_avgpool(y))
    yb = bf16_round(y)
    got = ops.global_avg_pool(dev(yb, torch.bfloat16).contiguous(memory_format=cl))
    assert_close_bf16(host(got), bf16_round(oracle.global_avgpool(yb)), "channels-last average pool bf16")
