"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

# north-star tolerances
F32_RTOL, F32_ATOL = 1e-4, 1e-5
BF16_RTOL = 2e-2
# bf16 results that cancel to ~0 have no meaningful relative error; this absolute floor is small
# against every test's output scale (values are O(1) or larger)
BF16_ATOL = 2e-3


def rng(seed):
    return np.random.default_rng(seed)


def dev(a, dtype=None):
    """numpy -> cuda tensor (bf16 via torch's round-to-nearest-even)."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def host(t):
    return t.detach().float().cpu().numpy() if t.dtype in (torch.bfloat16, torch.float16) else t.detach().cpu().numpy()


def bf16_round(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy()


def assert_close(got, want, rtol, atol, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, "%s: shape %s vs %s" % (what, got.shape, want.shape)
    both_nan = np.isnan(got) & np.isnan(want)
    err = np.abs(got - want)
    bad = ~(err <= atol + rtol * np.abs(want)) & ~both_nan
    same_inf = np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want))
    bad &= ~same_inf
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err, 0)), err.shape)
        raise AssertionError("%s: %d of %d elements outside rtol=%g atol=%g; worst at %s: got %r want %r (max abs err %g)"
                             % (what, int(bad.sum()), bad.size, rtol, atol, i, got[i], want[i], float(err[bad].max())))


def assert_close_f32(got, want, what=""):
    assert_close(got, want, F32_RTOL, F32_ATOL, what)


def assert_close_bf16(got, want, what=""):
    assert_close(got, want, BF16_RTOL, BF16_ATOL, what)


def assert_as_close_as_eager(got, eager, want64, rtol, atol, what):
    """`got` against the float64 evaluation `want64`, at the stated tolerance plus four times what a reference
    evaluation in the same storage type (`eager`: torch's own kernels, or the oracle rounded to the storage type)
    misses it by.  A fixed absolute floor is either too loose for well-conditioned outputs or too tight where the
    graph amplifies rounding (a layer norm over nearly constant rows, outputs that cancel to ~0): this bar follows
    what the storage type can deliver on that graph, and ours must be as good as the reference's, up to a factor."""
    got, eager, want64 = (np.asarray(t, dtype=np.float64) for t in (got, eager, want64))
    assert got.shape == want64.shape, "%s: shape %s vs %s" % (what, got.shape, want64.shape)
    noise = float(np.abs(eager - want64).max())
    err = np.abs(got - want64)
    bar = atol + rtol * np.abs(want64) + 4.0 * noise
    bad = ~(err <= bar)
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err, 0)), err.shape)
        raise AssertionError("%s: %d of %d elements outside rtol=%g atol=%g + 4 x the reference's own error %.3g; worst at %s: "
                             "got %r want %r" % (what, int(bad.sum()), bad.size, rtol, atol, noise, i, got[i], want64[i]))
