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


def assert_as_close_as_eager(got, eager, want64, rtol, atol, what, rms_factor=1.5):
    """`got` against the float64 evaluation `want64`, measured by what a reference evaluation in the same storage
    type (`eager`: torch's own kernels, or the oracle rounded to the storage type) achieves on the same graph.  A fixed
    absolute floor is either too loose for well-conditioned outputs or too tight where the graph amplifies rounding
    (a layer norm over nearly constant rows, outputs that cancel to ~0), so three things are asked instead:
      * every element within the stated tolerance plus four times the reference's own WORST error (a bound on outliers),
      * no more elements outside the plain stated tolerance than twice the reference's own count (+ 1e-4 of all, at
        least 3): an error on more than a few small outputs cannot hide inside the first bar's global slack,
      * an rms error of at most `rms_factor` (1.5) times the reference's, unless it is under a quarter of the rms of
        the plain tolerance itself (the bulk of the elements is as accurate as the reference's, or far inside the
        stated tolerance: fp32 sums in another order than torch's pairwise ones are legitimately a few times noisier
        at the 1e-9 level).  Networks in 16-bit storage whose batch norms are folded into their filters pass 3: the folded
        filters are rounded to the storage type once more (every filter carries a relative error of 2^-9, which the
        unfolded evaluation does not have), the price of one kernel per convolution unit.  Both rms values are
        estimates from n elements, uncertain by a fraction of about 1 / sqrt(2 n) each: the factor is widened by
        1 + 2 / sqrt(n) (1.45 for a network's 20 logits, 1.002 for a million activations).
    Returns the measured margins: the fractions of elements outside the plain bar (with atol, and with rtol alone)
    for `got` and for the reference, so that a test can print them."""
    got, eager, want64 = (np.asarray(t, dtype=np.float64) for t in (got, eager, want64))
    assert got.shape == want64.shape, "%s: shape %s vs %s" % (what, got.shape, want64.shape)
    noise = float(np.abs(eager - want64).max())
    err, ref_err = np.abs(got - want64), np.abs(eager - want64)
    plain = atol + rtol * np.abs(want64)
    bad = ~(err <= plain + 4.0 * noise)
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err, 0)), err.shape)
        raise AssertionError("%s: %d of %d elements outside rtol=%g atol=%g + 4 x the reference's own error %.3g; worst at %s: "
                             "got %r want %r" % (what, int(bad.sum()), bad.size, rtol, atol, noise, i, got[i], want64[i]))
    n_out, n_ref = int((err > plain).sum()), int((ref_err > plain).sum())
    assert n_out <= 2 * n_ref + max(3, int(1e-4 * err.size)), \
        "%s: %d elements outside rtol=%g atol=%g, the reference evaluation has %d" % (what, n_out, rtol, atol, n_ref)
    rms, ref_rms = float(np.sqrt((err ** 2).mean())), float(np.sqrt((ref_err ** 2).mean()))
    plain_rms = float(np.sqrt((plain ** 2).mean()))
    small_sample = 1.0 + 2.0 / np.sqrt(err.size)
    assert rms <= max(rms_factor * small_sample * ref_rms, 0.25 * plain_rms) + 1e-12, \
        "%s: rms error %.3g, the reference evaluation's %.3g, the tolerance's rms %.3g" % (what, rms, ref_rms, plain_rms)
    rel_only = rtol * np.abs(want64)
    stats = {"n": int(err.size), "outside_plain": n_out / err.size, "outside_plain_reference": n_ref / err.size,
             "outside_rtol_only": float((err > rel_only).mean()), "outside_rtol_only_reference": float((ref_err > rel_only).mean()),
             "rms": rms, "rms_reference": ref_rms}
    print("%s: outside rtol=%g/atol=%g: %.2e of %d elements (reference evaluation %.2e); outside rtol alone: %.2e (reference %.2e); "
          "rms error %.3g (reference %.3g)" % (what, rtol, atol, stats["outside_plain"], stats["n"], stats["outside_plain_reference"],
                                                stats["outside_rtol_only"], stats["outside_rtol_only_reference"], rms, ref_rms))
    return stats
