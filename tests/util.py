"""Helpers shared by the GPU parity tests."""
import numpy as np


def to_bf16_bits(oracle, x):
    return oracle.f32_to_bf16_bits(x).reshape(np.shape(x))


def from_bf16_bits(oracle, bits):
    return oracle.bf16_bits_to_f32(bits).reshape(np.shape(bits))


def rel_error(actual, expected):
    """(max abs error, error relative to the RMS of the expected tensor)."""
    actual = np.asarray(actual, np.float64)
    expected = np.asarray(expected, np.float64)
    diff = np.abs(actual - expected)
    rms = float(np.sqrt(np.mean(expected ** 2))) or 1.0
    return float(diff.max()), float(diff.max() / rms)


def assert_close(actual, expected, rel, what):
    """Elementwise |actual - expected| <= rel * (|expected| + rms(expected)).
    Used for FP32 arithmetic.  The max-abs error is printed."""
    actual = np.asarray(actual, np.float64)
    expected = np.asarray(expected, np.float64)
    assert actual.shape == expected.shape, (what, actual.shape, expected.shape)
    assert np.all(np.isfinite(actual)), what + ": non-finite values"
    rms = float(np.sqrt(np.mean(expected ** 2)))
    diff = np.abs(actual - expected)
    bound = rel * (np.abs(expected) + rms)
    worst = float(diff.max())
    print("%s: max-abs error %.3e, rms(expected) %.3e, max|expected| %.3e" % (
        what, worst, rms, float(np.abs(expected).max())))
    bad = diff > bound
    assert not bad.any(), "%s: %d of %d beyond %.1e relative; max-abs %.3e (rms %.3e)" % (
        what, int(bad.sum()), bad.size, rel, worst, rms)


def assert_close_bf16(actual, expected, what, rel=2e-2, outliers=1e-4, far=2.0):
    """Tolerance for kernels whose matrix-core operands are bf16.

    Every operand of a product is rounded to 8 mantissa bits, so the error of
    an element is set by the size of the terms summed into it, not by the
    element itself (sums that nearly cancel keep the error of their terms).
    Three conditions, all with the stated 2e-2:
      per element: |actual - expected| <= rel * (|expected| + rms(expected))
      max-norm:    max|actual - expected| <= rel * max|expected|
      L2-norm:     ||actual - expected||_2 <= rel * ||expected||_2
    The first is the form the FP32 comparisons use: an element may not be off
    by more than 2 % of its own size plus 2 % of the tensor's typical size, so
    a region of small values cannot hide behind a few large ones.  Isolated
    elements whose bf16-rounded terms nearly cancel can exceed it: at most the
    fraction `outliers` may (one in ten thousand for forward outputs; callers
    that compare gradients, which are sums of products of two rounded factors
    with heavy-tailed sizes, pass their own), and none by more than `far`
    times the bound.  The last condition rejects structured errors (a dropped
    tile, a wrong mask or index).  The max-abs error and the number of
    elements beyond the first bound are printed."""
    actual = np.asarray(actual, np.float64)
    expected = np.asarray(expected, np.float64)
    assert actual.shape == expected.shape, (what, actual.shape, expected.shape)
    assert np.all(np.isfinite(actual)), what + ": non-finite values"
    diff = np.abs(actual - expected)
    worst = float(diff.max())
    peak = float(np.abs(expected).max())
    rms = float(np.sqrt(np.mean(expected ** 2)))
    l2 = float(np.sqrt((diff ** 2).sum()) / (np.sqrt((expected ** 2).sum()) or 1.0))
    scale = np.abs(expected) + rms
    beyond = int((diff > rel * scale).sum())
    far_beyond = int((diff > far * rel * scale).sum())
    ratio = float((diff / (rel * scale)).max()) if diff.size else 0.0
    print("%s: max-abs error %.3e (%.2e of max|expected| %.3e), relative L2 error %.2e, "
          "%d of %d elements beyond %.0e * (|expected| + rms %.3e), the farthest at %.2f times "
          "that bound" % (what, worst, worst / (peak or 1.0), peak, l2, beyond, diff.size, rel, rms,
                          ratio))
    assert beyond <= outliers * diff.size and far_beyond == 0, (
        "%s: %d of %d elements beyond %.1e * (|expected| + rms %.3e), %d beyond %g times that" % (
            what, beyond, diff.size, rel, rms, far_beyond, far))
    assert worst <= rel * peak, "%s: max-abs %.3e > %.1e * max|expected| %.3e" % (
        what, worst, rel, peak)
    assert l2 <= rel, "%s: relative L2 error %.3e > %.1e" % (what, l2, rel)


def beyond_reference_tolerance(actual, expected, absolute, relative):
    """Fraction of elements outside the reference's own device-vs-CPU bound
    |actual - expected| <= absolute + relative * |expected|
    (attention_reference_test.cc:56-73: 2e-3 + 2e-3 |x| forward, 3e-3 backward)."""
    actual = np.asarray(actual, np.float64)
    expected = np.asarray(expected, np.float64)
    return float(np.mean(np.abs(actual - expected) > absolute + relative * np.abs(expected)))


def assert_close_bf16_gradient(actual, expected, what, outliers=2e-3, far=10.0):
    """assert_close_bf16 for gradients of the bf16 attention kernels: dS and P
    are rounded to bf16 before the products that sum them over hundreds of
    rows, so a few elements per thousand miss the per-element bound (measured:
    up to 0.15 % on random inputs; more when the scores are peaked and most
    gradients are tiny).  `far` is the worst miss observed, rounded up: over
    all 192 units of the training configuration the farthest element of dQ sits
    at 9.03 times the per-element bound (dK 4.4, dV 4.4; every call prints its
    own figure).  Max-norm and L2 bounds are the same 2e-2."""
    assert_close_bf16(actual, expected, what, outliers=outliers, far=far)
