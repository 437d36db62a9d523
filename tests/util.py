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


def assert_close_bf16(actual, expected, what, rel=2e-2):
    """Tolerance for kernels whose matrix-core operands are bf16.

    Every operand of a product is rounded to 8 mantissa bits, so the error of
    an element is set by the size of the terms summed into it, not by the
    element itself (sums that nearly cancel keep the error of their terms).
    Two conditions, both with the stated 2e-2:
      max-norm:  max|actual - expected| <= rel * max|expected|
      L2-norm:   ||actual - expected||_2 <= rel * ||expected||_2
    The first is the stated relative tolerance; the second rejects structured
    errors (a dropped tile, a wrong mask or index) that a max-norm over a
    tensor with a few large elements could hide.  The max-abs error is printed."""
    actual = np.asarray(actual, np.float64)
    expected = np.asarray(expected, np.float64)
    assert actual.shape == expected.shape, (what, actual.shape, expected.shape)
    assert np.all(np.isfinite(actual)), what + ": non-finite values"
    diff = np.abs(actual - expected)
    worst = float(diff.max())
    peak = float(np.abs(expected).max())
    l2 = float(np.sqrt((diff ** 2).sum()) / (np.sqrt((expected ** 2).sum()) or 1.0))
    print("%s: max-abs error %.3e (%.2e of max|expected| %.3e), relative L2 error %.2e" % (
        what, worst, worst / (peak or 1.0), peak, l2))
    assert worst <= rel * peak, "%s: max-abs %.3e > %.1e * max|expected| %.3e" % (
        what, worst, rel, peak)
    assert l2 <= rel, "%s: relative L2 error %.3e > %.1e" % (what, l2, rel)
