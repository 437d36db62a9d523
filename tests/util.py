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
    """|actual - expected| <= rel * (|expected| + rms(expected)) elementwise.
    The max-abs error is part of the failure message and is printed on success."""
    actual = np.asarray(actual, np.float64)
    expected = np.asarray(expected, np.float64)
    assert actual.shape == expected.shape, (what, actual.shape, expected.shape)
    assert np.all(np.isfinite(actual)), what + ": non-finite values"
    rms = float(np.sqrt(np.mean(expected ** 2)))
    diff = np.abs(actual - expected)
    bound = rel * (np.abs(expected) + rms)
    worst = float(diff.max())
    print("%s: max-abs error %.3e, rms(expected) %.3e" % (what, worst, rms))
    bad = diff > bound
    assert not bad.any(), "%s: %d of %d beyond %.1e relative; max-abs %.3e (rms %.3e)" % (
        what, int(bad.sum()), bad.size, rel, worst, rms)
