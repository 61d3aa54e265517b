"""CPU checks that pin the RMS-norm restatement in oracle/ (fusor rms_norm.rs:122-133,
normalization.rs:351-407), the q / k norm that precedes the rotary embedding.

The reference's tests give expected values to 1e-4 / 1e-2 (rms_norm.rs:140-186, normalization.rs:487-533,
core rms_norm_fused.rs:549-582); those are reproduced.  What they leave open (operation order, the
left-to-right sum) is pinned by cases the arithmetic fixes exactly: rows whose every step is exact,
scaling by powers of two, and a row where any other summation order gives a different f32 sum.
"""
import numpy as np

import oracle


def test_reference_expected_values():
    # rms_norm.rs:140-161 and normalization.rs:513-533
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    y = oracle.rms_norm(x, np.ones(3, np.float32), None, 1e-5)
    for row, tot in ((0, 14.0), (1, 77.0)):
        rms = np.sqrt(np.float32(tot) / np.float32(3) + np.float32(1e-5))
        assert np.abs(y[row] - x[row] / rms).max() < 1e-4
    # rms_norm.rs:163-186: weight 2, rows [3, 4] and [6, 8]
    x3 = np.array([[[3, 4], [6, 8]]], np.float32)
    y3 = oracle.rms_norm(x3, np.array([2, 2], np.float32), None, 1e-5)
    rms1 = np.sqrt(np.float32(12.5))
    assert abs(y3[0, 0, 0] - 3.0 / rms1 * 2.0) < 1e-4 and abs(y3[0, 0, 1] - 4.0 / rms1 * 2.0) < 1e-4
    # core rms_norm_fused.rs:549-582: weight [2, 3], expected 1.2649, 3.7947
    y2 = oracle.rms_norm(np.array([[1, 2], [3, 4], [5, 6]], np.float32), np.array([2, 3], np.float32), None, 1e-5)
    assert abs(y2[0, 0] - 1.2649) < 1e-3 and abs(y2[0, 1] - 3.7947) < 1e-3


def test_against_float64_definition():
    rng = np.random.default_rng(1)
    x = rng.normal(0, 3, (2, 3, 5, 128)).astype(np.float32)
    w = rng.normal(1, 0.2, 128).astype(np.float32)
    b = rng.normal(0, 0.1, 128).astype(np.float32)
    for bias in (None, b):
        y = oracle.rms_norm(x, w, bias, 1e-6)
        ref = oracle.rms_norm_f64(x, w, bias, 1e-6)
        assert np.abs(y - ref).max() <= 2e-6 * np.abs(ref).max()


def test_exact_rows_and_power_of_two_scaling():
    # every step exact: squares sum to 16, mean 4, rms 2
    x = np.array([[2, -2, 2, -2]], np.float32)
    w = np.array([1, 3, 0.5, -7], np.float32)
    assert np.array_equal(oracle.rms_norm(x, w, None, 0.0), np.array([[1, -3, 0.5, 7]], np.float32))
    assert np.array_equal(oracle.rms_norm(x, w, np.array([1, 1, 1, 1], np.float32), 0.0),
                          np.array([[2, -2, 1.5, 8]], np.float32))
    # without eps the norm does not see a power-of-two scale (all roundings scale with it)
    rng = np.random.default_rng(2)
    r = rng.normal(0, 1, (7, 64)).astype(np.float32)
    w = rng.normal(1, 0.1, 64).astype(np.float32)
    assert np.array_equal(oracle.rms_norm(r, w, None, 0.0), oracle.rms_norm(r * np.float32(8), w, None, 0.0))
    # eps is added to the MEAN of the squares, inside the root: a row of zeros gives 0 / sqrt(eps) = 0, not NaN
    assert np.array_equal(oracle.rms_norm(np.zeros((1, 8), np.float32), np.ones(8, np.float32), None, 1e-5),
                          np.zeros((1, 8), np.float32))


def test_sum_is_a_left_to_right_fold():
    # squares: 2^24, then 1 forty times.  Left to right every "+ 1" is lost to rounding (2^24 + 1 ties to even):
    # sum = 2^24.  Pairwise or lane-split sums keep them (2^24 + 40).  cpu/src/reduce.rs:752-757 is the fold.
    x = np.ones((1, 41), np.float32)
    x[0, 0] = 4096.0
    w = np.ones(41, np.float32)
    y = oracle.rms_norm(x, w, None, 0.0)
    rms_fold = np.sqrt(np.float32(2.0 ** 24) / np.float32(41))
    rms_other = np.sqrt(np.float32(2.0 ** 24 + 40) / np.float32(41))
    assert rms_fold != rms_other
    assert np.array_equal(y, (x / rms_fold).astype(np.float32))
    # and the fold starts at the FIRST element: with the large square last, the ones are all kept
    xr = x[:, ::-1].copy()
    rms_rev = np.sqrt(np.float32(40.0 + 2.0 ** 24) / np.float32(41))
    assert np.array_equal(oracle.rms_norm(xr, w, None, 0.0), (xr / rms_rev).astype(np.float32))
