"""CPU checks that pin the rotary-embedding restatement in oracle/ (fusor rope.rs:46-137).

The reference's own rope tests (rope.rs:270-400) only assert shape and finiteness on the inputs
reproduced here, so the arithmetic is pinned by what the mathematics fixes: the rotation is a complex
multiplication (float64 twin), position 0 is the identity, pairs keep their norm, rotating by the
tables of angle a and then b equals rotating by a + b, and the two pairings differ by a fixed
permutation of the head dimension.
"""
import numpy as np

import oracle


def _reference_inputs():
    # rope.rs:272-300: tables [11, 32] from i / 10000^(2j/64), x[k] = sin(k % 64), shape [1, 3, 11, 64]
    i = np.arange(11, dtype=np.float32)[:, None]
    j = np.arange(32, dtype=np.float32)[None, :]
    ang = (i / np.power(np.float32(10000.0), (2 * j) / np.float32(64), dtype=np.float32)).astype(np.float32)
    x = np.sin((np.arange(3 * 11 * 64) % 64).astype(np.float32)).astype(np.float32).reshape(1, 3, 11, 64)
    return x, np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def test_reference_test_inputs_shape_and_finiteness():
    x, cos, sin = _reference_inputs()
    for fn in (oracle.rope, oracle.rope_interleaved):
        y = fn(x, cos, sin)
        assert y.shape == (1, 3, 11, 64) and y.dtype == np.float32 and np.isfinite(y).all()


def test_against_float64_complex_rotation():
    x, cos, sin = _reference_inputs()
    rng = np.random.default_rng(3)
    x = (x + rng.normal(0, 1, x.shape)).astype(np.float32)
    for inter, fn in ((False, oracle.rope), (True, oracle.rope_interleaved)):
        for start in (0, 4):
            xs = x[:, :, :7]
            y = fn(xs, cos, sin, start)
            ref = oracle.rope_f64(xs, cos, sin, start, inter)
            assert np.abs(y - ref).max() <= 4e-7 * max(1.0, np.abs(ref).max())


def test_position_zero_is_identity_and_norms_are_kept():
    x, cos, sin = _reference_inputs()
    y = oracle.rope(x, cos, sin)
    yi = oracle.rope_interleaved(x, cos, sin)
    assert np.array_equal(y[:, :, 0], x[:, :, 0]) and np.array_equal(yi[:, :, 0], x[:, :, 0])  # cos 1, sin 0
    h = x.shape[3] // 2
    n_in = x[..., :h].astype(np.float64) ** 2 + x[..., h:].astype(np.float64) ** 2
    n_out = y[..., :h].astype(np.float64) ** 2 + y[..., h:].astype(np.float64) ** 2
    assert np.abs(n_in - n_out).max() < 1e-6
    ni_in = x[..., 0::2].astype(np.float64) ** 2 + x[..., 1::2].astype(np.float64) ** 2
    ni_out = yi[..., 0::2].astype(np.float64) ** 2 + yi[..., 1::2].astype(np.float64) ** 2
    assert np.abs(ni_in - ni_out).max() < 1e-6


def test_sign_and_pairing_conventions():
    # one pair, angle +90 degrees: (1, 0) -> (0, 1) in both pairings; a sign or pairing slip fails this
    cos = np.zeros((1, 2), np.float32)
    sin = np.ones((1, 2), np.float32)
    x = np.array([1, 2, 0, 0], np.float32).reshape(1, 1, 1, 4)       # normal: pairs (0,2), (1,3)
    assert np.array_equal(oracle.rope(x, cos, sin), np.array([0, 0, 1, 2], np.float32).reshape(1, 1, 1, 4))
    xi = np.array([1, 0, 2, 0], np.float32).reshape(1, 1, 1, 4)      # interleaved: pairs (0,1), (2,3)
    assert np.array_equal(oracle.rope_interleaved(xi, cos, sin), np.array([0, 1, 0, 2], np.float32).reshape(1, 1, 1, 4))
    x2 = np.array([0, 0, 1, 2], np.float32).reshape(1, 1, 1, 4)      # (0, 1) -> (-1, 0)
    assert np.array_equal(oracle.rope(x2, cos, sin), np.array([-1, -2, 0, 0], np.float32).reshape(1, 1, 1, 4))


def test_pairings_differ_by_a_permutation():
    x, cos, sin = _reference_inputs()
    d = x.shape[3]
    perm = np.concatenate([np.arange(0, d, 2), np.arange(1, d, 2)])  # interleaved index of normal slot
    y_from_inter = oracle.rope_interleaved(x, cos, sin)[..., perm]
    y_normal = oracle.rope(x[..., perm], cos, sin)
    assert np.array_equal(y_from_inter, y_normal)


def test_rotations_compose():
    cos_a, sin_a = oracle.rope_tables(64, 6, 10000.0)
    x = np.random.default_rng(1).normal(0, 1, (1, 2, 1, 64)).astype(np.float32)
    # rotate by position 2, then by position 3 (tables narrowed to one row each) == rotate by position 5
    y = oracle.rope(oracle.rope(x, cos_a, sin_a, 2), cos_a, sin_a, 3)
    z = oracle.rope(x, cos_a, sin_a, 5)
    assert np.abs(y - z).max() < 2e-6


def test_tables_follow_the_closed_form():
    cos, sin = oracle.rope_tables(8, 5, 10000.0)
    assert cos.shape == (5, 4) and sin.shape == (5, 4)
    ref = np.arange(5)[:, None] / (10000.0 ** (np.arange(0, 8, 2)[None, :] / 8.0))
    assert np.abs(cos - np.cos(ref)).max() < 1e-6 and np.abs(sin - np.sin(ref)).max() < 1e-6
    assert np.array_equal(cos[0], np.ones(4, np.float32)) and np.array_equal(sin[0], np.zeros(4, np.float32))
