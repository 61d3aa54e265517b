"""Pins the CPU checker (oracle/) before anything is compared with it.

The C restatement is checked against: the float64 textbook twin, an independently written naive
restatement, hand-computed values of the reference's own test inputs, closed forms (causal row 0
equals V[0], equal scores give the mean of V, a single key returns its V row, a constant added to
a mask row changes nothing, -inf BatchKeyMask padding equals the un-padded call, GQA equals
expand-then-MHA), the committed golden fixtures, and the mask vectors the reference's tests hold.
"""
import json
import math
import os

import numpy as np
import pytest

import oracle
from floneum_amd import synth
from conftest import rel_l2

HERE = os.path.dirname(os.path.abspath(__file__))
NEG = float("-inf")


def rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def test_splitmix64_known_answer():
    # published SplitMix64 test vector (seed 1234567)
    got = [int(x) for x in synth.splitmix64(1234567, 0, 5)]
    assert got == [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431,
                   16408922859458223821]
    # counter-based: any window of the stream can be regenerated on its own
    assert [int(x) for x in synth.splitmix64(1234567, 3, 2)] == got[3:5]
    a = synth.normal(5, 1, (1000,))
    assert np.array_equal(a, synth.normal(5, 1, (1000,), chunk=64))
    x = synth.normal(9, 0, (200000,))
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01


def test_hand_computed_2x2():
    # reference inputs of fusor flash_attention.rs:207-239, worked by hand:
    # scores = I * scale; row 0 weights = softmax([s, 0]); out0 = w0*[1,2] + w1*[3,4]
    q = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    v = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 2, 2)
    s = 1 / math.sqrt(2)
    w = math.exp(s) / (math.exp(s) + 1.0)
    want = np.array([[w * 1 + (1 - w) * 3, w * 2 + (1 - w) * 4], [(1 - w) * 1 + w * 3, (1 - w) * 2 + w * 4]])
    out = oracle.flash_attention(q, q, v, s)
    assert np.allclose(out[0, 0], want, rtol=0, atol=1e-6)
    # causal mask: row 0 sees only key 0 -> exactly V[0] (fusor flash_attention.rs:241-276)
    out = oracle.flash_attention(q, q, v, s, np.array([[0, NEG], [0, 0]], np.float32), "qk")
    assert np.array_equal(out[0, 0, 0], v[0, 0, 0])
    assert np.allclose(out[0, 0, 1], want[1], atol=1e-6)


def test_golden_cases():
    cases = json.load(open(os.path.join(HERE, "golden", "attention_cases.json")))
    assert len(cases) >= 5
    dec = lambda xs, shape: np.array([NEG if x is None else x for x in xs], np.float32).reshape(shape)  # noqa: E731
    for c in cases:
        q, k, v = dec(c["q"], c["q_shape"]), dec(c["k"], c["k_shape"]), dec(c["v"], c["k_shape"])
        mask = None if c["mask"] is None else dec(c["mask"], c["mask_shape"])
        out = oracle.flash_attention(q, k, v, c["scale"], mask, c["mask_kind"])
        want = np.array(c["expected"]).reshape(c["q_shape"])
        assert np.isfinite(out).all(), c["name"]
        assert np.abs(out - want).max() < 2e-6, c["name"]


@pytest.mark.parametrize("B,H,Hkv,Sq,Skv,D", [(1, 4, 2, 33, 47, 16), (2, 6, 3, 5, 64, 7), (1, 1, 1, 128, 128, 64),
                                              (2, 8, 1, 17, 9, 32)])
def test_against_float64_twin_and_naive(B, H, Hkv, Sq, Skv, D):
    q, k, v = rand((B, H, Sq, D), 1), rand((B, Hkv, Skv, D), 2), rand((B, Hkv, Skv, D), 3)
    bias = (np.random.default_rng(4).random((Sq, Skv)) * 0.5 - 0.25).astype(np.float32)
    bias[np.arange(Skv)[None, :] > np.arange(Sq)[:, None] + (Skv - Sq if Skv >= Sq else 0)] = NEG
    bias[:, 0] = np.where(np.isneginf(bias[:, 0]), 0.0, bias[:, 0])  # every row keeps a visible key
    for mask, kind in [(None, None), (bias, "qk"), (np.where(np.arange(Skv) % 5 == 4, NEG, 0).astype(np.float32)[None].repeat(B, 0), "batch_key")]:
        out = oracle.flash_attention(q, k, v, D ** -0.5, mask, kind)
        twin = oracle.flash_attention_f64(q, k, v, D ** -0.5, mask, kind)
        naive = oracle.flash_attention(q, k, v, D ** -0.5, mask, kind, naive=True)
        assert rel_l2(out, twin) < 1e-6
        assert rel_l2(naive, twin) < 1e-6
        assert np.array_equal(out, naive), "the two C restatements follow the same operation order"


def test_row_subset_matches_full():
    q, k, v = rand((1, 4, 40, 16), 5), rand((1, 2, 40, 16), 6), rand((1, 2, 40, 16), 7)
    mask = oracle.get_mask(40, 0)
    full = oracle.flash_attention(q, k, v, 0.25, mask, "qk")
    rows = np.array([0, 7, 39], np.int32)
    sub = oracle.flash_attention(q[:, :, rows], k, v, 0.25, mask[rows], "qk")
    assert np.array_equal(sub, full[:, :, rows])


def test_closed_forms():
    B, H, S, D = 2, 3, 19, 8
    q, k, v = rand((B, H, S, D), 8), rand((B, H, S, D), 9), rand((B, H, S, D), 10)
    causal = oracle.get_mask(S, 0)
    out = oracle.flash_attention(q, k, v, 0.3, causal, "qk")
    assert np.array_equal(out[:, :, 0], v[:, :, 0]), "causal row 0 attends to key 0 only"
    # equal scores -> plain mean of V (q = 0)
    out = oracle.flash_attention(np.zeros_like(q), k, v, 0.3)
    assert np.allclose(out, v.mean(axis=2, keepdims=True).repeat(S, 2), atol=2e-6)
    # single key -> its V row, whatever the score
    out = oracle.flash_attention(q, k[:, :, :1], v[:, :, :1], 5.0)
    assert np.array_equal(out, v[:, :, :1].repeat(S, 2))
    # adding a constant to a mask row leaves the output unchanged (softmax shift invariance)
    shift = causal + np.linspace(-3, 3, S, dtype=np.float32)[:, None]
    a = oracle.flash_attention(q, k, v, 0.3, causal, "qk")
    b = oracle.flash_attention(q, k, v, 0.3, shift, "qk")
    assert rel_l2(b, a) < 1e-6
    # scaling: doubling q and halving scale is the same computation (exact in binary floating point)
    c = oracle.flash_attention(q * 2, k, v, 0.15, causal, "qk")
    assert np.array_equal(c, a)
    # -inf BatchKeyMask padding == un-padded call, exactly (exp(-inf) = 0 adds nothing)
    pad = 6
    kp = np.concatenate([k, rand((B, H, pad, D), 11)], axis=2)
    vp = np.concatenate([v, rand((B, H, pad, D), 12)], axis=2)
    bk = np.zeros((B, S + pad), np.float32)
    bk[:, S:] = NEG
    assert np.array_equal(oracle.flash_attention(q, kp, vp, 0.3, bk, "batch_key"), oracle.flash_attention(q, k, v, 0.3))
    # transposed-operand guard: swapping K and V changes the result
    assert rel_l2(oracle.flash_attention(q, v, k, 0.3), oracle.flash_attention(q, k, v, 0.3)) > 0.1


def test_gqa_head_mapping_is_h_div_g():
    # kv head of query head h is h // G (fusor flash_attention.rs:104-138; core :137,163-167): equal to
    # expanding K/V with repeat along heads (core test_flash_attention_gqa_fuzz :1001-1029), bit for bit
    B, Hkv, G, S, D = 2, 3, 4, 11, 8
    q, k, v = rand((B, Hkv * G, S, D), 13), rand((B, Hkv, S, D), 14), rand((B, Hkv, S, D), 15)
    a = oracle.flash_attention(q, k, v, 0.35)
    b = oracle.flash_attention(q, np.repeat(k, G, axis=1), np.repeat(v, G, axis=1), 0.35)
    assert np.array_equal(a, b)
    # and NOT the interleaved mapping h % Hkv
    c = oracle.flash_attention(q, np.tile(k, (1, G, 1, 1)), np.tile(v, (1, G, 1, 1)), 0.35)
    assert not np.array_equal(a, c)
    with pytest.raises(AssertionError, match="must be divisible"):
        oracle.flash_attention(q[:, :5], k, v, 1.0)


def test_fully_masked_row_is_nan():
    q, k, v = rand((1, 1, 3, 4), 16), rand((1, 1, 3, 4), 17), rand((1, 1, 3, 4), 18)
    mask = np.zeros((3, 3), np.float32)
    mask[1] = NEG
    out = oracle.flash_attention(q, k, v, 1.0, mask, "qk")
    assert np.isnan(out[0, 0, 1]).all() and np.isfinite(out[0, 0, [0, 2]]).all()


# ---- masks -----------------------------------------------------------------------------------------

def brute_get_mask(n, off, w):
    """MaskCache::get_mask by literal loops (mask_cache.rs:36-116, attention_mask.rs:26-34)."""
    if w is not None:
        off = min(off, max(w - n, 0))
    base = [[0.0] * n for _ in range(n)]
    for i in range(n):
        for j in range(n):
            if (w is None and j > i) or (w is not None and (i < j or j + w <= i)):
                base[i][j] = NEG
    if off == 0:
        return np.array(base, np.float32).reshape(n, n)
    return np.array([[0.0] * off + row for row in base], np.float32)


def test_masks_reference_vectors():
    g = json.load(open(os.path.join(HERE, "golden", "masks.json")))
    for name in ("causal_3", "causal_4", "sliding_4_w2"):
        c = g[name]
        want = np.where(np.array(c["masked"]) == 1, NEG, 0.0).astype(np.float32)
        for got in (oracle.get_mask(c["seq_len"], c["offset"], c["window"]), oracle.get_mask_c(c["seq_len"], c["offset"], c["window"])):
            assert got.shape == want.shape and np.array_equal(got, want), name
    c = g["offset_shape"]
    assert list(oracle.get_mask(c["seq_len"], c["offset"]).shape) == c["shape"]
    assert list(oracle.get_mask_c(c["seq_len"], c["offset"]).shape) == c["shape"]


def test_masks_brute_force():
    for n in range(1, 8):
        for off in (0, 1, 3, 10):
            for w in (None, 1, 2, 3, 5, 9, 20):
                want = brute_get_mask(n, off, w)
                a, b = oracle.get_mask(n, off, w), oracle.get_mask_c(n, off, w)
                assert a.shape == want.shape and np.array_equal(a, want), (n, off, w)
                assert b.shape == want.shape and np.array_equal(b, want), (n, off, w)
                assert a.dtype == np.float32 and set(np.unique(a.view(np.uint32))) <= {0, 0xFF800000}
    # the configuration of the sliding-window benchmark: 512 new tokens on a 16384-token cache, W = 4096
    m = oracle.get_mask(512, 16384, 4096)
    assert m.shape == (512, 4096) and not np.isneginf(m[:, :3584]).any()
    assert np.array_equal(m[:, 3584:], oracle.mask_causal(512))
    assert int((~np.isneginf(m)).sum()) == 1966336


# ---- KV cache ------------------------------------------------------------------------------------------

def test_tensor_cache_reference_cases():
    # tensor_cache.rs:130-186
    c = oracle.TensorCache(1, 2)
    t = np.array([1, 2, 3, 4], np.float32).reshape(2, 1, 2)
    r = c.append(t)
    assert r.shape == (2, 1, 2) and c.current_seq_len == 1 and np.array_equal(r, t)
    c = oracle.TensorCache(1, 3)
    c.append(np.array([1, 2], np.float32).reshape(1, 1, 2))
    r = c.append(np.array([3, 4], np.float32).reshape(1, 1, 2))
    assert r.shape == (1, 2, 2) and c.current_seq_len == 2 and r.ravel().tolist() == [1, 2, 3, 4]
    c.reset()
    assert c.current_seq_len == 0 and c.current_data() is None


def test_tensor_cache_growth_and_truncation():
    rng = np.random.default_rng(3)
    for max_len in (5, 8, 64):
        c = oracle.KvCache(2, max_len)
        hist_k = np.zeros((2, 3, 0, 4), np.float32)
        allocs = []
        for step in range(12):
            n = int(rng.integers(1, 4))
            k = rng.standard_normal((2, 3, n, 4)).astype(np.float32)
            ka, va = c.append(k, -k)
            hist_k = np.concatenate([hist_k, k], axis=2)[:, :, -max_len:]
            assert np.array_equal(ka, hist_k) and np.array_equal(va, -hist_k)
            assert c.current_seq_len() == hist_k.shape[2]
            allocs.append(c.key.allocated_seq_len)
        # growth is to the next power of two of the required length until the cap is hit (tensor_cache.rs:80-96)
        for a in allocs[1:]:
            assert a == max_len or (a & (a - 1)) == 0 or a == allocs[0]
