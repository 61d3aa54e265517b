"""GPU tests of the fused rotary embedding (fhip_rope, fhip_kv_cache_rope_append) through the C ABI.

Bit-exact against the CPU restatement of fusor's rope (rope.rs:46-137) for f32, and for 16-bit tensors
against cast -> rope in f32 -> cast, which is what kalosm-llama does (raw/rope.rs:103-111).
"""
import numpy as np
import pytest

import floneum_amd as fa
import oracle
from test_attention_gpu import rounded

pytestmark = pytest.mark.gpu


def _cast_out(y, dtype):
    """y rounded to the element type, in the form Tensor.to_numpy() returns it (bf16 comes back as f32)."""
    if dtype == fa.F32:
        return y.astype(np.float32)
    if dtype == fa.F16:
        return y.astype(np.float16)
    return fa.bf16_bits_to_f32(fa.f32_to_bf16_bits(y)).reshape(y.shape)


def _x(seed, shape):
    return np.random.default_rng(seed).normal(0, 1, shape).astype(np.float32)


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16, fa.BF16])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("D,start", [(64, 0), (128, 37), (96, 5), (2, 1)])
def test_rope_bit_exact(device, dtype, interleaved, D, start):
    rc = fa.RopeCache(D, 64, 10000.0, device)
    x = _x(D + start, (2, 3, 11, D))
    t = fa.Tensor.from_numpy(device, x, dtype)
    out = rc.apply(t, start, interleaved).to_numpy()
    fn = oracle.rope_interleaved if interleaved else oracle.rope
    ref = _cast_out(fn(rounded(x, dtype), rc.cos_host, rc.sin_host, start), dtype)
    assert np.array_equal(out.view(np.uint8), ref.view(np.uint8))


def test_rope_reference_test_inputs(device):
    # the inputs of fusor's rope tests (rope.rs:272-330)
    i = np.arange(11, dtype=np.float32)[:, None]
    j = np.arange(32, dtype=np.float32)[None, :]
    ang = (i / np.power(np.float32(10000.0), (2 * j) / np.float32(64), dtype=np.float32)).astype(np.float32)
    rc = fa.RopeCache.from_parts(np.cos(ang), np.sin(ang), device)
    x = np.sin((np.arange(3 * 11 * 64) % 64).astype(np.float32)).astype(np.float32).reshape(1, 3, 11, 64)
    t = fa.Tensor.from_numpy(device, x, fa.F32)
    q, k = rc.forward(t, t, 0)
    qi, ki = rc.forward_interleaved(t, t, 0)
    assert q.shape == (1, 3, 11, 64) and np.isfinite(q.to_numpy()).all() and np.isfinite(qi.to_numpy()).all()
    assert np.array_equal(q.to_numpy(), oracle.rope(x, rc.cos_host, rc.sin_host))
    assert np.array_equal(ki.to_numpy(), oracle.rope_interleaved(x, rc.cos_host, rc.sin_host))


def test_rope_on_the_transposed_projection_view_and_type_change(device):
    """kalosm-llama's projections are [b, seq, heads, hd] transposed to [b, heads, seq, hd]
    (attention_layer.rs:226-229): the op takes that view as it is, and can hand f16 to the attention call."""
    B, S, H, D = 2, 9, 4, 64
    rc = fa.RopeCache(D, 32, 500000.0, device)
    proj = _x(7, (B, S, H, D))
    t = fa.Tensor.from_numpy(device, proj, fa.F32).transpose(1, 2)
    out = rc.apply(t, 3, False, out_dtype=fa.F16).to_numpy()
    ref = oracle.rope(proj.transpose(0, 2, 1, 3), rc.cos_host, rc.sin_host, 3).astype(np.float16)
    assert out.dtype == np.float16 and np.array_equal(out, ref)


def test_rope_rejects_bad_arguments(device):
    rc = fa.RopeCache(64, 8, 10000.0, device)
    t = fa.Tensor.from_numpy(device, _x(1, (1, 1, 4, 64)), fa.F32)
    with pytest.raises(AssertionError, match="exceed"):
        rc.apply(t, 5)            # positions 5..9 of 8
    odd = fa.Tensor.from_numpy(device, _x(1, (1, 1, 4, 63)), fa.F32)
    with pytest.raises(AssertionError, match="even"):
        rc.apply(odd, 0)


@pytest.mark.parametrize("cache_dtype,in_dtype", [(fa.F32, fa.F32), (fa.F16, fa.F32), (fa.F16, fa.F16)])
@pytest.mark.parametrize("interleaved", [False, True])
def test_kv_cache_rope_append_equals_rope_then_append(device, cache_dtype, in_dtype, interleaved):
    """Growth, in-place appends and truncation to max_sequence_len, with the rotation fused into the write."""
    B, Hkv, D, max_len = 2, 2, 64, 40
    rc = fa.RopeCache(D, 128, 10000.0, device)
    fused = fa.KvCache(2, max_len, cache_dtype, device)
    ref_cache = oracle.KvCache(2, max_len)
    fn = oracle.rope_interleaved if interleaved else oracle.rope
    pos = 0
    for step, n in enumerate([5, 1, 1, 9, 1, 17, 1, 1, 12, 3]):
        k = _x(100 + step, (B, Hkv, n, D))
        v = _x(200 + step, (B, Hkv, n, D))
        tk, tv = fa.Tensor.from_numpy(device, k, in_dtype), fa.Tensor.from_numpy(device, v, in_dtype)
        ka, va = fused.append_rope(rc, tk, tv, pos, interleaved)
        k_rot = _cast_out(fn(rounded(k, in_dtype), rc.cos_host, rc.sin_host, pos), cache_dtype)
        v_cast = _cast_out(rounded(v, in_dtype), cache_dtype)
        rk, rv = ref_cache.append(k_rot, v_cast)
        assert ka.shape == rk.shape and va.shape == rv.shape
        assert np.array_equal(ka.to_numpy().view(np.uint8), np.ascontiguousarray(rk).view(np.uint8)), f"keys, step {step}"
        assert np.array_equal(va.to_numpy().view(np.uint8), np.ascontiguousarray(rv).view(np.uint8)), f"values, step {step}"
        pos += n
    assert fused.current_seq_len() == max_len


# ---- q / k RMS-norm fused into the rotation (attention_q_norm / attention_k_norm) ---------------------

def _norm_then_rope(x, dtype, w, b, eps, rc, start, interleaved, out_dtype):
    """What the reference computes (attention_layer.rs:229-235,272-278): the norm in f32 rounded to the
    tensor's type, then cast -> rope -> cast."""
    n = rounded(oracle.rms_norm(rounded(x, dtype), rounded(w, dtype), None if b is None else rounded(b, dtype), eps), dtype)
    fn = oracle.rope_interleaved if interleaved else oracle.rope
    return _cast_out(fn(n, rc.cos_host, rc.sin_host, start), out_dtype)


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16, fa.BF16])
@pytest.mark.parametrize("interleaved,bias", [(False, False), (True, True)])
@pytest.mark.parametrize("D,start", [(64, 0), (128, 37), (96, 5), (256, 2), (2, 1)])
def test_norm_rope_bit_exact(device, dtype, interleaved, bias, D, start):
    rc = fa.RopeCache(D, 64, 1000000.0, device)
    rng = np.random.default_rng(D)
    x = _x(D + start, (2, 5, 11, D)) * 3
    w = rng.normal(1, 0.3, D).astype(np.float32)
    b = rng.normal(0, 0.1, D).astype(np.float32) if bias else None
    norm = fa.RmsNorm(w, b, 1e-6, dtype, device)
    t = fa.Tensor.from_numpy(device, x, dtype)
    out = rc.apply(t, start, interleaved, norm=norm).to_numpy()
    ref = _norm_then_rope(x, dtype, w, b, 1e-6, rc, start, interleaved, dtype)
    assert np.array_equal(out.view(np.uint8), ref.view(np.uint8))
    # the norm alone (RmsNorm::forward_generic_4d)
    alone = norm.forward_generic_4d(t).to_numpy()
    ref_n = _cast_out(oracle.rms_norm(rounded(x, dtype), rounded(w, dtype), None if b is None else rounded(b, dtype), 1e-6), dtype)
    assert np.array_equal(alone.view(np.uint8), ref_n.view(np.uint8))


@pytest.mark.parametrize("in_dtype,out_dtype", [(fa.F32, fa.F32), (fa.F32, fa.F16), (fa.F16, fa.F16), (fa.BF16, fa.F32)])
@pytest.mark.parametrize("D,interleaved", [(128, False), (256, False), (64, True), (128, True)])
def test_prompt_sized_rope_and_norm_rope_bit_exact(device, in_dtype, out_dtype, D, interleaved):
    """The rows of a prompt (thousands, in row blocks of the wide forms, the last block partial; the sum of squares of
    head_dim 128 and 256 rows whose order matters) with the conversion to the cache's type on the way out."""
    B, H, S, start = 1, 6, 333, 19
    rc = fa.RopeCache(D, 512, 500000.0, device)
    rng = np.random.default_rng(D + S)
    x = (_x(5, (B, H, S, D)) * rng.choice([1.0, 30.0, 1e-3], (B, H, S, 1))).astype(np.float32)
    w = rng.normal(1, 0.3, D).astype(np.float32)
    t = fa.Tensor.from_numpy(device, x, in_dtype)
    out = rc.apply(t, start, interleaved, out_dtype=out_dtype).to_numpy()
    fn = oracle.rope_interleaved if interleaved else oracle.rope
    ref = _cast_out(fn(rounded(x, in_dtype), rc.cos_host, rc.sin_host, start), out_dtype)
    assert np.array_equal(out.view(np.uint8), ref.view(np.uint8)), "rope"
    norm = fa.RmsNorm(w, None, 1e-6, in_dtype, device)
    out = rc.apply(t, start, interleaved, out_dtype=out_dtype, norm=norm).to_numpy()
    ref = _norm_then_rope(x, in_dtype, w, None, 1e-6, rc, start, interleaved, out_dtype)
    assert np.array_equal(out.view(np.uint8), ref.view(np.uint8)), "norm + rope"


def test_norm_sum_order_and_reference_test_rows(device):
    """The device sum is the reference's left-to-right fold (a row where any other order differs), and the
    rows of the reference's own tests (rms_norm.rs:163-186) come out as expected."""
    x = np.ones((1, 1, 2, 42), np.float32)
    x[0, 0, 0, 0] = 4096.0
    x[0, 0, 1, 40] = 4096.0
    norm = fa.RmsNorm(np.ones(42, np.float32), None, 0.0, fa.F32, device)
    out = norm.forward_generic_4d(fa.Tensor.from_numpy(device, x, fa.F32)).to_numpy()
    assert np.array_equal(out, oracle.rms_norm(x, np.ones(42, np.float32), None, 0.0))
    x2 = np.array([3, 4, 6, 8], np.float32).reshape(1, 1, 2, 2)
    out2 = fa.RmsNorm(np.array([2, 2], np.float32), None, 1e-5, fa.F32, device).forward_generic_4d(
        fa.Tensor.from_numpy(device, x2, fa.F32)).to_numpy()
    rms1 = np.sqrt(np.float32(12.5))
    assert abs(out2[0, 0, 0, 0] - 3.0 / rms1 * 2.0) < 1e-4 and abs(out2[0, 0, 0, 1] - 4.0 / rms1 * 2.0) < 1e-4


def test_norm_rope_in_place_on_a_strided_view(device):
    """out may be x itself, and x may be the transposed projection: rows are read whole before they are written."""
    B, S, H, D = 2, 33, 6, 128
    rc = fa.RopeCache(D, 64, 10000.0, device)
    proj = _x(9, (B, S, H, D))
    w = np.random.default_rng(4).normal(1, 0.2, D).astype(np.float32)
    norm = fa.RmsNorm(w, None, 1e-6, fa.F32, device)
    t = fa.Tensor.from_numpy(device, proj, fa.F32).transpose(1, 2)
    import ctypes
    cx, cn, tables = t._c4(), norm._c(), rc._tables(7, False)
    fa.check(fa.lib().fhip_norm_rope(device.stream, ctypes.byref(cn), ctypes.byref(tables), ctypes.byref(cx), fa.F32,
                                     ctypes.byref(cx), fa.F32))
    ref = oracle.rope(oracle.rms_norm(proj.transpose(0, 2, 1, 3), w, None, 1e-6), rc.cos_host, rc.sin_host, 7)
    assert np.array_equal(t.to_numpy(), ref)


@pytest.mark.parametrize("cache_dtype,in_dtype", [(fa.F32, fa.F32), (fa.F16, fa.F32), (fa.F16, fa.F16)])
def test_kv_cache_norm_rope_append(device, cache_dtype, in_dtype):
    B, Hkv, D, max_len = 2, 2, 128, 24
    rc = fa.RopeCache(D, 64, 10000.0, device)
    w = np.random.default_rng(6).normal(1, 0.2, D).astype(np.float32)
    norm = fa.RmsNorm(w, None, 1e-6, in_dtype, device)
    fused = fa.KvCache(2, max_len, cache_dtype, device)
    ref_cache = oracle.KvCache(2, max_len)
    pos = 0
    for step, n in enumerate([5, 1, 9, 1, 17, 2]):
        k = _x(300 + step, (B, Hkv, n, D))
        v = _x(400 + step, (B, Hkv, n, D))
        tk, tv = fa.Tensor.from_numpy(device, k, in_dtype), fa.Tensor.from_numpy(device, v, in_dtype)
        ka, va = fused.append_rope(rc, tk, tv, pos, False, k_norm=norm)
        k_rot = _norm_then_rope(k, in_dtype, w, None, 1e-6, rc, pos, False, cache_dtype)
        rk, rv = ref_cache.append(k_rot, _cast_out(rounded(v, in_dtype), cache_dtype))
        assert np.array_equal(ka.to_numpy().view(np.uint8), np.ascontiguousarray(rk).view(np.uint8)), f"keys, step {step}"
        assert np.array_equal(va.to_numpy().view(np.uint8), np.ascontiguousarray(rv).view(np.uint8)), f"values, step {step}"
        pos += n


@pytest.mark.parametrize("cache_dtype,in_dtype,norms", [(fa.F32, fa.F32, False), (fa.F16, fa.F32, True), (fa.F16, fa.F16, True),
                                                        (fa.F32, fa.F32, True)])
def test_q_k_v_prepared_in_one_launch_equals_the_separate_calls(device, cache_dtype, in_dtype, norms):
    """fhip_kv_cache_qkv_rope_append (q rotated, new keys rotated and appended, new values appended, all in one launch)
    against fhip_rope / fhip_norm_rope + fhip_kv_cache_(norm_)rope_append, through first append, growth, in-place appends
    and truncation."""
    B, H, Hkv, D, max_len = 2, 4, 2, 64, 40
    rc = fa.RopeCache(D, 128, 10000.0, device)
    rng = np.random.default_rng(7)
    qn = fa.RmsNorm(rng.normal(1, 0.2, D).astype(np.float32), None, 1e-6, in_dtype, device) if norms else None
    kn = fa.RmsNorm(rng.normal(1, 0.2, D).astype(np.float32), None, 1e-6, in_dtype, device) if norms else None
    fused, separate = fa.KvCache(2, max_len, cache_dtype, device), fa.KvCache(2, max_len, cache_dtype, device)
    pos = 0
    for step, n in enumerate([5, 1, 1, 9, 1, 17, 1, 1, 12, 3]):
        q, k, v = _x(500 + step, (B, H, n, D)), _x(600 + step, (B, Hkv, n, D)), _x(700 + step, (B, Hkv, n, D))
        tq, tk, tv = (fa.Tensor.from_numpy(device, a, in_dtype) for a in (q, k, v))
        q1, k1, v1 = fused.qkv_rope_append(rc, tq, tk, tv, pos, False, qn, kn, q_out_dtype=cache_dtype)
        q2 = rc.apply(tq, pos, False, out_dtype=cache_dtype, norm=qn)
        k2, v2 = separate.append_rope(rc, tk, tv, pos, False, k_norm=kn)
        assert k1.shape == k2.shape and v1.shape == v2.shape
        for a, b_, what in ((q1, q2, "q"), (k1, k2, "keys"), (v1, v2, "values")):
            assert np.array_equal(a.to_numpy().view(np.uint8), b_.to_numpy().view(np.uint8)), f"{what}, step {step}"
        pos += n
    assert fused.current_seq_len() == max_len
