"""GPU parity tests: the HIP kernels, called through the C ABI, against the CPU checker.

Structure follows the reference's own tests: the unit cases of
fusor-ml/fusor/src/composite/flash_attention.rs:207-359 and the fuzz tests of
fusor-ml/core/src/composite/flash_attention.rs:559-1060 (same shape ranges, seeded here), then the
benchmark configurations at reduced and full size.
"""
import ctypes

import numpy as np
import pytest

import floneum_amd as fa
import oracle
from floneum_amd import synth
from conftest import TOL_16, TOL_F32, assert_parity, rel_l2

pytestmark = pytest.mark.gpu

NEG_INF = float("-inf")


def run(device, q, k, v, scale, mask=None, kind=None, dtype=fa.F32, **kw):
    tq = fa.Tensor.from_numpy(device, q, dtype)
    tk = fa.Tensor.from_numpy(device, k, dtype)
    tv = fa.Tensor.from_numpy(device, v, dtype)
    m = None
    if mask is not None:
        m = (fa.Tensor.from_numpy(device, mask, dtype), kind)
    return tq.flash_attention(tk, tv, scale, m, **kw).to_numpy()


def rounded(a, dtype):
    """The values the device sees after the host rounds to the element type, as float32."""
    if dtype == fa.F32:
        return np.asarray(a, np.float32)
    if dtype == fa.F16:
        return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)
    return fa.bf16_bits_to_f32(fa.f32_to_bf16_bits(a))


KIND = {fa.MaskKind.QKMask: "qk", fa.MaskKind.BatchKeyMask: "batch_key"}


def check(device, q, k, v, scale, mask=None, kind=None, dtype=fa.F32, what="", tol=None, **kw):
    out = run(device, q, k, v, scale, mask, kind, dtype, **kw)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale,
                                 None if mask is None else rounded(mask, dtype), KIND.get(kind))
    tol = tol or (TOL_F32 if dtype == fa.F32 else TOL_16)
    return assert_parity(out, ref, tol, what)


# ---- the reference's unit cases ---------------------------------------------------------------------

@pytest.mark.parametrize("kernel", [fa.KERNEL_AUTO, fa.KERNEL_GENERIC])
def test_flash_attention_2x2(device, kernel):
    # fusor flash_attention.rs:207-239
    q = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    k = q.copy()
    v = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 2, 2)
    out = run(device, q, k, v, 1 / np.sqrt(2), force_kernel=kernel)
    assert out.shape == (1, 1, 2, 2) and np.isfinite(out).all()
    check(device, q, k, v, 1 / np.sqrt(2), force_kernel=kernel)


def test_flash_attention_causal_row0_is_v0(device):
    # fusor flash_attention.rs:241-276, core flash_attention.rs:605-673
    q = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    v = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 2, 2)
    mask = np.array([[0, NEG_INF], [0, 0]], np.float32)
    out = run(device, q, q, v, 1 / np.sqrt(2), mask, fa.MaskKind.QKMask)
    assert abs(out[0, 0, 0, 0] - 1.0) < 0.01 and abs(out[0, 0, 0, 1] - 2.0) < 0.01
    check(device, q, q, v, 1 / np.sqrt(2), mask, fa.MaskKind.QKMask)


def test_flash_attention_gqa_ramp(device):
    # fusor flash_attention.rs:278-313
    q = (np.arange(16, dtype=np.float32) * 0.1).reshape(1, 4, 2, 2)
    k = (np.arange(8, dtype=np.float32) * 0.1 + 1.0).reshape(1, 2, 2, 2)
    v = (np.arange(8, dtype=np.float32) * 0.1 + 2.0).reshape(1, 2, 2, 2)
    out = run(device, q, k, v, 1 / np.sqrt(2))
    assert out.shape == (1, 4, 2, 2) and np.isfinite(out).all()
    check(device, q, k, v, 1 / np.sqrt(2))


def test_flash_attention_batch_key_mask(device):
    # fusor flash_attention.rs:315-358
    q = (np.arange(12, dtype=np.float32) * 0.1).reshape(2, 1, 3, 2)
    k = (np.arange(12, dtype=np.float32) * 0.1 + 1.0).reshape(2, 1, 3, 2)
    v = (np.arange(12, dtype=np.float32) * 0.1 + 2.0).reshape(2, 1, 3, 2)
    mask = np.array([[0, 0, 0], [0, 0, NEG_INF]], np.float32)
    out = run(device, q, k, v, 1 / np.sqrt(2), mask, fa.MaskKind.BatchKeyMask)
    assert out.shape == (2, 1, 3, 2) and np.isfinite(out).all()
    check(device, q, k, v, 1 / np.sqrt(2), mask, fa.MaskKind.BatchKeyMask)


def test_head_divisibility_panics(device):
    # fusor flash_attention.rs:94-99
    q = np.zeros((1, 3, 2, 2), np.float32)
    k = np.zeros((1, 2, 2, 2), np.float32)
    with pytest.raises(AssertionError, match=r"Number of Q heads \(3\) must be divisible by number of K/V heads \(2\)"):
        run(device, q, k, k, 1.0)


def test_mask_shape_panics(device):
    # fusor flash_attention.rs:153-172
    q = np.zeros((2, 1, 3, 2), np.float32)
    with pytest.raises(AssertionError, match=r"QKMask shape \[2, 3\] does not match expected \[3, 3\]"):
        run(device, q, q, q, 1.0, np.zeros((2, 3), np.float32), fa.MaskKind.QKMask)
    with pytest.raises(AssertionError, match=r"BatchKeyMask shape \[3, 3\] does not match expected \[2, 3\]"):
        run(device, q, q, q, 1.0, np.zeros((3, 3), np.float32), fa.MaskKind.BatchKeyMask)


# ---- the reference's fuzz tests, seeded ---------------------------------------------------------------

def _uniform(rng, shape):
    return (rng.random(shape, dtype=np.float32) * 2.0 - 1.0).astype(np.float32)


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16])
def test_masked_fuzz(device, dtype):
    # core flash_attention.rs:675-805: B 1..2, H 1..16, S 1..128, D 1..64; -inf above the diagonal,
    # random finite bias U(-0.25, 0.25) on and below it
    rng = np.random.default_rng(0xF10E)
    for it in range(40):
        B, H, S, D = rng.integers(1, 3), rng.integers(1, 17), rng.integers(1, 129), rng.integers(1, 65)
        q, k, v = (_uniform(rng, (B, H, S, D)) for _ in range(3))
        bias = rng.random((S, S), dtype=np.float32) * 0.5 - 0.25
        mask = np.where(np.arange(S)[None, :] > np.arange(S)[:, None], NEG_INF, bias).astype(np.float32)
        check(device, q, k, v, 1 / np.sqrt(np.float32(D)), mask, fa.MaskKind.QKMask, dtype,
              what=f"it{it} B{B} H{H} S{S} D{D}")


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16])
def test_kv_cache_fuzz(device, dtype):
    # core flash_attention.rs:807-921: Sq 1..4, Skv = Sq + 0..31, zero mask [Sq, Skv]
    rng = np.random.default_rng(0xF10F)
    for it in range(40):
        B, H, D = rng.integers(1, 3), rng.integers(1, 9), rng.integers(1, 65)
        Sq = rng.integers(1, 5)
        Skv = Sq + rng.integers(0, 32)
        q = _uniform(rng, (B, H, Sq, D))
        k, v = _uniform(rng, (B, H, Skv, D)), _uniform(rng, (B, H, Skv, D))
        mask = np.zeros((Sq, Skv), np.float32)
        check(device, q, k, v, 1 / np.sqrt(np.float32(D)), mask, fa.MaskKind.QKMask, dtype,
              what=f"it{it} B{B} H{H} Sq{Sq} Skv{Skv} D{D}")


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16, fa.BF16])
def test_gqa_fuzz(device, dtype):
    # core flash_attention.rs:923-1060: Hkv 1..4, G 1..4; reference there = K/V expanded by kv_h = h / G
    rng = np.random.default_rng(0xF110)
    tol = dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else None
    for it in range(30):
        B, Hkv, G = rng.integers(1, 3), rng.integers(1, 5), rng.integers(1, 5)
        S, D = rng.integers(1, 65), rng.integers(1, 65)
        q = _uniform(rng, (B, Hkv * G, S, D))
        k, v = _uniform(rng, (B, Hkv, S, D)), _uniform(rng, (B, Hkv, S, D))
        check(device, q, k, v, 1 / np.sqrt(np.float32(D)), None, None, dtype, tol=tol,
              what=f"it{it} B{B} Hkv{Hkv} G{G} S{S} D{D}")
        # bit-exact head mapping: expanding K/V on the host and calling with H == Hkv gives identical bits
        if it < 6:
            out_g = run(device, q, k, v, 0.25, dtype=dtype)
            out_e = run(device, q, np.repeat(k, G, axis=1), np.repeat(v, G, axis=1), 0.25, dtype=dtype)
            assert np.array_equal(out_g, out_e), "GQA head mapping differs from expand-then-MHA"


# ---- tiled kernels against the checker on shapes that select them ---------------------------------------

def _normal_qkv(seed, B, H, Hkv, Sq, Skv, D, scale=1.0):
    q = synth.normal(seed, 0, (B, H, Sq, D), scale)
    k = synth.normal(seed, 1, (B, Hkv, Skv, D), scale)
    v = synth.normal(seed, 2, (B, Hkv, Skv, D), scale)
    return q, k, v


def _analytic_mask(Sq, Skv, causal, off, window):
    i = np.arange(Sq)[:, None] + off
    j = np.arange(Skv)[None, :]
    masked = np.zeros((Sq, Skv), bool)
    if causal:
        masked |= j > i
    if window:
        masked |= (j + window) <= i
    return np.where(masked, NEG_INF, 0.0).astype(np.float32)


@pytest.mark.parametrize("dtype,D", [(fa.F16, 128), (fa.F16, 64), (fa.F16, 96), (fa.BF16, 128), (fa.F32, 64),
                                      (fa.F32, 128), (fa.F32, 32), (fa.F32, 96)])
@pytest.mark.parametrize("case", ["full", "causal", "causal_offset", "window", "ragged_tail"])
def test_prefill_tiled(device, dtype, D, case):
    want = fa.KERNEL_PREFILL_F32 if dtype == fa.F32 else fa.KERNEL_PREFILL_MFMA
    B, H, Hkv = 2, 4, 2
    Sq, Skv, analytic = {"full": (200, 333, None), "causal": (257, 257, (True, 0, 0)),
                         "causal_offset": (130, 400, (True, 270, 0)), "window": (300, 300, (True, 0, 100)),
                         "ragged_tail": (65, 127, None)}[case]
    q, k, v = _normal_qkv(11, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic) == want
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic).to_numpy()
    mask = None if analytic is None else _analytic_mask(Sq, Skv, *analytic)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask,
                                 "qk" if mask is not None else None)
    tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16)
    assert_parity(out, ref, tol, f"{case} D{D}")
    # the generic kernel with the dense mask tensor must agree too
    if mask is not None:
        tm = fa.Tensor.from_numpy(device, mask, dtype)
        out_g = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask), force_kernel=fa.KERNEL_GENERIC).to_numpy()
        assert_parity(out_g, ref, tol, f"generic {case} D{D}")


@pytest.mark.parametrize("D,B,H,Sq,Skv,analytic,form", [
    (64, 1, 4, 200, 200, (True, 0, 0), "four groups"),
    (64, 1, 8, 95, 700, (True, 605, 150), "four groups, window and cached keys"),
    (32, 1, 6, 333, 333, None, "four groups, no mask"),
    (64, 2, 32, 700, 700, (True, 0, 0), "two groups"),
    (64, 4, 48, 900, 900, (True, 0, 300), "one group"),
    (128, 1, 4, 300, 300, (True, 0, 0), "four groups of one wavefront that moves its tiles alone"),
    (96, 1, 4, 161, 417, (True, 256, 0), "four single-wavefront groups, cached keys"),
    (128, 1, 8, 95, 700, (True, 605, 150), "four single-wavefront groups, window and cached keys"),
    (100, 2, 6, 333, 333, None, "four single-wavefront groups, no mask, head_dim below the tile width"),
    (128, 1, 32, 700, 700, (True, 0, 0), "two groups"),
    (96, 2, 16, 700, 900, (True, 200, 0), "two groups, cached keys"),
    (128, 2, 40, 1000, 1000, (True, 0, 0), "one group"),
])
def test_prefill_f32_key_split_forms(device, D, B, H, Sq, Skv, analytic, form):
    """The f32 kernel splits a query block's keys over 1, 2 or 4 wavefront groups depending on how many
    workgroups the call has; each form is checked at ragged sizes (the grid sizes here select the form named)."""
    Hkv = H // 2
    q, k, v = _normal_qkv(12, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic) == fa.KERNEL_PREFILL_F32
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic).to_numpy()
    mask = None if analytic is None else _analytic_mask(Sq, Skv, *analytic)
    ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, "qk" if mask is not None else None)
    assert_parity(out, ref, TOL_F32, f"f32 D{D} {form}")


@pytest.mark.parametrize("dtype,D,B,H,Sq,Skv,analytic,form", [
    (fa.F16, 128, 2, 40, 600, 600, (True, 0, 0), "256-row blocks"),
    (fa.BF16, 64, 3, 32, 520, 900, (True, 380, 200), "256-row blocks, window and cached keys"),
    (fa.F16, 96, 4, 32, 300, 300, None, "256-row blocks, no mask"),
    (fa.F16, 128, 1, 8, 600, 600, (True, 0, 0), "key-split"),
    (fa.BF16, 64, 1, 8, 100, 1000, (True, 900, 300), "key-split, few rows, window and cached keys"),
    (fa.F16, 96, 2, 6, 333, 333, None, "key-split, no mask"),
    (fa.F16, 128, 1, 8, 130, 190, (True, 60, 0), "key-split, three key tiles"),
    (fa.F16, 128, 1, 32, 2000, 2000, (True, 0, 0), "key-split, one 256-row block per CU"),
])
def test_prefill_16_bit_workgroup_forms(device, dtype, D, B, H, Sq, Skv, analytic, form):
    """The 16-bit kernel runs 256 query rows per workgroup, or 128 rows with the key tiles alternating between
    its two wavefront groups, depending on how many workgroups the call has; each form is checked at ragged
    sizes (the grid sizes here select the form named)."""
    Hkv = H // 2
    q, k, v = _normal_qkv(13, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic) == fa.KERNEL_PREFILL_MFMA
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic).to_numpy()
    mask = None if analytic is None else _analytic_mask(Sq, Skv, *analytic)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask,
                                 "qk" if mask is not None else None)
    tol = dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16
    assert_parity(out, ref, tol, f"D{D} {form}")


@pytest.mark.parametrize("D", [80, 48, 4, 100, 124, 20])
@pytest.mark.parametrize("case", ["causal", "full_ragged", "bias"])
def test_prefill_f32_head_dims_between_the_tile_widths(device, D, case):
    """The f32 kernel pads head_dim to the next multiple of 32 with zeros on the way into LDS: Qwen-VL's vision
    blocks have head_dim 80 (models/kalosm-llama/src/raw/vision), other widths are covered for the same price."""
    B, H, Hkv = 2, 4, 2
    Sq, Skv = (150, 150) if case == "causal" else (70, 333)
    q, k, v = _normal_qkv(13, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v))
    mask, kind, analytic, mt = None, None, None, None
    if case == "causal":
        analytic = (True, 0, 0)
        mask, kind = _analytic_mask(Sq, Skv, True, 0, 0), "qk"
    elif case == "bias":
        mask, kind = np.random.default_rng(3).normal(0, 1, (Sq, Skv)).astype(np.float32), "qk"
        mask[:, 100:140] = NEG_INF
        mt = (fa.Tensor.from_numpy(device, mask, fa.F32), fa.MaskKind.QKMask)
    assert tq.selected_kernel(tk, tv, 0.1, mt, analytic=analytic) == fa.KERNEL_PREFILL_F32
    out = tq.flash_attention(tk, tv, D ** -0.5, mt, analytic=analytic).to_numpy()
    ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, kind)
    assert_parity(out, ref, TOL_F32, f"f32 head_dim {D} {case}")


@pytest.mark.parametrize("D", [256, 192, 132, 160])
@pytest.mark.parametrize("case", ["causal", "full_ragged", "window_offset", "mask_tensor", "bias_tensor"])
def test_prefill_f32_wide_heads(device, D, case):
    """head_dim 129..256 (Gemma-3's key length is 256): two wavefronts share 32 query rows, each owning half of
    the dims; the halves of every score are exchanged and added before the softmax."""
    B, H, Hkv = 2, 4, 2
    Sq, Skv = {"causal": (150, 150), "full_ragged": (70, 333), "window_offset": (97, 400), "mask_tensor": (130, 130),
               "bias_tensor": (64, 100)}[case]
    q, k, v = _normal_qkv(14, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v))
    mask, kind, analytic, mt, want = None, None, None, None, fa.KERNEL_PREFILL_F32
    if case == "causal":
        analytic = (True, 0, 0)
    elif case == "window_offset":
        analytic = (True, Skv - Sq, 120)
    elif case == "mask_tensor":
        mask = oracle.get_mask(Sq, 0, 50)
        mt = (fa.Tensor.from_numpy(device, mask, fa.F32), fa.MaskKind.QKMask)
    elif case == "bias_tensor":  # no interval form and no mask-adding form this wide: the general kernel
        mask = np.random.default_rng(3).normal(0, 1, (Sq, Skv)).astype(np.float32)
        mt = (fa.Tensor.from_numpy(device, mask, fa.F32), fa.MaskKind.QKMask)
    if analytic is not None:
        mask = _analytic_mask(Sq, Skv, *analytic)
    out = tq.flash_attention(tk, tv, D ** -0.5, mt, analytic=analytic).to_numpy()
    ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, None if mask is None else "qk")
    assert_parity(out, ref, TOL_F32, f"f32 head_dim {D} {case}")
    if mt is None:
        assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic) == want


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("D,case", [(84, "causal"), (148, "causal"), (204, "window_offset"), (36, "full_ragged"), (44, "causal"),
                                    (128, "bias"), (64, "bias"), (96, "bias_batch_key")])
def test_16_bit_tensors_on_the_f32_arithmetic_kernel(device, dtype, D, case):
    """Head dims (multiples of 4 that are not multiples of 8) and mask tensors the 16-bit matrix-core kernels do not take
    run on the tiled kernel that computes in f32: rows are widened on their way into LDS, the result is rounded to the
    tensors' type."""
    B, H, Hkv = 2, 4, 2
    Sq, Skv = {"causal": (150, 150), "window_offset": (97, 400), "full_ragged": (70, 333), "bias": (90, 200),
               "bias_batch_key": (90, 200)}[case]
    q, k, v = _normal_qkv(15, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    mask, kind, analytic, mt = None, None, None, None
    if case == "causal":
        analytic = (True, 0, 0)
    elif case == "window_offset":
        analytic = (True, Skv - Sq, 120)
    elif case == "bias":
        mask, kind = np.random.default_rng(3).normal(0, 1, (Sq, Skv)).astype(np.float32), "qk"
        mask[:, 100:140] = NEG_INF
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif case == "bias_batch_key":
        mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
        mask[0, 150:] = -10000.0
        mask[1, :20] = -10000.0
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.BatchKeyMask)
    if analytic is not None:
        mask, kind = _analytic_mask(Sq, Skv, *analytic), "qk"
    if mt is None:
        assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic) == fa.KERNEL_PREFILL_F32
    out = tq.flash_attention(tk, tv, D ** -0.5, mt, analytic=analytic).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                 None if mask is None else rounded(mask, dtype), kind)
    tol = dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16
    assert_parity(out, ref, tol, f"16-bit on the f32 kernel, D{D} {case}")
    # and with an f32 result the only rounding left is the inputs'
    if mt is None:
        out32 = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic, out_dtype=fa.F32).to_numpy()
        assert out32.dtype == np.float32
        assert_parity(out32, ref, TOL_F32, f"f32 result, D{D} {case}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("D", [160, 192, 224, 256, 8, 40, 80, 144, 200, 32])
@pytest.mark.parametrize("case", ["causal", "chunk_window", "ragged", "mask_tensor", "bias", "padding_mask", "cache_views", "full"])
def test_wide_head_dims_on_the_16_bit_matrix_cores(device, dtype, D, case):
    """Head dims 160 ... 256 (Gemma-3's key length is 256), and every other multiple of 8 that is not 64 / 96 / 128 (80 in
    Qwen-VL's vision blocks), padded with zeros to the next multiple of 32, in 16-bit: the four-wavefront tiled kernel, 128 query rows per
    workgroup and 32-key tiles; every way of masking, rows and keys that do not fill their last block or tile, K and V
    as narrowed views of a larger cache allocation, GQA, and the output in f32 as well."""
    B, H, Hkv = 2, 6, 2
    Sq, Skv = {"causal": (300, 300), "chunk_window": (130, 1000), "ragged": (70, 777), "mask_tensor": (150, 419),
               "bias": (90, 200), "padding_mask": (129, 333), "cache_views": (200, 200), "full": (33, 1)}[case]
    q, k, v = _normal_qkv(16, B, H, Hkv, Sq, Skv, D)
    tq = fa.Tensor.from_numpy(device, q, dtype)
    if case == "cache_views":
        kbuf, vbuf = np.zeros((B, Hkv, 256, D), np.float32), np.zeros((B, Hkv, 256, D), np.float32)
        kbuf[:, :, :Skv], vbuf[:, :, :Skv] = k, v
        tk = fa.Tensor.from_numpy(device, kbuf, dtype).narrow(2, 0, Skv)
        tv = fa.Tensor.from_numpy(device, vbuf, dtype).narrow(2, 0, Skv)
    else:
        tk, tv = fa.Tensor.from_numpy(device, k, dtype), fa.Tensor.from_numpy(device, v, dtype)
    mask, kind, mt, kw = None, None, None, {}
    lens = None
    if case in ("causal", "cache_views"):
        kw["analytic"] = (True, 0, 0)
        mask, kind = _analytic_mask(Sq, Skv, True, 0, 0), "qk"
    elif case == "chunk_window":
        kw["analytic"] = (True, Skv - Sq, 333)
        mask, kind = _analytic_mask(Sq, Skv, True, Skv - Sq, 333), "qk"
    elif case == "ragged":
        lens = np.array([777, 95], np.int32)
        kw["kv_lens"] = fa.IntTensor(device, lens)
    elif case == "mask_tensor":
        mask, kind = oracle.get_mask(Sq, Skv - Sq, None), "qk"
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif case == "bias":  # not made of intervals: the kernel queued behind the tiled one serves the call
        mask, kind = np.random.default_rng(3).normal(0, 1, (Sq, Skv)).astype(np.float32), "qk"
        mask[:, 100:140] = NEG_INF
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif case == "padding_mask":
        mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
        mask[0, 300:] = NEG_INF
        mask[1, :50] = NEG_INF
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.BatchKeyMask)
    if mt is None:
        assert tq.selected_kernel(tk, tv, 0.1, **kw) == fa.KERNEL_PREFILL_MFMA
    tol = dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16
    for out_dtype in (None, fa.F32):
        out = tq.flash_attention(tk, tv, D ** -0.5, mt, out_dtype=out_dtype, **kw).to_numpy()
        if lens is None:
            ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                         None if mask is None else rounded(mask, dtype), kind)
            assert_parity(out, ref, tol, f"D{D} {case} out {out_dtype}")
        else:
            for b in range(B):
                n = int(lens[b])
                ref = oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                             rounded(v[b:b + 1, :, :n], dtype), D ** -0.5)
                assert_parity(out[b:b + 1], ref, tol, f"D{D} ragged b{b} out {out_dtype}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16, fa.F32])
@pytest.mark.parametrize("G,D,Skv", [(4, 128, 1000), (1, 96, 777), (8, 64, 513), (2, 128, 64), (3, 128, 300),
                                     (4, 32, 5000), (1, 128, 1), (16, 128, 260), (20, 64, 700), (4, 72, 900),
                                     (2, 40, 333), (8, 8, 100), (2, 256, 1500), (4, 192, 700), (1, 160, 300),
                                     (8, 256, 260), (4, 224, 2100), (16, 256, 130)])
def test_decode_splitkv(device, dtype, G, D, Skv):
    B, Hkv = 3, 2
    q, k, v = _normal_qkv(12, B, Hkv * G, Hkv, 1, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5)
    tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=1e-2, rel_l2=5e-3) if dtype == fa.BF16 else TOL_16)
    assert_parity(out, ref, tol, f"decode G{G} D{D} Skv{Skv}")


def test_decode_f32_with_the_masks_the_reference_passes(device):
    """kalosm-llama decodes in f32 with get_mask(1, pos, window) as a QKMask (raw/mod.rs:618-620,
    attention_layer.rs:400-448); a padded batch would come as a BatchKeyMask."""
    B, H, Hkv, D, Skv = 2, 8, 2, 128, 1500
    q, k, v = _normal_qkv(18, B, H, Hkv, 1, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v))
    qk = oracle.get_mask(1, Skv - 1, None)                       # [1, 1500] zeros
    assert qk.shape == (1, Skv)
    out = tq.flash_attention(tk, tv, D ** -0.5, (fa.Tensor.from_numpy(device, qk, fa.F32), fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(q, k, v, D ** -0.5, qk, "qk")
    assert_parity(out, ref, TOL_F32, "f32 decode, QKMask")
    bk = np.zeros((B, Skv), np.float32)
    bk[0, 1000:] = NEG_INF
    bk[1, :200] = NEG_INF
    out = tq.flash_attention(tk, tv, D ** -0.5, (fa.Tensor.from_numpy(device, bk, fa.F32), fa.MaskKind.BatchKeyMask)).to_numpy()
    ref = oracle.flash_attention(q, k, v, D ** -0.5, bk, "batch_key")
    assert_parity(out, ref, TOL_F32, "f32 decode, BatchKeyMask")
    # cached K/V arrive as narrowed views of a power-of-two allocation (tensor_cache.rs:107-110)
    kbuf = np.zeros((B, Hkv, 2048, D), np.float32)
    vbuf = np.zeros((B, Hkv, 2048, D), np.float32)
    kbuf[:, :, :Skv], vbuf[:, :, :Skv] = k, v
    tkn = fa.Tensor.from_numpy(device, kbuf, fa.F32).narrow(2, 0, Skv)
    tvn = fa.Tensor.from_numpy(device, vbuf, fa.F32).narrow(2, 0, Skv)
    assert tq.selected_kernel(tkn, tvn, 0.1) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tkn, tvn, D ** -0.5).to_numpy()
    assert_parity(out, oracle.flash_attention(q, k, v, D ** -0.5), TOL_F32, "f32 decode, cache views")


@pytest.mark.parametrize("dtype,B,H,Hkv,D,Skv", [(fa.F16, 1, 8, 2, 128, 6000), (fa.F32, 1, 4, 2, 256, 5200),
                                                  (fa.F32, 2, 6, 3, 64, 9000), (fa.BF16, 3, 4, 1, 96, 7000),
                                                  (fa.F16, 1, 8, 4, 256, 9000), (fa.BF16, 2, 4, 2, 160, 6000),
                                                  (fa.F32, 1, 8, 4, 192, 5000)])
def test_decode_with_many_splits_and_few_rows(device, dtype, B, H, Hkv, D, Skv):
    """One chat stream on a long cache: tens of splits per (batch, head) row and only a few rows, which the combine
    pass handles with four wavefronts per row (two rounds of 128 dims at head_dim 256); ragged lengths on top."""
    q, k, v = _normal_qkv(31, B, H, Hkv, 1, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1) == fa.KERNEL_DECODE_SPLITKV
    tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16)
    out = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5)
    assert_parity(out, ref, tol, "all keys")
    lens = np.array([Skv - 7, 300, 4097][:B], np.int32)
    out = tq.flash_attention(tk, tv, D ** -0.5, kv_lens=fa.IntTensor(device, lens)).to_numpy()
    for b in range(B):
        n = int(lens[b])
        ref = oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                     rounded(v[b:b + 1, :, :n], dtype), D ** -0.5)
        assert_parity(out[b:b + 1], ref, tol, f"sequence {b} of length {n}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16, fa.F32])
@pytest.mark.parametrize("case", ["window", "window_as_tensor", "padding_mask", "full"])
def test_decode_at_head_dim_256_with_a_sliding_window(device, dtype, case):
    """Gemma-3's attention shape (key length 256, 8 query heads on 4 KV heads, sliding layers with a window of 1024):
    a decode step on a long cache, the window as the analytic descriptor and as the [1, Skv] tensor
    MaskCache::get_mask builds; a left- and right-padded batch as a BatchKeyMask.  16-bit tensors run on the
    matrix-core variant (one workgroup per CU at this head_dim), f32 tensors on the vector variant."""
    B, H, Hkv, D, Skv, W = 5, 8, 4, 256, 3100, 1024
    q, k, v = _normal_qkv(71, B, H, Hkv, 1, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=1e-2, rel_l2=5e-3) if dtype == fa.BF16 else TOL_16)
    mask = kind = None
    kw = {}
    m = None
    if case in ("window", "window_as_tensor"):
        mask, kind = _analytic_mask(1, Skv, True, Skv - 1, W), "qk"
        if case == "window":
            kw["analytic"] = (True, Skv - 1, W)
        else:
            m = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif case == "padding_mask":
        mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
        mask[0, 3000:] = NEG_INF
        mask[1, :700] = NEG_INF
        mask[3, 1:] = NEG_INF
        m = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.BatchKeyMask)
    assert tq.selected_kernel(tk, tv, 0.1, m, **kw) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5, m, **kw).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask, kind)
    assert_parity(out, ref, tol, case)


def test_decode_ragged_kv_lens(device):
    # per-sequence lengths == un-padded calls == -inf BatchKeyMask padding
    B, H, Hkv, D, Smax = 5, 4, 4, 96, 3000
    lens = np.array([3000, 1, 129, 1024, 2047], np.int32)
    q, k, v = _normal_qkv(13, B, H, Hkv, 1, Smax, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    out = tq.flash_attention(tk, tv, D ** -0.5, kv_lens=fa.IntTensor(device, lens)).to_numpy()
    bk = np.where(np.arange(Smax)[None, :] < lens[:, None], 0.0, NEG_INF).astype(np.float32)
    out_m = tq.flash_attention(tk, tv, D ** -0.5, (fa.Tensor.from_numpy(device, bk, fa.F16), fa.MaskKind.BatchKeyMask)).to_numpy()
    for b in range(B):
        n = int(lens[b])
        ref = oracle.flash_attention(rounded(q[b:b + 1], fa.F16), rounded(k[b:b + 1, :, :n], fa.F16),
                                     rounded(v[b:b + 1, :, :n], fa.F16), D ** -0.5)
        assert_parity(out[b:b + 1], ref, TOL_16, f"kv_lens b{b} len{n}")
        assert_parity(out_m[b:b + 1], ref, TOL_16, f"batch-key mask b{b} len{n}")


def test_strided_views(device):
    # K/V as narrowed views of a larger cache allocation, V as the transposed view of [B,S,Hkv,D],
    # Q transposed from [B,S,H,D] (kalosm-llama attention_layer.rs:257-270; tensor_cache.rs:107-110)
    B, H, Hkv, S, D, alloc = 2, 8, 2, 150, 64, 256
    q, k, v = _normal_qkv(14, B, H, Hkv, S, S, D)
    for dtype in (fa.F32, fa.F16):
        kbuf = np.zeros((B, Hkv, alloc, D), np.float32)
        kbuf[:, :, :S] = k
        tk = fa.Tensor.from_numpy(device, kbuf, dtype).narrow(2, 0, S)
        tv = fa.Tensor.from_numpy(device, np.ascontiguousarray(v.transpose(0, 2, 1, 3)), dtype).transpose(1, 2)
        tq = fa.Tensor.from_numpy(device, np.ascontiguousarray(q.transpose(0, 2, 1, 3)), dtype).transpose(1, 2)
        assert tk.strides[1] == alloc * D and tv.strides == (S * Hkv * D, D, Hkv * D, 1)
        out = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, 0, 0)).to_numpy()
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                     oracle.get_mask(S, 0), "qk")
        assert_parity(out, ref, TOL_F32 if dtype == fa.F32 else TOL_16, "strided views")
        # fully general strides (innermost stride != 1) fall back to the generic kernel
        tq2 = fa.Tensor.from_numpy(device, np.ascontiguousarray(q.transpose(0, 1, 3, 2)), dtype).transpose(2, 3)
        assert tq2.selected_kernel(tk, tv, 1.0) == fa.KERNEL_GENERIC
        out2 = tq2.flash_attention(tk, tv, D ** -0.5, analytic=(True, 0, 0)).to_numpy()
        assert_parity(out2, ref, TOL_F32 if dtype == fa.F32 else TOL_16, "generic strided")


def test_f32_output_for_f16_inputs(device):
    q, k, v = _normal_qkv(15, 1, 4, 2, 300, 300, 128)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    out = tq.flash_attention(tk, tv, 128 ** -0.5, analytic=(True, 0, 0), out_dtype=fa.F32).to_numpy()
    assert out.dtype == np.float32
    ref = oracle.flash_attention(rounded(q, fa.F16), rounded(k, fa.F16), rounded(v, fa.F16), 128 ** -0.5,
                                 oracle.get_mask(300, 0), "qk")
    assert_parity(out, ref, TOL_16, "f32 out")


def test_fully_masked_row_is_nan(device):
    # the reference gives NaN for a row with no visible key ((-inf) - (-inf), fusor :184-196)
    q, k, v = _normal_qkv(16, 1, 1, 1, 4, 4, 8)
    mask = np.zeros((4, 4), np.float32)
    mask[2, :] = NEG_INF
    out = run(device, q, k, v, 1.0, mask, fa.MaskKind.QKMask)
    ref = oracle.flash_attention(q, k, v, 1.0, mask, "qk")
    assert np.isnan(out[0, 0, 2]).all() and np.isnan(ref[0, 0, 2]).all()
    keep = [0, 1, 3]
    assert_parity(out[:, :, keep], ref[:, :, keep], TOL_F32, "unmasked rows")


@pytest.mark.parametrize("dtype,Sq", [(fa.F16, 200), (fa.F32, 200), (fa.F16, 1), (fa.BF16, 70)])
def test_output_written_as_batch_seq_heads_dim(device, dtype, Sq):
    """The layout kalosm-llama needs next: attention output transposed to [B, Sq, H, D] and flattened for
    attention_wo (attention_layer.rs:450-454).  The caller passes that buffer as a strided [B, H, Sq, D]
    view and the kernels (tiled prefill, split-KV decode, general) write it in place of a transpose pass."""
    B, H, Hkv, D, Skv = 2, 8, 2, 128, 300
    q, k, v = _normal_qkv(17, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    analytic = (True, Skv - Sq, 0)
    plain = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic).to_numpy()
    for kernel in (fa.KERNEL_AUTO, fa.KERNEL_GENERIC):
        buf = fa.Tensor.empty(device, (B, Sq, H, D), dtype)           # [B, Sq, H*D] once flattened
        tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic, out=buf.transpose(1, 2), force_kernel=kernel)
        got = buf.to_numpy().transpose(0, 2, 1, 3)
        if kernel == fa.KERNEL_AUTO:
            assert np.array_equal(got, plain), "same kernel, different output strides: bits must agree"
        else:
            tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16)
            assert_parity(got.astype(np.float32), plain.astype(np.float32), tol, "general kernel, transposed output")


@pytest.mark.parametrize("dtype,Sq", [(fa.F16, 300), (fa.F32, 200), (fa.F16, 1)])
def test_broadcast_views_of_one_kv_head(device, dtype, Sq):
    """The reference expands K/V over the query heads with reshape + broadcast_to (stride 0) before its matmuls
    (fusor flash_attention.rs:104-138).  The op takes such a view directly: one stored KV head repeated for every
    query head gives the same result as the grouped call."""
    B, H, D, Skv = 2, 8, 64, 333
    q, k, v = _normal_qkv(31, B, H, 1, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    kb, vb = tk.broadcast_to((B, H, Skv, D)), tv.broadcast_to((B, H, Skv, D))
    assert kb.strides[1] == 0 and kb.shape == (B, H, Skv, D)
    out_b = tq.flash_attention(kb, vb, D ** -0.5).to_numpy()
    out_g = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, None, None)
    tol = TOL_F32 if dtype == fa.F32 else TOL_16
    assert_parity(out_b, ref, tol, "broadcast kv heads")
    assert_parity(out_g, ref, tol, "one kv head, grouped")
    if Sq > 1:  # the tiled kernels walk the keys in the same order either way (the decode split differs)
        assert np.array_equal(out_b.view(np.uint8), out_g.view(np.uint8))


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16])
def test_tensors_without_elements(device, dtype):
    """No output element: nothing is computed.  No key: the reference's composite multiplies [Sq, 0] probabilities
    with [0, D] values, which is all zeros, not NaN (fusor flash_attention.rs:141-199; a row whose keys are all
    MASKED is the NaN case)."""
    D = 64
    for B, H, Hkv, Sq, Skv in ((0, 4, 2, 5, 7), (2, 0, 0, 5, 7), (2, 4, 2, 0, 7)):
        tq = fa.Tensor.from_numpy(device, np.zeros((B, H, Sq, D), np.float32), dtype)
        tk = fa.Tensor.from_numpy(device, np.zeros((B, Hkv, Skv, D), np.float32), dtype)
        out = tq.flash_attention(tk, tk, 0.125).to_numpy()
        assert out.shape == (B, H, Sq, D) and out.size == 0
    q = _normal_qkv(41, 2, 4, 2, 5, 1, D)[0]
    tq = fa.Tensor.from_numpy(device, q, dtype)
    tk = fa.Tensor.from_numpy(device, np.zeros((2, 2, 0, D), np.float32), dtype)
    out_t = fa.Tensor.from_numpy(device, np.full((2, 4, 5, D), 7.0, np.float32), dtype)  # must be overwritten
    args = tq._attn_args(tk, tk, 0.125, None, None, None, None, fa.KERNEL_AUTO, out_t)
    import ctypes
    fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    out = out_t.to_numpy()
    assert out.shape == (2, 4, 5, D) and not out.any()
    # the same into an output view whose innermost stride is not 1 (the zeros are written element by element)
    out_s = fa.Tensor.from_numpy(device, np.full((2, 4, D, 5), 7.0, np.float32), dtype).transpose(2, 3)
    assert out_s.shape == (2, 4, 5, D) and out_s.strides[3] == 5
    args = tq._attn_args(tk, tk, 0.125, None, None, None, None, fa.KERNEL_AUTO, out_s)
    fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    assert not out_s.to_numpy().any()
    # heads that cannot be grouped still panic, as u32::is_multiple_of does for a zero divisor
    with pytest.raises(AssertionError, match="divisible"):
        tq.flash_attention(fa.Tensor.from_numpy(device, np.zeros((2, 0, 3, D), np.float32), dtype),
                           fa.Tensor.from_numpy(device, np.zeros((2, 0, 3, D), np.float32), dtype), 0.125)


@pytest.mark.parametrize("dtype,D", [(fa.F16, 128), (fa.F32, 64)])
def test_decode_over_a_very_long_cache(device, dtype, D):
    """Half a million keys for one sequence: hundreds of splits, 64-bit row offsets, several rounds in the merge."""
    Skv = 500_003
    q, k, v = _normal_qkv(16, 1, 2, 1, 1, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
    # Half a million f32 terms summed left to right (the reference's fold) carry more rounding error than the 1e-5
    # the benchmark sizes are held to, so the referee here is the float64 definition: the device result must be at
    # least as close to it as the f32 restatement is, and within the usual bound
    qr, kr, vr = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
    exact = oracle.flash_attention_f64(qr, kr, vr, D ** -0.5)
    restated = oracle.flash_attention(qr, kr, vr, D ** -0.5)
    from conftest import rel_l2
    err_dev, err_restated = rel_l2(out, exact), rel_l2(restated, exact)
    bound = 1e-5 if dtype == fa.F32 else 1e-3
    assert err_dev <= max(bound, 1.5 * err_restated), (err_dev, err_restated)
    assert not np.isnan(out).any()
    # the last position only (a sliding window of one key) must return that key's value row
    out1 = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, Skv - 1, 1)).to_numpy()
    want = rounded(v, dtype)[:, :1, Skv - 1:Skv].repeat(2, axis=1)
    assert_parity(out1, want, dict(max_abs=1e-6, rel_l2=1e-6) if dtype == fa.F32 else TOL_16, "window of one key at the end")


@pytest.mark.parametrize("dtype,D", [(fa.F32, 128), (fa.F32, 64), (fa.F32, 80), (fa.F16, 80), (fa.BF16, 40), (fa.F16, 128),
                                     (fa.BF16, 64), (fa.F16, 96), (fa.F32, 256), (fa.F16, 192)])
@pytest.mark.parametrize("case", ["causal_offset", "window", "mask_tensor", "bias_tensor", "kv_lens", "full"])
def test_few_query_rows_on_a_long_cache_split_the_keys(device, dtype, D, case):
    """A new chat turn on a long cached context: few query blocks, thousands of keys.  Both tiled prefill kernels
    then split the keys over workgroups and merge the shares; the result must not depend on it."""
    B, H, Hkv, Sq, Skv = 1, 4, 2, 100, 5000
    q, k, v = _normal_qkv(17, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    mask, kind, analytic, mt, lens_t = None, None, None, None, None
    if case == "causal_offset":
        analytic = (True, Skv - Sq, 0)
    elif case == "window":
        analytic = (True, Skv - Sq, 1500)
    elif case == "mask_tensor":
        mask, kind = oracle.get_mask(Sq, Skv - Sq), "qk"
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif case == "bias_tensor":
        mask, kind = np.random.default_rng(4).normal(0, 1, (Sq, Skv)).astype(np.float32), "qk"
        mask[:, 700:2100] = NEG_INF
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif case == "kv_lens":
        lens_t = fa.IntTensor(device, np.array([3333], np.int32))
        mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
        mask[0, 3333:] = NEG_INF
    if analytic is not None:
        mask, kind = _analytic_mask(Sq, Skv, *analytic), "qk"
    # with the workspace the library asks for (the keys are split) ...
    need = ctypes.c_size_t()
    args = tq._attn_args(tk, tv, D ** -0.5, mt, analytic, lens_t, None, fa.KERNEL_AUTO, None)
    fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
    assert need.value > B * H * Sq * 2 * (D + 2) * 4, "the size query must ask for room for at least two shares"
    out = tq.flash_attention(tk, tv, D ** -0.5, mt, analytic=analytic, kv_lens=lens_t).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                 None if mask is None else rounded(mask, dtype), kind)
    tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16)
    assert_parity(out, ref, tol, f"split keys, {case} D{D}")
    # ... and without any workspace (one workgroup walks all keys of its query block)
    out_t = fa.Tensor.empty(device, (B, H, Sq, D), dtype)
    args = tq._attn_args(tk, tv, D ** -0.5, mt, analytic, lens_t, None, fa.KERNEL_AUTO, out_t)
    fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    assert_parity(out_t.to_numpy(), ref, tol, f"unsplit, {case} D{D}")


@pytest.mark.parametrize("dtype,D,G,Sq", [(fa.F32, 256, 4, 20), (fa.F32, 256, 2, 32), (fa.F32, 160, 4, 17), (fa.F32, 200, 6, 17),
                                          (fa.F16, 148, 2, 30), (fa.F32, 256, 3, 20)])
@pytest.mark.parametrize("case", ["causal_offset", "window", "mask_tensor", "kv_lens", "full"])
def test_few_rows_above_head_dim_128_in_f32_arithmetic_pair_two_heads(device, dtype, D, G, Sq, case):
    """Up to 32 new rows on a long cache above head_dim 128 on the f32-arithmetic kernel (Gemma-3's key length in the
    type kalosm-llama calls with): with an even GQA group the workgroup's two wavefront pairs hold the rows of two query
    heads of one KV head and share its K/V tiles; with an odd group (the last case) one head per workgroup as before.
    With the workspace the library asks for (keys split over workgroups) and without any."""
    B, Hkv, Skv = 2, 2, 3000
    H = Hkv * G
    q, k, v = _normal_qkv(19, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    mask, kind, analytic, mt, lens_t = None, None, None, None, None
    if case == "causal_offset":
        analytic = (True, Skv - Sq, 0)
    elif case == "window":
        analytic = (True, Skv - Sq, 1000)
    elif case == "mask_tensor":
        mask, kind = oracle.get_mask(Sq, Skv - Sq), "qk"
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif case == "kv_lens":
        lens = np.array([2222, 77], np.int32)
        lens_t = fa.IntTensor(device, lens)
        mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
        mask[0, 2222:] = NEG_INF
        mask[1, 77:] = NEG_INF
    if analytic is not None:
        mask, kind = _analytic_mask(Sq, Skv, *analytic), "qk"
    if mt is None:
        assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic, kv_lens=lens_t) == fa.KERNEL_PREFILL_F32
    out = tq.flash_attention(tk, tv, D ** -0.5, mt, analytic=analytic, kv_lens=lens_t).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                 None if mask is None else rounded(mask, dtype), kind)
    tol = TOL_F32 if dtype == fa.F32 else TOL_16
    assert_parity(out, ref, tol, f"split keys, {case} D{D} G{G} Sq{Sq}")
    out_t = fa.Tensor.empty(device, (B, Sq, H, D), dtype)  # written as [B, Sq, H, D], no workspace
    args = tq._attn_args(tk, tv, D ** -0.5, mt, analytic, lens_t, None, fa.KERNEL_AUTO, out_t.transpose(1, 2))
    fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    assert_parity(out_t.to_numpy().transpose(0, 2, 1, 3), ref, tol, f"unsplit, {case} D{D} G{G} Sq{Sq}")


@pytest.mark.parametrize("dtype,D,Sq", [(fa.F16, 96, 1), (fa.BF16, 128, 1), (fa.F16, 64, 2), (fa.F16, 32, 1)])
def test_decode_with_a_unit_per_cu_takes_the_eight_wavefront_form(device, dtype, D, Sq):
    """At least one (batch, kv head) unit per CU and more than 2048 keys: the 16-bit matrix-core variant runs with eight
    wavefronts per workgroup on chunks of 2048 keys (fewer, longer workgroups).  All keys, then ragged lengths."""
    B, H, Hkv, Skv = 9, 32, 32, 4500
    assert B * Hkv >= device.compute_units
    q, k, v = _normal_qkv(47, B, H, Hkv, Sq, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1) == fa.KERNEL_DECODE_SPLITKV
    # three splits of 2048 keys per (batch, head, row) on eight wavefronts; the workspace holds their partials (and, up to
    # 8 splits, the padding and counters of the merge inside the main kernel)
    plan = tq.decode_plan(tk, tv, 0.1)
    assert (plan["nsplit"], plan["chunk"], plan["wavefronts"]) == (3, 2048, 8), plan
    need = ctypes.c_size_t()
    args = tq._attn_args(tk, tv, 0.1, None, None, None, None, fa.KERNEL_AUTO, None)
    fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
    partials = B * H * Sq * 3 * (D + 2) * 4
    assert partials <= need.value <= partials + B * Hkv * (3 * 128 + 4) + 256
    tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=1e-2, rel_l2=5e-3) if dtype == fa.BF16 else TOL_16)
    analytic = (True, Skv - Sq, 0) if Sq > 1 else None
    mask = _analytic_mask(Sq, Skv, True, Skv - Sq, 0) if Sq > 1 else None
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask,
                                 None if mask is None else "qk")
    assert_parity(out, ref, tol, "all keys")
    if Sq == 1:
        lens = np.array([4500, 1, 2048, 2049, 4096, 300, 4097, 2047, 3333], np.int32)
        out = tq.flash_attention(tk, tv, D ** -0.5, kv_lens=fa.IntTensor(device, lens)).to_numpy()
        for b in range(B):
            n = int(lens[b])
            ref = oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                         rounded(v[b:b + 1, :, :n], dtype), D ** -0.5)
            assert_parity(out[b:b + 1], ref, tol, f"sequence {b} of length {n}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("D", [160, 192, 224, 256])
@pytest.mark.parametrize("case", ["causal", "chunk_window", "ragged"])
def test_wide_head_dims_on_a_grid_that_fills_the_chip(device, dtype, D, case):
    """The wide-head kernel has three workgroup shapes: 64 query rows (two workgroups per CU) on small grids, and where
    128-row workgroups fill the chip twice over 128 rows (head dims 224 and 256; also every split or packed call) or
    256 rows (32 rows per wavefront, up to head_dim 192).  The other tests of these head dims are small grids; here
    4 x 64 heads x 130 rows reach twice the CU count in 128-row blocks (the second block holds two rows)."""
    B, H, Hkv, Sq = 4, 64, 16, 130
    assert B * H * ((Sq + 127) // 128) >= 2 * device.compute_units
    Skv = {"causal": 130, "chunk_window": 400, "ragged": 333}[case]
    q, k, v = _normal_qkv(23, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    kw, mask, lens = {}, None, None
    if case == "causal":
        kw["analytic"] = (True, 0, 0)
        mask = _analytic_mask(Sq, Skv, True, 0, 0)
    elif case == "chunk_window":
        kw["analytic"] = (True, Skv - Sq, 200)
        mask = _analytic_mask(Sq, Skv, True, Skv - Sq, 200)
    else:
        lens = np.array([333, 41, 1, 200], np.int32)
        kw["kv_lens"] = fa.IntTensor(device, lens)
    assert tq.selected_kernel(tk, tv, 0.1, **kw) == fa.KERNEL_PREFILL_MFMA
    out = tq.flash_attention(tk, tv, D ** -0.5, **kw).to_numpy()
    tol = dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16
    for b in range(B):
        n = Skv if lens is None else int(lens[b])
        ref = oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                     rounded(v[b:b + 1, :, :n], dtype), D ** -0.5, mask, None if mask is None else "qk")
        assert_parity(out[b:b + 1], ref, tol, f"D{D} {case}, sequence {b}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16, fa.F32])
@pytest.mark.parametrize("D", [64, 128, 160, 256])
def test_memory_behind_a_cache_view_is_never_used(device, dtype, D):
    """K and V are views of the first 333 rows of a 512-row cache allocation whose other rows hold NaN.  The tiled kernels
    fetch whole 32- or 64-key tiles; the rows of the last tile that lie beyond the view must not reach the result (the
    16-bit kernels fetch them through a buffer descriptor that ends with the view and get zeros; a NaN there would
    survive the masking as 0 x NaN in P . V)."""
    B, H, Hkv, Sq, Skv, cap = 1, 4, 2, 200, 333, 512
    rng = np.random.default_rng(12)
    q = rng.normal(0, 1, (B, H, Sq, D)).astype(np.float32)
    kbuf = np.full((B, Hkv, cap, D), np.nan, np.float32)
    vbuf = np.full((B, Hkv, cap, D), np.nan, np.float32)
    kbuf[:, :, :Skv] = rng.normal(0, 1, (B, Hkv, Skv, D))
    vbuf[:, :, :Skv] = rng.normal(0, 1, (B, Hkv, Skv, D))
    tq = fa.Tensor.from_numpy(device, q, dtype)
    tk = fa.Tensor.from_numpy(device, kbuf, dtype).narrow(2, 0, Skv)
    tv = fa.Tensor.from_numpy(device, vbuf, dtype).narrow(2, 0, Skv)
    for analytic in ((True, Skv - Sq, 0), None):
        kw = {} if analytic is None else {"analytic": analytic}
        assert tq.selected_kernel(tk, tv, D ** -0.5, **kw) == (fa.KERNEL_PREFILL_F32 if dtype == fa.F32 else fa.KERNEL_PREFILL_MFMA)
        out = tq.flash_attention(tk, tv, D ** -0.5, **kw).to_numpy()
        mask = None if analytic is None else _analytic_mask(Sq, Skv, *analytic)
        ref = oracle.flash_attention(rounded(q, dtype), rounded(kbuf[:, :, :Skv], dtype), rounded(vbuf[:, :, :Skv], dtype),
                                     D ** -0.5, mask, None if mask is None else "qk")
        tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16)
        assert_parity(out, ref, tol, f"D{D}, mask {analytic}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16, fa.F32])
@pytest.mark.parametrize("D", [64, 80, 128, 160, 256])
@pytest.mark.parametrize("Sq", [1, 4, 40, 200])
def test_rows_beyond_a_sequence_s_own_keys_are_never_used(device, dtype, D, Sq):
    """A ragged batch in one cache allocation: kv_lens below the view's length, and NaN in the rows between a
    sequence's own keys and the end of the view (what an uninitialised cache holds there is the caller's business).
    Decode and prefill kernels fetch whole steps or tiles; none of it may reach the result."""
    B, H, Hkv, Skv = 2, 4, 2, 700
    lens = np.array([333, 401], np.int32)
    rng = np.random.default_rng(13)
    q = rng.normal(0, 1, (B, H, Sq, D)).astype(np.float32)
    k = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    v = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    kn, vn = k.copy(), v.copy()
    for b in range(B):
        kn[b, :, lens[b]:] = np.nan
        vn[b, :, lens[b]:] = np.nan
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, kn, vn))
    out = tq.flash_attention(tk, tv, D ** -0.5, kv_lens=fa.IntTensor(device, lens)).to_numpy()
    tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16)
    for b in range(B):
        n = int(lens[b])
        ref = oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                     rounded(v[b:b + 1, :, :n], dtype), D ** -0.5)
        assert_parity(out[b:b + 1], ref, tol, f"D{D} Sq{Sq}, sequence {b} of length {n}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16, fa.F32])
@pytest.mark.parametrize("D", [64, 80, 128, 160, 256])
@pytest.mark.parametrize("Sq", [1, 4, 40, 200])
def test_rows_behind_the_last_query_position_are_never_used(device, dtype, D, Sq):
    """The view is the whole cache allocation (700 rows), the new rows stand at positions 300 ... inside it (a causal
    descriptor with q_pos_offset + Sq below the view's length) and the rows behind them hold NaN: causality hides them,
    and no kernel may fetch them into a tile either."""
    B, H, Hkv, Skv, pos = 2, 4, 2, 700, 300
    rng = np.random.default_rng(14)
    q = rng.normal(0, 1, (B, H, Sq, D)).astype(np.float32)
    k = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    v = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    kn, vn = k.copy(), v.copy()
    kn[:, :, pos + Sq:] = np.nan
    vn[:, :, pos + Sq:] = np.nan
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, kn, vn))
    for window in (0, 100):
        out = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, pos, window)).to_numpy()
        n = pos + Sq
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k[:, :, :n], dtype), rounded(v[:, :, :n], dtype), D ** -0.5,
                                     _analytic_mask(Sq, n, True, pos, window), "qk")
        tol = TOL_F32 if dtype == fa.F32 else (dict(max_abs=2e-2, rel_l2=1e-2) if dtype == fa.BF16 else TOL_16)
        assert_parity(out, ref, tol, f"D{D} Sq{Sq} window {window}")


@pytest.mark.parametrize("dtype,tol", [(fa.F16, 2e-3), (fa.BF16, 8e-3)])
@pytest.mark.parametrize("D", [160, 256])
@pytest.mark.parametrize("growth", [0.02, 0.3, 3.0, 40.0])
def test_wide_head_prefill_when_the_row_maximum_keeps_rising(device, dtype, tol, D, growth):
    """The wide-head kernel moves a column's reference maximum (and rescales its accumulators) only when a tile
    exceeds it by more than 2^8.  Scores that climb along the keys by `growth` per 32-key tile on top of unit noise
    walk through every regime: never again after the first tile, once in many tiles, every tile, and every tile by
    far more than the slack (softmax rows close to one-hot on the last visible key)."""
    B, H, Hkv, Sq, Skv = 1, 4, 2, 200, 1100
    rng = np.random.default_rng(5)
    q = rng.normal(0, 1, (B, H, Sq, D)).astype(np.float32)
    k = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    v = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    # dim 0 of every query is sqrt(D), dim 0 of key j is growth * j / 32: the scaled score gains growth per tile
    q[..., 0] = D ** 0.5
    k[..., 0] = (growth / 32.0) * np.arange(Skv, dtype=np.float32)[None, None, :]
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    for analytic in ((True, Skv - Sq, 0), (True, Skv - Sq, 300), None):
        kw = {} if analytic is None else {"analytic": analytic}
        assert tq.selected_kernel(tk, tv, D ** -0.5, **kw) == fa.KERNEL_PREFILL_MFMA
        out = tq.flash_attention(tk, tv, D ** -0.5, out_dtype=fa.F32, **kw).to_numpy()
        mask = None if analytic is None else _analytic_mask(Sq, Skv, *analytic)
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask,
                                     None if mask is None else "qk")
        assert np.isfinite(out).all()
        rl = rel_l2(out, ref)
        assert rl <= tol, f"rel-L2 {rl:.2e} at growth {growth}, D{D}, mask {analytic}"


@pytest.mark.parametrize("dtype,std,rel_gate,abs_gate", [(fa.BF16, 8.0, 8e-3, None), (fa.BF16, 30.0, 8e-3, None),
                                                        (fa.F16, 3.0, 1e-3, 2e-3), (fa.F16, 8.0, 1e-3, 2e-3), (fa.F16, 30.0, 1e-3, 2e-3)])
@pytest.mark.parametrize("D,Sq,Skv", [(128, 300, 300), (64, 200, 1500), (96, 260, 260)])
def test_tiled_16bit_prefill_at_large_score_magnitudes(device, dtype, std, rel_gate, abs_gate, D, Sq, Skv):
    """Queries and keys far wider than the unit-variance benchmark tensors: scaled scores of standard deviation std^2
    (9 ... 900), softmax rows close to one-hot.  The kernel multiplies Q by the power-of-two part of scale * log2(e)
    only (exact) and the scores by the rest in f32, as the reference multiplies the f32 dot product by the scale, so
    the error does not grow with the scores: f16 stays inside the gate of the benchmark configurations (rel-L2 1e-3,
    max-abs 2e-3 on the f32 output) at every magnitude.  Values are unit-variance in the gated run, so that the absolute
    gate means what it means for the benchmark tensors; a second run with values as wide as the keys checks rel-L2.
    bf16 is an extension over the reference's types and is held to 8e-3."""
    B, H, Hkv = 1, 4, 2
    rng = np.random.default_rng(77)
    q = rng.normal(0, std, (B, H, Sq, D)).astype(np.float32)
    k = rng.normal(0, std, (B, Hkv, Skv, D)).astype(np.float32)
    v1 = rng.normal(0, 1.0, (B, Hkv, Skv, D)).astype(np.float32)
    analytic = (True, Skv - Sq, 0)
    mask = _analytic_mask(Sq, Skv, True, Skv - Sq, 0)
    for v in (v1, v1 * np.float32(std)):
        tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
        assert tq.selected_kernel(tk, tv, D ** -0.5, analytic=analytic) == fa.KERNEL_PREFILL_MFMA
        out = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic, out_dtype=fa.F32).to_numpy()
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask, "qk")
        assert np.isfinite(out).all()
        rl = rel_l2(out, ref)
        assert rl <= rel_gate, f"rel-L2 {rl:.2e} at std {std}, D{D}"
        if abs_gate is not None and v is v1:
            err = float(np.abs(out - ref).max())
            assert err <= abs_gate, f"max-abs {err:.2e} at std {std}, D{D}"
