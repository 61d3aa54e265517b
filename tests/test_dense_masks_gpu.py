"""GPU tests of dense mask tensors on the tiled prefill kernels.

fusor passes its masks as tensors (MaskCache::get_mask, fusor-ml/fusor/src/cache/mask_cache.rs:36-116;
the padding masks of the BatchKeyMask kind, fusor flash_attention.rs:161-176).  The library reduces
such a tensor to one visible interval per row on the device and runs the tiled kernel when every
row has that form, the general kernel otherwise.  Both outcomes are checked against the CPU checker,
and the interval outcome is checked to be the tiled kernel by bit-equality with the analytic call.
"""
import ctypes

import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, TOL_F32, assert_parity
from test_attention_gpu import _normal_qkv, rounded

pytestmark = pytest.mark.gpu

NEG_INF = float("-inf")
TOL_BF16 = dict(max_abs=2e-2, rel_l2=1e-2)


def _tol(dtype):
    return TOL_F32 if dtype == fa.F32 else (TOL_BF16 if dtype == fa.BF16 else TOL_16)


def _tensors(device, dtype, *arrays):
    return [fa.Tensor.from_numpy(device, a, dtype) for a in arrays]


@pytest.mark.parametrize("dtype,D", [(fa.F16, 128), (fa.F16, 64), (fa.BF16, 96), (fa.F32, 64), (fa.F32, 128)])
@pytest.mark.parametrize("seq,offset,window", [(257, 0, None), (130, 270, None), (300, 0, 100), (96, 500, 200),
                                               (64, 1000, 64)])
def test_get_mask_tensor_runs_the_tiled_kernel(device, dtype, D, seq, offset, window):
    """The tensors MaskCache::get_mask builds give bit for bit what the analytic description gives."""
    mask = oracle.get_mask(seq, offset, window)
    Skv = mask.shape[1]
    q, k, v = _normal_qkv(21, 2, 4, 2, seq, Skv, D)
    tq, tk, tv, tm = _tensors(device, dtype, q, k, v, mask)
    scale = D ** -0.5
    out = tq.flash_attention(tk, tv, scale, (tm, fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale, mask, "qk")
    assert_parity(out, ref, _tol(dtype), f"dense get_mask({seq},{offset},{window}) D{D}")
    analytic = (True, Skv - seq, window or 0)  # what get_mask builds: causal after Skv - seq cached keys, plus the window
    out_a = tq.flash_attention(tk, tv, scale, analytic=analytic).to_numpy()
    assert np.array_equal(out.view(np.uint8), out_a.view(np.uint8)), "dense interval mask did not take the tiled kernel"


@pytest.mark.parametrize("dtype,D", [(fa.F16, 128), (fa.F32, 64)])
def test_padding_batch_key_mask(device, dtype, D):
    """Left and right padding per sequence (BatchKeyMask): the tiled kernel with a key range per batch."""
    B, H, Hkv, Sq, Skv = 3, 4, 2, 130, 333
    q, k, v = _normal_qkv(22, B, H, Hkv, Sq, Skv, D)
    mask = np.zeros((B, Skv), np.float32)
    mask[0, 300:] = NEG_INF          # right padding
    mask[1, :77] = NEG_INF           # left padding
    mask[2, :5] = NEG_INF
    mask[2, 200:] = NEG_INF          # both
    tq, tk, tv, tm = _tensors(device, dtype, q, k, v, mask)
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.BatchKeyMask)).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask, "batch_key")
    assert_parity(out, ref, _tol(dtype), "padding mask")
    # the same call, sequence by sequence on the un-padded keys (tiled kernel, no mask at all)
    for b, (lo, hi) in enumerate([(0, 300), (77, Skv), (5, 200)]):
        tqb, tkb, tvb = _tensors(device, dtype, q[b:b + 1], k[b:b + 1, :, lo:hi], v[b:b + 1, :, lo:hi])
        out_b = tqb.flash_attention(tkb, tvb, D ** -0.5).to_numpy()
        assert_parity(out[b:b + 1], out_b, dict(max_abs=1e-6 if dtype == fa.F32 else 2e-3, rel_l2=1e-5 if dtype == fa.F32 else 1e-3),
                      f"un-padded sequence {b}")


@pytest.mark.parametrize("dtype,D", [(fa.F32, 64), (fa.F32, 128), (fa.F16, 128)])
def test_block_diagonal_mask_of_the_vision_blocks(device, dtype, D):
    """Qwen-VL's vision blocks mask with a block-diagonal [S, S] tensor built from cu_seqlens
    (models/kalosm-llama/src/raw/vision/qwen_vision_block.rs:211-226): every row sees one contiguous run of
    keys, so the interval form applies and the tiled kernel runs; the result equals running each block alone."""
    cu_seqlens = [0, 70, 71, 300, 513]
    S = cu_seqlens[-1]
    mask = np.full((S, S), NEG_INF, np.float32)
    for last, nxt in zip(cu_seqlens[:-1], cu_seqlens[1:]):
        mask[last:nxt, last:nxt] = 0.0
    q, k, v = _normal_qkv(27, 1, 4, 4, S, S, D)
    tq, tk, tv, tm = _tensors(device, dtype, q, k, v, mask)
    want = fa.KERNEL_PREFILL_F32 if dtype == fa.F32 else fa.KERNEL_PREFILL_MFMA
    ws, ws_bytes = device.workspace(1 << 20)
    out_t = fa.Tensor.empty(device, (1, 4, S, D), dtype)
    args = tq._attn_args(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask), None, None, None, fa.KERNEL_AUTO, out_t)
    args.workspace, args.workspace_bytes = ws, ws_bytes
    kid = ctypes.c_int32()
    fa.check(fa.lib().fhip_flash_attention_select(ctypes.byref(args), ctypes.byref(kid)))
    assert kid.value == want
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask, "qk")
    assert_parity(out, ref, _tol(dtype), "block-diagonal mask")
    for last, nxt in zip(cu_seqlens[:-1], cu_seqlens[1:]):
        tqb, tkb, tvb = _tensors(device, dtype, q[:, :, last:nxt], k[:, :, last:nxt], v[:, :, last:nxt])
        alone = tqb.flash_attention(tkb, tvb, D ** -0.5).to_numpy()
        assert_parity(out[:, :, last:nxt], alone, dict(max_abs=2e-6 if dtype == fa.F32 else 2e-3, rel_l2=1e-5 if dtype == fa.F32 else 1e-3),
                      f"block {last}:{nxt} alone")


@pytest.mark.parametrize("dtype,D", [(fa.F16, 128), (fa.BF16, 64), (fa.F32, 64)])
@pytest.mark.parametrize("shape", ["bias", "two_runs", "nan", "positive_inf"])
def test_masks_that_are_not_intervals_fall_back(device, dtype, D, shape):
    """Finite biases, several visible runs, NaN or +inf entries: the mask values are added as the reference adds
    them (fusor flash_attention.rs:161-176), by the mask-adding form of the f32-arithmetic tiled kernel (which widens
    16-bit rows on load)."""
    B, H, Hkv, Sq, Skv = 1, 2, 1, 140, 200
    q, k, v = _normal_qkv(23, B, H, Hkv, Sq, Skv, D)
    rng = np.random.default_rng(5)
    mask = np.zeros((Sq, Skv), np.float32)
    if shape == "bias":
        mask = rng.normal(0, 1, (Sq, Skv)).astype(np.float32)
        mask[:, 150:] = NEG_INF
    elif shape == "two_runs":
        mask[:, 40:60] = NEG_INF
        mask[7, :] = 0.0
    elif shape == "nan":
        mask[:, 100:] = NEG_INF
        mask[3, 5] = np.nan
    else:
        mask[:, 100:] = NEG_INF
        mask[9, 120] = np.inf
    tq, tk, tv, tm = _tensors(device, dtype, q, k, v, mask)
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                 rounded(mask, dtype), "qk")
    bad_rows = {"nan": [3], "positive_inf": [9]}.get(shape, [])
    keep = [r for r in range(Sq) if r not in bad_rows]
    assert_parity(out[:, :, keep], ref[:, :, keep], _tol(dtype), f"fallback {shape}")
    for r in bad_rows:
        assert np.isnan(out[0, :, r]).all() and np.isnan(ref[0, :, r]).all()


@pytest.mark.parametrize("Skv", [90, 330])
def test_rows_without_visible_keys_and_negative_zero(device, Skv):
    """Empty rows give NaN like the reference; -0.0 counts as zero; a one-key row works.  (330 keys: the workgroup
    form whose two wavefront groups merge their halves of the keys, some rows seeing keys in one half only.)"""
    D, Sq = 128, 70
    q, k, v = _normal_qkv(24, 1, 2, 2, Sq, Skv, D)
    mask = np.full((Sq, Skv), NEG_INF, np.float32)
    for r in range(Sq):
        if r % 7 == 3:
            continue                      # nothing visible
        lo = (r * 37) % (Skv - 75)
        mask[r, lo:lo + 1 + r] = -0.0 if r % 2 else 0.0
    tq, tk, tv, tm = _tensors(device, fa.F16, q, k, v, mask)
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(rounded(q, fa.F16), rounded(k, fa.F16), rounded(v, fa.F16), D ** -0.5, mask, "qk")
    empty = [r for r in range(Sq) if r % 7 == 3]
    keep = [r for r in range(Sq) if r % 7 != 3]
    assert np.isnan(out[:, :, empty]).all() and np.isnan(ref[:, :, empty]).all()
    assert_parity(out[:, :, keep], ref[:, :, keep], TOL_16, "interval rows")


def test_strided_and_broadcast_mask_views(device):
    """A mask that is a transposed view, and one with a zero row stride, go through the scan as well."""
    D, S = 64, 150
    q, k, v = _normal_qkv(25, 1, 2, 1, S, S, D)
    causal = oracle.get_mask(S, 0)
    tq, tk, tv = _tensors(device, fa.F16, q, k, v)
    # the transpose of the anti-causal mask is the causal mask
    t_anti = fa.Tensor.from_numpy(device, np.ascontiguousarray(causal.T), fa.F16).transpose(0, 1)
    out = tq.flash_attention(tk, tv, D ** -0.5, (t_anti, fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(rounded(q, fa.F16), rounded(k, fa.F16), rounded(v, fa.F16), D ** -0.5, causal, "qk")
    assert_parity(out, ref, TOL_16, "transposed mask view")


def test_without_workspace_the_mask_is_added_element_by_element(device):
    """The C ABI never allocates: a masked call that brings no scratch is served by the f32-arithmetic tiled kernel,
    which adds the mask as it is (16-bit rows are widened on load)."""
    D, S = 64, 100
    q, k, v = _normal_qkv(26, 1, 2, 1, S, S, D)
    mask = oracle.get_mask(S, 0)
    tq, tk, tv, tm = _tensors(device, fa.F16, q, k, v, mask)
    assert tq.selected_kernel(tk, tv, 0.1, (tm, fa.MaskKind.QKMask)) == fa.KERNEL_PREFILL_F32
    out_t = fa.Tensor.empty(device, (1, 2, S, D), fa.F16)
    args = tq._attn_args(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask), None, None, None, fa.KERNEL_AUTO, out_t)
    fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    ref = oracle.flash_attention(rounded(q, fa.F16), rounded(k, fa.F16), rounded(v, fa.F16), D ** -0.5, mask, "qk")
    assert_parity(out_t.to_numpy(), ref, TOL_16, "no workspace")



@pytest.mark.parametrize("D,B,H,S", [(64, 3, 4, 200), (128, 2, 4, 333), (64, 8, 12, 512), (96, 1, 2, 100)])
@pytest.mark.parametrize("workspace", [True, False])
def test_padding_mask_with_a_large_finite_value(device, D, B, H, S, workspace):
    """rbert masks padded keys with -10000.0 instead of -inf (models/rbert/src/raw/qwen/attention.rs:91-113,
    BatchKeyMask, f32).  That is a finite bias, so no interval form exists; the f32 tiled kernel adds it element by
    element, with or without scratch memory."""
    q, k, v = _normal_qkv(28, B, H, H, S, S, D)
    mask = np.zeros((B, S), np.float32)
    for b in range(B):
        mask[b, S - 1 - 13 * b:] = -10000.0
    tq, tk, tv, tm = _tensors(device, fa.F32, q, k, v, mask)
    out_t = fa.Tensor.empty(device, (B, H, S, D), fa.F32)
    args = tq._attn_args(tk, tv, D ** -0.5, (tm, fa.MaskKind.BatchKeyMask), None, None, None, fa.KERNEL_AUTO, out_t)
    if workspace:
        need = ctypes.c_size_t()
        fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
        ws, ws_bytes = device.workspace(max(need.value, 16))
        args.workspace, args.workspace_bytes = ws, ws_bytes
    kid = ctypes.c_int32()
    fa.check(fa.lib().fhip_flash_attention_select(ctypes.byref(args), ctypes.byref(kid)))
    assert kid.value == fa.KERNEL_PREFILL_F32
    fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, "batch_key")
    assert_parity(out_t.to_numpy(), ref, TOL_F32, "-10000 padding mask")


@pytest.mark.parametrize("D,S", [(64, 150), (128, 300), (32, 77)])
def test_additive_bias_matrix_on_the_f32_tiled_kernel(device, D, S):
    """A [Sq, Skv] tensor of finite biases (with a masked band and one fully masked row) through the tiled kernel."""
    q, k, v = _normal_qkv(29, 2, 4, 2, S, S + 40, D)
    rng = np.random.default_rng(8)
    mask = rng.normal(0, 2, (S, S + 40)).astype(np.float32)
    mask[:, 20:50] = NEG_INF
    mask[5, :] = NEG_INF
    tq, tk, tv, tm = _tensors(device, fa.F32, q, k, v, mask)
    assert tq.selected_kernel(tk, tv, 0.1, (tm, fa.MaskKind.QKMask)) == fa.KERNEL_PREFILL_F32
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, "qk")
    keep = [r for r in range(S) if r != 5]
    assert np.isnan(out[:, :, 5]).all() and np.isnan(ref[:, :, 5]).all()
    assert_parity(out[:, :, keep], ref[:, :, keep], TOL_F32, "bias matrix")


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16, fa.BF16])
def test_masks_built_on_the_device_equal_the_host_builders(device, dtype):
    """fhip_mask_get_mask_device writes, bit for bit, what MaskCache::get_mask builds on the host
    (mask_cache.rs:36-116), for the reference's own cases (mask_cache.rs:120-175) and a sweep."""
    cases = [(3, 0, None), (4, 0, 2), (2, 3, None), (1, 4095, None), (5, 2, 3), (5, 2, 9), (7, 100, 4), (64, 1000, 64),
             (130, 270, None), (300, 0, 100), (1, 0, 1), (9, 5, 0)]
    mc = fa.MaskCache(dtype)
    for seq, off, w in cases:
        on_dev = mc.get_mask_on_device(seq, off, w, device).mask().to_numpy()
        host = oracle.get_mask(seq, off, w)
        assert on_dev.shape == host.shape, (seq, off, w)
        want = fa.Tensor.from_numpy(device, host, dtype).to_numpy()
        assert np.array_equal(on_dev.view(np.uint8), want.view(np.uint8)), (seq, off, w)


# ---- head_dim <= 64: the f32 tiled kernel holds both mask forms ---------------------------------------------------
# Two launches (the scan, the tiled kernel) and no hand-over kernel: the tiled kernel reads what the scan found and
# masks by interval (bit for bit the analytic call) or adds the mask values, also in its key-split forms.

def _qk_call(device, dtype, q, k, v, mask, **kw):
    tq, tk, tv, tm = _tensors(device, dtype, q, k, v, mask)
    return tq, tk, tv, tq.flash_attention(tk, tv, q.shape[-1] ** -0.5, (tm, fa.MaskKind.QKMask), **kw).to_numpy()


@pytest.mark.parametrize("dtype,D", [(fa.F32, 64), (fa.F32, 32), (fa.F32, 48), (fa.F16, 40), (fa.BF16, 16)])
@pytest.mark.parametrize("seq,offset,window", [(512, 0, None), (40, 0, None), (200, 312, None), (96, 160, 64), (304, 0, 7),
                                               (64, 960, None), (33, 95, None)])
def test_mask_tensors_made_of_intervals_on_the_two_form_kernel(device, dtype, D, seq, offset, window):
    mask = oracle.get_mask(seq, offset, window)
    Skv = mask.shape[1]
    q, k, v = _normal_qkv(61, 2, 4, 2, seq, Skv, D)
    tq, tk, tv, out = _qk_call(device, dtype, q, k, v, mask)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask, "qk")
    assert_parity(out, ref, _tol(dtype), f"get_mask({seq},{offset},{window}) D{D}")
    out_a = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, Skv - seq, window or 0)).to_numpy()
    assert np.array_equal(out.view(np.uint8), out_a.view(np.uint8)), "the interval form was not taken"


@pytest.mark.parametrize("dtype,D", [(fa.F32, 64), (fa.F32, 32), (fa.F16, 40)])
@pytest.mark.parametrize("kind", ["bias", "two_runs", "bias_in_some_blocks", "empty_rows", "plus_inf", "block_diagonal"])
def test_masks_that_are_not_intervals_on_the_two_form_kernel(device, dtype, D, kind):
    B, H, Hkv, Sq, Skv = 2, 4, 2, 200, 328
    rng = np.random.default_rng(9)
    q, k, v = _normal_qkv(62, B, H, Hkv, Sq, Skv, D)
    mask = oracle.get_mask(Sq, Skv - Sq, None).copy()
    if kind == "bias":
        mask = np.where(np.isneginf(mask), mask, rng.normal(0, 1, mask.shape)).astype(np.float32)
    elif kind == "two_runs":
        mask[:, 40:50] = NEG_INF      # a hole in every row that reaches it
    elif kind == "bias_in_some_blocks":
        mask[70:75, 3] = -2.5         # a few finite entries: the whole call adds values
        mask[199, 0] = 0.75
    elif kind == "empty_rows":
        mask[5, :] = NEG_INF          # rows without a visible key: NaN on both sides
        mask[130, :] = NEG_INF
    elif kind == "plus_inf":
        mask[9, 2] = np.inf
    elif kind == "block_diagonal":
        mask[:] = NEG_INF
        for lo, hi in ((0, 60), (60, 61), (61, 200)):
            mask[lo:hi, lo:hi + 100] = 0
    tq, tk, tv, out = _qk_call(device, dtype, q, k, v, mask)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, rounded(mask, dtype), "qk")
    dead = np.isnan(ref).any(-1)
    assert np.array_equal(np.isnan(out).any(-1), dead), "rows without a usable value differ"
    if (~dead).any():
        assert_parity(out[~dead], ref[~dead], _tol(dtype), kind)


@pytest.mark.parametrize("fill", [NEG_INF, -10000.0])
def test_padding_masks_on_the_two_form_kernel(device, fill):
    """A BatchKeyMask row per batch: -inf padding is an interval, rbert's -10000.0 is added as it is."""
    B, H, Hkv, Sq, Skv, D = 3, 4, 4, 150, 256, 64
    q, k, v = _normal_qkv(63, B, H, Hkv, Sq, Skv, D)
    mask = np.zeros((B, Skv), np.float32)
    mask[0, 200:] = fill
    mask[1, :31] = fill
    tq, tk, tv, tm = _tensors(device, fa.F32, q, k, v, mask)
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.BatchKeyMask)).to_numpy()
    ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, "batch_key")
    assert_parity(out, ref, TOL_F32, f"padding with {fill}")


def test_strided_mask_views_on_the_two_form_kernel(device):
    """Mask rows that are not contiguous or not 16-byte aligned."""
    B, H, Hkv, Sq, Skv, D = 1, 4, 2, 100, 200, 64
    q, k, v = _normal_qkv(64, B, H, Hkv, Sq, Skv, D)
    mask = oracle.get_mask(Sq, Skv - Sq, None)
    wide = np.zeros((Sq, Skv + 3), np.float32)
    wide[:, 1:Skv + 1] = mask
    tq, tk, tv = _tensors(device, fa.F32, q, k, v)
    tm = fa.Tensor.from_numpy(device, wide, fa.F32).narrow(1, 1, Skv)       # rows start 4 bytes off a 16-byte boundary
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask)).to_numpy()
    ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, "qk")
    assert_parity(out, ref, TOL_F32, "misaligned rows")
    tmt = fa.Tensor.from_numpy(device, np.ascontiguousarray(mask.T), fa.F32).transpose(0, 1)  # column-major mask
    out = tq.flash_attention(tk, tv, D ** -0.5, (tmt, fa.MaskKind.QKMask)).to_numpy()
    assert_parity(out, ref, TOL_F32, "transposed mask")


@pytest.mark.parametrize("dtype,D", [(fa.F32, 64), (fa.F32, 128), (fa.F16, 128), (fa.F16, 160), (fa.BF16, 96)])
@pytest.mark.parametrize("kind", ["get_mask", "window_after_cache", "bias", "batch_key", "empty_rows"])
def test_interval_table_computed_once_and_passed_with_the_mask(device, dtype, D, kind):
    """fhip_mask_intervals computes a mask tensor's interval form once; a call that carries the table skips its own scan
    and needs no workspace for the mask.  Every call with the table gives bit for bit what the call without it gives
    (interval masks on the tiled kernel, other masks added element by element), on repeated calls and in the no-alloc
    entry point, and stays inside the gate against the CPU checker."""
    B, H, Hkv, Sq = 2, 4, 2, 150
    mkind, okind = fa.MaskKind.QKMask, "qk"
    if kind == "get_mask":
        mask = oracle.get_mask(Sq, 0, None)
    elif kind == "window_after_cache":
        mask = oracle.get_mask(Sq, 400, 200)
    elif kind == "bias":
        mask = np.random.default_rng(9).normal(0, 1, (Sq, 260)).astype(np.float32)
        mask[:, 100:130] = NEG_INF
    elif kind == "batch_key":
        mask = np.zeros((B, 300), np.float32)
        mask[0, 250:] = NEG_INF
        mask[1, :40] = NEG_INF
        mkind, okind = fa.MaskKind.BatchKeyMask, "batch_key"
    else:
        mask = oracle.get_mask(Sq, 100, None)
        mask[7] = NEG_INF      # rows that see nothing give NaN with or without the table
        mask[149] = NEG_INF
    Skv = mask.shape[1]
    q, k, v = _normal_qkv(91, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv, tm = _tensors(device, dtype, q, k, v, mask)
    scale = D ** -0.5
    plain = tq.flash_attention(tk, tv, scale, (tm, mkind)).to_numpy()
    table = fa.MaskIntervals(tm)
    # the call needs no workspace for the mask any more (what is left, if anything, is for a key split)
    need, need_plain = ctypes.c_size_t(), ctypes.c_size_t()
    args = tq._attn_args(tk, tv, scale, (tm, mkind, table), None, None, None, fa.KERNEL_AUTO, None)
    fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
    args = tq._attn_args(tk, tv, scale, (tm, mkind), None, None, None, fa.KERNEL_AUTO, None)
    fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need_plain)))
    assert need.value + 16 + 8 * mask.shape[0] <= need_plain.value + 256
    # and is served by the type's own tiled kernel even when it brings no workspace at all
    assert tq.selected_kernel(tk, tv, scale, mask=(tm, mkind, table)) == (fa.KERNEL_PREFILL_F32 if dtype == fa.F32 else fa.KERNEL_PREFILL_MFMA)
    for rep in range(3):
        out = tq.flash_attention(tk, tv, scale, (tm, mkind, table)).to_numpy()
        assert np.array_equal(out.view(np.uint8), plain.view(np.uint8)), f"{kind} rep {rep}: differs from the call without the table"
    out_t = fa.Tensor.from_numpy(device, np.full(q.shape, 7.0, np.float32), dtype)
    tq.flash_attention_noalloc(tk, tv, scale, out_t, (tm, mkind, table))
    assert np.array_equal(out_t.to_numpy().view(np.uint8), plain.view(np.uint8)), f"{kind}: no-alloc entry point differs"
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale, rounded(mask, dtype), okind)
    if kind == "empty_rows":
        assert np.isnan(out[:, :, [7, 149]]).all() and np.isnan(ref[:, :, [7, 149]]).all()
        keep = np.setdiff1d(np.arange(Sq), [7, 149])
        out, ref = out[:, :, keep], ref[:, :, keep]
    assert_parity(out, ref, _tol(dtype), f"{kind} with the interval table")


def test_interval_table_arguments_are_checked(device):
    tm = fa.Tensor.from_numpy(device, oracle.get_mask(20, 0, None), fa.F32)
    need = ctypes.c_size_t()
    fa.check(fa.lib().fhip_mask_intervals_bytes(20, ctypes.byref(need)))
    assert need.value >= 16 + 20 * 8 and need.value % 16 == 0
    small = fa.Buffer(device, 64)
    cm = tm._c2()
    rc = fa.lib().fhip_mask_intervals(device.stream, ctypes.byref(cm), fa.F32, ctypes.c_void_p(small.ptr), 64)
    assert rc == fa.ERR_WORKSPACE and str(need.value) in fa.lib().fhip_last_error().decode()
    # a table without a mask tensor is refused
    q = fa.Tensor.from_numpy(device, np.zeros((1, 2, 20, 64), np.float32), fa.F32)
    args = q._attn_args(q, q, 0.1, None, None, None, None, fa.KERNEL_AUTO, None)
    args.mask_intervals = small.ptr
    assert fa.lib().fhip_flash_attention_validate(ctypes.byref(args)) == fa.ERR_INVALID_ARG
