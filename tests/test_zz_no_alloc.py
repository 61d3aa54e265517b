"""GPU test of fhip_flash_attention_noalloc: the attention call on the library's own fixed workspace.

Every case runs the new entry point and the existing one (fhip_flash_attention with a workspace the caller
allocated) through the C ABI on the same tensors and compares the outputs bit for bit, twice in a row, the second
time with a smaller input, so that what the first call left in the shared array is still there.  The existing entry
point's result is itself held to the parity gate against the CPU checker.
"""
import ctypes

import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, TOL_F32, assert_parity
from test_attention_gpu import NEG_INF, _analytic_mask, _normal_qkv, rounded

pytestmark = pytest.mark.gpu


def _both(device, dtype, q, k, v, scale, mask=None, kind=None, analytic=None, expect_kernel=None, what=""):
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    mt = None
    if mask is not None:
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask if kind == "qk" else fa.MaskKind.BatchKeyMask)
    # the existing entry point, workspace allocated by the caller
    args = tq._attn_args(tk, tv, scale, mt, analytic, None, None, fa.KERNEL_AUTO, None)
    need = ctypes.c_size_t()
    fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
    assert 0 < need.value <= fa.NOALLOC_WORKSPACE_BYTES, f"{what}: the case must use a workspace ({need.value} bytes)"
    ws = fa.Buffer(device, need.value)
    args.workspace, args.workspace_bytes = ws.ptr, need.value
    if expect_kernel is not None:
        kid = ctypes.c_int32()
        fa.check(fa.lib().fhip_flash_attention_select(ctypes.byref(args), ctypes.byref(kid)))
        assert kid.value == expect_kernel, f"{what}: kernel {kid.value}"
    fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    want = args._out_tensor.to_numpy()
    # the new one: no workspace in the arguments, output pre-filled so that a call that does nothing is seen
    out = fa.Tensor.from_numpy(device, np.full(q.shape, 7.0, np.float32), dtype)
    args2 = tq._attn_args(tk, tv, scale, mt, analytic, None, None, fa.KERNEL_AUTO, out)
    assert not args2.workspace and args2.workspace_bytes == 0
    fa.check(fa.lib().fhip_flash_attention_noalloc(device.stream, ctypes.byref(args2)))
    got = out.to_numpy()
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), f"{what}: differs from fhip_flash_attention"
    if analytic is not None:
        mask, kind = _analytic_mask(q.shape[2], k.shape[2], *analytic), "qk"
    amask = None if mask is None else rounded(mask, dtype)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale, amask, kind)
    assert_parity(want, ref, TOL_F32 if dtype == fa.F32 else TOL_16, what)


def test_noalloc_decode_split_kv_two_calls_in_a_row(device):
    """Split-KV decode parks (acc, m, l) per split in the workspace; the second call has fewer rows and fewer splits."""
    D = 128
    for seed, (B, H, Hkv, Skv) in enumerate([(4, 8, 2, 4096), (2, 8, 2, 1000)]):
        q, k, v = _normal_qkv(300 + seed, B, H, Hkv, 1, Skv, D, 0.5)
        _both(device, fa.F16, q, k, v, D ** -0.5, expect_kernel=fa.KERNEL_DECODE_SPLITKV, what=f"decode B{B} Skv{Skv}")


def test_noalloc_prefill_with_a_mask_tensor_two_calls_in_a_row(device):
    """A mask tensor is reduced to intervals in the workspace (rows and the not-an-interval mark); the second call is
    shorter, and its mask is NOT made of intervals, so the mark left by nobody must not be mistaken for this call's."""
    D = 64
    q, k, v = _normal_qkv(310, 1, 4, 2, 300, 300, D)
    _both(device, fa.F16, q, k, v, D ** -0.5, oracle.get_mask(300, 0), "qk", expect_kernel=fa.KERNEL_PREFILL_MFMA,
          what="prefill causal mask tensor 300")
    q, k, v = _normal_qkv(311, 1, 4, 2, 100, 100, D)
    bias = np.random.default_rng(5).normal(0, 1, (100, 100)).astype(np.float32)
    bias[:, 40:60] = NEG_INF
    _both(device, fa.F16, q, k, v, D ** -0.5, bias, "qk", what="prefill bias tensor 100")
    q, k, v = _normal_qkv(312, 1, 4, 2, 64, 64, D)
    _both(device, fa.F16, q, k, v, D ** -0.5, oracle.get_mask(64, 0), "qk", what="prefill causal mask tensor 64")


def test_noalloc_few_rows_on_a_long_cache_two_calls_in_a_row(device):
    """The tiled f32 prefill kernel parks one partial row per key share in the workspace and a second kernel merges
    them; then the same with fewer rows and keys."""
    D = 64
    for seed, (Sq, Skv) in enumerate([(100, 5000), (40, 2100)]):
        q, k, v = _normal_qkv(320 + seed, 1, 4, 2, Sq, Skv, D)
        _both(device, fa.F32, q, k, v, D ** -0.5, analytic=(True, Skv - Sq, 0), expect_kernel=fa.KERNEL_PREFILL_F32,
              what=f"key shares {Sq} rows on {Skv} keys")


def test_noalloc_prefill_whose_planned_key_split_exceeds_the_array_still_runs(device):
    """A chat turn of 256 new rows on a 16384-key cache (f16, 32/8 heads, head_dim 128) plans 66 MiB of partial rows,
    twice the array.  Those are optional: the call takes the largest key split that fits, bit for bit what
    fhip_flash_attention does with a workspace of the array's size, and close to the unsplit call (workspace NULL);
    then a smaller call whose split fits."""
    D, H, Hkv = 128, 32, 8
    for seed, (Sq, Skv, beyond) in enumerate([(256, 16384, True), (64, 4096, False)]):
        q, k, v = _normal_qkv(330 + seed, 1, H, Hkv, Sq, Skv, D)
        tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
        analytic = (True, Skv - Sq, 0)
        args = tq._attn_args(tk, tv, D ** -0.5, None, analytic, None, None, fa.KERNEL_AUTO, None)
        need = ctypes.c_size_t()
        fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
        assert (need.value > fa.NOALLOC_WORKSPACE_BYTES) == beyond, need.value
        fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))  # workspace NULL: unsplit
        unsplit = args._out_tensor.to_numpy()
        ws = fa.Buffer(device, fa.NOALLOC_WORKSPACE_BYTES)
        args.workspace, args.workspace_bytes = ws.ptr, fa.NOALLOC_WORKSPACE_BYTES
        fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
        want = args._out_tensor.to_numpy()
        out = fa.Tensor.from_numpy(device, np.full(q.shape, 7.0, np.float32), fa.F16)
        args2 = tq._attn_args(tk, tv, D ** -0.5, None, analytic, None, None, fa.KERNEL_AUTO, out)
        fa.check(fa.lib().fhip_flash_attention_noalloc(device.stream, ctypes.byref(args2)))
        got = out.to_numpy()
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), f"{Sq} rows on {Skv}: differs from fhip_flash_attention"
        assert not np.array_equal(got.view(np.uint8), unsplit.view(np.uint8)), "the keys were not split at all"
        # the CPU checker on the first KV head's group of query heads
        G = H // Hkv
        ref = oracle.flash_attention(rounded(q[:, :G], fa.F16), rounded(k[:, :1], fa.F16), rounded(v[:, :1], fa.F16), D ** -0.5,
                                     _analytic_mask(Sq, Skv, *analytic), "qk")
        assert_parity(got[:, :G], ref, TOL_16, f"{Sq} rows on {Skv} keys, largest split that fits")
        assert_parity(unsplit[:, :G], ref, TOL_16, f"{Sq} rows on {Skv} keys, unsplit")


def test_noalloc_rejects_a_call_beyond_its_workspace(device):
    """64 x 64 rows over 65536 keys would park 136 MB of partial results: refused, nothing runs, the output is
    untouched.  (K and V are stride-0 views of a single row: the shape is large, the memory is not.)"""
    B, H, Hkv, Skv, D = 64, 64, 64, 65536, 128
    tq = fa.Tensor.from_numpy(device, np.zeros((B, H, 1, D), np.float32), fa.F16)
    row = fa.Tensor.from_numpy(device, np.zeros((1, 1, 1, D), np.float32), fa.F16)
    tk = fa.Tensor(row.buffer, fa.F16, (B, Hkv, Skv, D), (0, 0, 0, 1))
    out = fa.Tensor.from_numpy(device, np.full((B, H, 1, D), 7.0, np.float32), fa.F16)
    args = tq._attn_args(tk, tk, 0.1, None, None, None, None, fa.KERNEL_AUTO, out)
    need = ctypes.c_size_t()
    fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
    assert need.value > fa.NOALLOC_WORKSPACE_BYTES
    rc = fa.lib().fhip_flash_attention_noalloc(device.stream, ctypes.byref(args))
    assert rc == fa.ERR_WORKSPACE
    msg = fa.lib().fhip_last_error().decode()
    assert str(need.value) in msg and str(fa.NOALLOC_WORKSPACE_BYTES) in msg, msg
    assert (out.to_numpy() == 7.0).all()
