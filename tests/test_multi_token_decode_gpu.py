"""Multi-token decode steps (a few new query rows on a cache) on the split-KV decode kernels.

The reference fuzzes exactly this shape (fusor-ml/core/src/composite/flash_attention.rs:807-921: q_seq_len 1..4,
kv_seq_len = q_seq_len + 0..31, a [q_seq_len, kv_seq_len] mask tensor); kalosm-llama reaches it when a turn feeds a
few tokens on top of a cached context, with MaskCache::get_mask(n, pos, window) as the mask
(models/kalosm-llama/src/raw/mod.rs:618-620).  The rows ride as further columns beside the query heads that share a
KV head, so the cache is still streamed once; every case asserts that the decode kernel is the one selected and
compares with the CPU checker.
"""
import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, TOL_F32, assert_parity
from test_attention_gpu import NEG_INF, _analytic_mask, _normal_qkv, _uniform, rounded

pytestmark = pytest.mark.gpu


def _tol(dtype):
    return TOL_F32 if dtype == fa.F32 else (dict(max_abs=1e-2, rel_l2=5e-3) if dtype == fa.BF16 else TOL_16)


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16])
def test_reference_kv_cache_fuzz_ranges_select_the_decode_kernel(device, dtype):
    """The reference's ranges, seeded: batch 1..2, heads 1..8, Sq 1..4, Skv = Sq + 0..31, head_dim 1..64, zero mask.
    Head dims that are a multiple of 8 run on the decode kernel (the others have no 16-byte rows and take the general
    kernel)."""
    rng = np.random.default_rng(0xF111)
    on_decode = 0
    for it in range(60):
        B, H, D = rng.integers(1, 3), rng.integers(1, 9), rng.integers(1, 65)
        if it % 2:
            D = 8 * rng.integers(1, 9)
        Sq = rng.integers(1, 5)
        Skv = Sq + rng.integers(0, 32)
        q = _uniform(rng, (B, H, Sq, D))
        k, v = _uniform(rng, (B, H, Skv, D)), _uniform(rng, (B, H, Skv, D))
        mask = np.zeros((Sq, Skv), np.float32)
        tq, tk, tv, tm = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v, mask))
        sel = tq.selected_kernel(tk, tv, 0.1, mask=(tm, fa.MaskKind.QKMask))
        if D % 8 == 0:
            assert sel == fa.KERNEL_DECODE_SPLITKV, f"it{it} Sq{Sq} D{D}: kernel {sel}"
            on_decode += 1
        out = tq.flash_attention(tk, tv, 1 / np.sqrt(np.float32(D)), (tm, fa.MaskKind.QKMask)).to_numpy()
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), 1 / np.sqrt(np.float32(D)),
                                     mask, "qk")
        assert_parity(out, ref, _tol(dtype), f"it{it} B{B} H{H} Sq{Sq} Skv{Skv} D{D}")
    assert on_decode >= 30


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16, fa.F32])
@pytest.mark.parametrize("G,D,Sq,Skv", [(4, 128, 4, 3000), (4, 128, 2, 700), (1, 96, 3, 777), (8, 64, 4, 1500), (2, 128, 4, 64),
                                        (3, 128, 3, 300), (16, 128, 2, 260), (4, 72, 4, 900), (2, 256, 2, 1500), (5, 32, 3, 5000),
                                        (4, 128, 4, 4)])
@pytest.mark.parametrize("case", ["causal", "window", "mask_tensor", "full"])
def test_multi_token_step(device, dtype, G, D, Sq, Skv, case):
    """New rows at the end of the cache: row r sits at position Skv - Sq + r and sees the keys up to its own
    (causal among the new rows), optionally through a sliding window; the same mask as a tensor; and no mask."""
    B, Hkv = 2, 2
    q, k, v = _normal_qkv(41, B, Hkv * G, Hkv, Sq, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    off = Skv - Sq
    window = max(3, Skv // 3)
    analytic, mask = {"causal": ((True, off, 0), _analytic_mask(Sq, Skv, True, off, 0)),
                      "window": ((True, off, window), _analytic_mask(Sq, Skv, True, off, window)),
                      "mask_tensor": (None, _analytic_mask(Sq, Skv, True, off, window)),
                      "full": (None, None)}[case]
    kw = {}
    if analytic:
        kw["analytic"] = analytic
    elif mask is not None:
        kw["mask"] = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    assert tq.selected_kernel(tk, tv, 0.1, **kw) == fa.KERNEL_DECODE_SPLITKV
    m = kw.pop("mask", None)
    out = tq.flash_attention(tk, tv, D ** -0.5, m, **kw).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask,
                                 None if mask is None else "qk")
    assert_parity(out, ref, _tol(dtype), f"{case} G{G} D{D} Sq{Sq} Skv{Skv}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("case", ["causal", "window", "full"])
def test_multi_token_step_of_a_batch_that_fills_the_chip(device, dtype, case):
    """More than 8 columns per KV head and enough (batch, KV head, 2048-key chunk) units for every compute unit: the step
    runs on the 8-wavefront form of the 16-bit kernel; the last chunk holds 4 keys."""
    B, Hkv, G, D, Sq, Skv = 11, 8, 4, 128, 3, 4100
    q, k, v = _normal_qkv(47, B, Hkv * G, Hkv, Sq, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    off = Skv - Sq
    analytic, mask = {"causal": ((True, off, 0), _analytic_mask(Sq, Skv, True, off, 0)),
                      "window": ((True, off, 2500), _analytic_mask(Sq, Skv, True, off, 2500)),
                      "full": (None, None)}[case]
    kw = {"analytic": analytic} if analytic else {}
    assert tq.selected_kernel(tk, tv, 0.1, **kw) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5, **kw).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask,
                                 None if mask is None else "qk")
    assert_parity(out, ref, _tol(dtype), f"{case}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.F32])
def test_multi_token_step_ragged_batch_and_padding_mask(device, dtype):
    """Per-sequence key counts and a BatchKeyMask on a multi-token step; the output written as [B, Sq, H, D]."""
    B, H, Hkv, D, Sq, Smax = 4, 8, 2, 128, 3, 2500
    lens = np.array([2500, 3, 1029, 640], np.int32)
    q, k, v = _normal_qkv(43, B, H, Hkv, Sq, Smax, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    out_buf = fa.Tensor.empty(device, (B, Sq, H, D), dtype)
    out = tq.flash_attention(tk, tv, D ** -0.5, kv_lens=fa.IntTensor(device, lens), out=out_buf.transpose(1, 2))
    assert tq.selected_kernel(tk, tv, 0.1, kv_lens=fa.IntTensor(device, lens)) == fa.KERNEL_DECODE_SPLITKV
    got = out_buf.to_numpy().transpose(0, 2, 1, 3)
    bk = np.where(np.arange(Smax)[None, :] < lens[:, None], 0.0, NEG_INF).astype(np.float32)
    got_m = tq.flash_attention(tk, tv, D ** -0.5, (fa.Tensor.from_numpy(device, bk, dtype), fa.MaskKind.BatchKeyMask)).to_numpy()
    for b in range(B):
        n = int(lens[b])
        ref = oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                     rounded(v[b:b + 1, :, :n], dtype), D ** -0.5)
        assert_parity(got[b:b + 1], ref, _tol(dtype), f"kv_lens b{b} len{n}")
        assert_parity(got_m[b:b + 1], ref, _tol(dtype), f"batch-key mask b{b} len{n}")
    del out


@pytest.mark.parametrize("dtype", [fa.F16, fa.F32, fa.BF16])
@pytest.mark.parametrize("Sq,off,window,D", [(1, 1000, 300, 128), (3, 1000, 300, 128), (4, 2995, 0, 64), (2, 140, 0, 128),
                                             (1, 2999, 129, 96), (8, 1500, 1400, 128), (1, 5, 3, 80)])
def test_decode_sees_only_a_stretch_of_the_cache(device, dtype, Sq, off, window, D):
    """The analytic descriptor leaves the start of the cache (a window) and / or its end (query positions in the middle
    of the cache) out: the split-KV plan and the kernels work on the visible stretch alone."""
    B, H, Hkv, Skv = 2, 8, 2, 3000
    q, k, v = _normal_qkv(49, B, H, Hkv, Sq, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    analytic = (True, off, window)
    assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                 _analytic_mask(Sq, Skv, True, off, window), "qk")
    assert_parity(out, ref, _tol(dtype), f"Sq{Sq} off{off} window{window} D{D}")


def test_rows_fully_masked_by_their_own_limits_are_nan(device):
    """A window so short and an offset so placed that some rows see no key: those rows are NaN (0/0) as in the
    reference, the others are right."""
    B, H, Hkv, D, Sq, Skv = 1, 4, 2, 64, 4, 40
    q, k, v = _normal_qkv(44, B, H, Hkv, Sq, Skv, D)
    mask = np.zeros((Sq, Skv), np.float32)
    mask[1, :] = NEG_INF
    mask[3, :] = NEG_INF
    tq, tk, tv, tm = (fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v, mask))
    assert tq.selected_kernel(tk, tv, 0.1, mask=(tm, fa.MaskKind.QKMask)) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask)).to_numpy()
    assert np.isnan(out[:, :, [1, 3]]).all()
    ref = oracle.flash_attention(q, k, v, D ** -0.5)
    assert_parity(out[:, :, [0, 2]], ref[:, :, [0, 2]], TOL_F32, "visible rows")


@pytest.mark.parametrize("dtype,G,Sq,D", [(fa.F16, 1, 16, 128), (fa.F32, 2, 8, 64), (fa.BF16, 1, 9, 96), (fa.F16, 4, 4, 128),
                                          (fa.F16, 4, 8, 128), (fa.F32, 4, 7, 128), (fa.BF16, 2, 16, 64), (fa.F16, 1, 32, 96),
                                          (fa.F32, 4, 8, 128), (fa.BF16, 4, 5, 128), (fa.F16, 8, 3, 32), (fa.F16, 1, 16, 256),
                                          (fa.F32, 2, 8, 192), (fa.F32, 1, 32, 32), (fa.F32, 4, 16, 128), (fa.F32, 1, 32, 192),
                                          (fa.F32, 4, 11, 64), (fa.F32, 4, 8, 256), (fa.F32, 4, 2, 256), (fa.F32, 1, 5, 224),
                                          (fa.F32, 8, 4, 256), (fa.F32, 1, 4, 256), (fa.F32, 2, 3, 224), (fa.F32, 4, 16, 192),
                                          (fa.F32, 4, 8, 160), (fa.F32, 2, 32, 192), (fa.F32, 4, 5, 192)])
def test_longer_drafts_while_rows_times_group_fit_one_workgroup(device, dtype, G, Sq, D):
    """More than 4 rows while rows x GQA group fit the columns one workgroup of a matrix-core variant takes: two blocks
    of 16 up to head_dim 128 (an 8-token draft on a 4-way GQA model, 32 tokens on an MHA model), one block above; f32
    tensors two blocks up to head_dim 192 and twice the columns, on two workgroups per KV head.  One row more, or a head_dim the matrix-core variants do not
    take, and the call is a prefill call again."""
    B, Hkv, Skv = 2, 2, 2100
    q, k, v = _normal_qkv(45, B, Hkv * G, Hkv, Sq, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    analytic = (True, Skv - Sq, 0)
    assert tq.selected_kernel(tk, tv, 0.1, analytic=analytic) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic).to_numpy()
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                 _analytic_mask(Sq, Skv, True, Skv - Sq, 0), "qk")
    assert_parity(out, ref, _tol(dtype), f"G{G} Sq{Sq} D{D}")
    # the same rows through a sliding window and as a mask tensor (one mask row per query row)
    w = 700
    mask = _analytic_mask(Sq, Skv, True, Skv - Sq, w)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask, "qk")
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, Skv - Sq, w)).to_numpy()
    assert_parity(out, ref, _tol(dtype), f"window, G{G} Sq{Sq} D{D}")
    tm = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    assert tq.selected_kernel(tk, tv, 0.1, tm) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5, tm).to_numpy()
    assert_parity(out, ref, _tol(dtype), f"window as a tensor, G{G} Sq{Sq} D{D}")
    if Sq * G == ((64 if D <= 192 else 32) if dtype == fa.F32 else (32 if D <= 128 else 16)):
        q2 = np.concatenate([q, q[:, :, :1]], 2)
        t2 = fa.Tensor.from_numpy(device, q2, dtype)
        assert t2.selected_kernel(tk, tv, 0.1, analytic=(True, Skv - Sq - 1, 0)) != fa.KERNEL_DECODE_SPLITKV


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("G,Sq,D,case", [(4, 12, 128, "causal"), (4, 32, 128, "window"), (8, 17, 64, "mask_tensor"),
                                         (4, 9, 96, "ragged"), (4, 24, 128, "full"),
                                         # the wide-head kernel's packed form (four wavefronts of 32 rows at 256, eight of 16 below)
                                         (4, 5, 256, "causal"), (4, 32, 256, "window"), (8, 17, 256, "mask_tensor"),
                                         (4, 9, 160, "ragged"), (4, 24, 192, "full"), (4, 31, 224, "causal")])
def test_rows_beyond_the_decode_kernel_share_the_kv_tiles_of_a_gqa_group(device, dtype, G, Sq, D, case):
    """9..32 new rows on a long cache in 16-bit: the tiled prefill kernel in its packed form, where a workgroup's four
    32-row blocks are four query heads of one KV head (the cache is read once per KV head); taken when the packed
    grid still fills the chip, which this batch does."""
    B, Hkv, Skv = 16, 4, 4100
    H = Hkv * G
    assert B * (H // 4) * (Skv // 1024) >= device.compute_units, "the packed form would not be chosen"
    q, k, v = _normal_qkv(48, B, H, Hkv, Sq, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    off = Skv - Sq
    kw, m, mask, kind = {}, None, None, None
    if case in ("causal", "window", "mask_tensor"):
        w = 0 if case == "causal" else 1500
        mask, kind = _analytic_mask(Sq, Skv, True, off, w), "qk"
        if case == "mask_tensor":
            m = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
        else:
            kw["analytic"] = (True, off, w)
    out_buf = fa.Tensor.empty(device, (B, Sq, H, D), dtype)      # written as [B, Sq, H, D]
    lens = None
    if case == "ragged":
        lens = np.array([Skv - 3 * i * 67 for i in range(B)], np.int32)
        lens[3] = 40
        kw["kv_lens"] = fa.IntTensor(device, lens)
    if m is None:  # (the selection of a call with a mask tensor depends on the workspace the call brings)
        assert tq.selected_kernel(tk, tv, 0.1, **kw) == fa.KERNEL_PREFILL_MFMA
    tq.flash_attention(tk, tv, D ** -0.5, m, out=out_buf.transpose(1, 2), **kw)
    got = out_buf.to_numpy().transpose(0, 2, 1, 3)
    if lens is None:
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask, kind)
        assert_parity(got, ref, _tol(dtype), f"{case} G{G} Sq{Sq} D{D}")
    else:
        for b in range(B):
            n = int(lens[b])
            ref = oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                         rounded(v[b:b + 1, :, :n], dtype), D ** -0.5)
            assert_parity(got[b:b + 1], ref, _tol(dtype), f"ragged b{b} len{n}")


def test_five_rows_at_a_head_dim_of_the_vector_variant_is_a_prefill_call(device):
    q, k, v = _normal_qkv(46, 1, 2, 2, 5, 300, 80)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, 0.1) == fa.KERNEL_PREFILL_F32
