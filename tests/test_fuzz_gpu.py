"""A seeded sweep across every feature of the attention call at once, against the CPU checker.

The reference fuzzes its fused kernel against its unfused path over random shapes
(fusor-ml/core/src/composite/flash_attention.rs:559-1060); this does the same through the C ABI with everything the
boundary accepts mixed freely: the three element types, head dims on and off the tile widths (8 ... 256, odd ones for
the general kernel), GQA group sizes, batch, decode / multi-token decode / longer drafts / square / chunk-on-cache / tiny / long-cache shapes, and every way
of masking (none, the analytic descriptor, MaskCache tensors, finite biases, padding masks with -inf or -10000.0, key
counts).  Rows without a visible key must be NaN on both sides.
"""
import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import max_abs, rel_l2
from test_attention_gpu import rounded

pytestmark = pytest.mark.gpu

NEG = float("-inf")
# The parity gate, (max-abs, rel-L2): f32 tensors relative L2 1e-5; f16 tensors max-abs 2e-3 and relative L2 1e-3.
# 16-bit cases are held to it on the f32 output the ABI offers (out_dtype = F32): the arithmetic is the same, and the
# comparison is then free of the final rounding to 16 bits, which alone is half a unit in the last place of the value
# (4.9e-4 of a value of order 1 in f16).  bf16 is not a type the gate names: its probabilities carry 8 bits, the bound
# below is what that allows.
GATE = {fa.F32: (None, 1e-5), fa.F16: (2e-3, 1e-3), fa.BF16: (2e-2, 8e-3)}
# second, looser check of the same call with the output in the tensors' own type (what the reference returns)
NATIVE = {fa.F16: (1e-2, 2e-3), fa.BF16: (1e-1, 2e-2)}


def _case(rng, device):
    dtype = [fa.F32, fa.F16, fa.BF16][rng.integers(3)]
    D = int(rng.choice([8, 16, 32, 40, 64, 80, 96, 128, 160, 192, 224, 256, 12, 36, 100, 33]))
    Hkv = int(rng.integers(1, 4))
    H = Hkv * int(rng.choice([1, 2, 4, 8]))
    B = int(rng.integers(1, 4))
    mode = rng.choice(["decode", "multi", "draft", "square", "chunk", "tiny", "long"])
    if mode == "decode":
        Sq, Skv = 1, int(rng.integers(1, 3000))
    elif mode == "multi":  # a multi-token decode step: a few new rows at the end of a cache
        Sq = int(rng.integers(2, 5))
        Skv = Sq + int(rng.integers(0, 3000))
    elif mode == "draft":  # more rows than 4: on the decode kernels while rows x GQA group fit a workgroup's columns
        Sq = int(rng.integers(5, 17))
        Skv = Sq + int(rng.integers(0, 3000))
    elif mode == "square":
        Sq = Skv = int(rng.integers(1, 400))
    elif mode == "chunk":
        Sq, Skv = int(rng.integers(1, 200)), int(rng.integers(200, 1500))
    elif mode == "tiny":
        Sq, Skv = int(rng.integers(1, 9)), int(rng.integers(1, 9))
    else:
        Sq, Skv, B = int(rng.integers(1, 70)), int(rng.integers(2000, 6000)), 1
    if Skv < Sq and mode != "tiny":
        Skv = Sq
    q = rng.normal(0, 1, (B, H, Sq, D)).astype(np.float32)
    k = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    v = rng.normal(0, 1, (B, Hkv, Skv, D)).astype(np.float32)
    mk = rng.choice(["none", "analytic", "get_mask", "bias", "batch_key", "kv_lens"])
    mask = kind = analytic = mt = lens_t = None
    if mk == "analytic" and Skv >= Sq:
        w = int(rng.integers(1, Skv + 5)) if rng.random() < 0.5 else 0
        analytic = (True, Skv - Sq, w)
        i = np.arange(Sq)[:, None] + (Skv - Sq)
        j = np.arange(Skv)[None, :]
        hidden = j > i
        if w:
            hidden |= (j + w) <= i
        mask, kind = np.where(hidden, NEG, 0).astype(np.float32), "qk"
    elif mk == "get_mask" and Skv >= Sq:
        w = int(rng.integers(1, 2 * Skv)) if rng.random() < 0.5 else None
        full = oracle.get_mask(Sq, Skv - Sq, w)
        if full.shape == (Sq, Skv):
            mask, kind = full, "qk"
            mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif mk == "bias":
        mask, kind = rng.normal(0, 1, (Sq, Skv)).astype(np.float32), "qk"
        if Skv > 3:
            mask[:, rng.integers(0, Skv - 1):] = NEG
            mask[:, 0] = 0
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
    elif mk == "batch_key":
        mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
        for b in range(B):
            mask[b, int(rng.integers(1, Skv + 1)):] = NEG if rng.random() < 0.5 else -10000.0
        mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.BatchKeyMask)
    elif mk == "kv_lens":
        lens = rng.integers(1, Skv + 1, B).astype(np.int32)
        lens_t = fa.IntTensor(device, lens)
        mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
        for b in range(B):
            mask[b, lens[b]:] = NEG
    what = f"dtype {dtype} D {D} B {B} H {H} Hkv {Hkv} Sq {Sq} Skv {Skv} {mk} {analytic}"
    return dtype, D, q, k, v, mask, kind, analytic, mt, lens_t, what


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_mixed_feature_sweep(device, seed):
    rng = np.random.default_rng(seed)
    used = set()
    for it in range(60):
        dtype, D, q, k, v, mask, kind, analytic, mt, lens_t, what = _case(rng, device)
        tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
        scale = float(D) ** -0.5
        used.add(tq.selected_kernel(tk, tv, scale, mt, analytic=analytic, kv_lens=lens_t))
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale,
                                     None if mask is None else rounded(mask, dtype), kind)
        dead_ref = np.isnan(ref).any(-1)
        live = ~dead_ref
        passes = [(fa.F32, GATE[dtype], "f32 output")] if dtype == fa.F32 else \
                 [(fa.F32, GATE[dtype], "f32 output"), (dtype, NATIVE[dtype], "native output")]
        for out_dtype, (tol_abs, tol_rel), label in passes:
            out = tq.flash_attention(tk, tv, scale, mt, analytic=analytic, kv_lens=lens_t, out_dtype=out_dtype).to_numpy()
            dead_out = np.isnan(out).any(-1)
            assert np.array_equal(dead_out, dead_ref), f"case {it} ({label}): rows without a visible key differ: {what}"
            if live.any():
                rl = rel_l2(out[live], ref[live])
                assert rl <= tol_rel, f"case {it} ({label}): rel-L2 {rl:.3e} > {tol_rel:.0e}: {what}"
                if tol_abs is not None:
                    ma = max_abs(out[live], ref[live])
                    assert ma <= tol_abs, f"case {it} ({label}): max-abs {ma:.3e} > {tol_abs:.0e}: {what}"
    assert len(used) >= 3, "the sweep is meant to cross kernels"
