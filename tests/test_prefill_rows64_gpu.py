"""GPU parity tests of the 64-rows-per-wavefront form of the tiled 16-bit prefill kernel at head_dim 128: 256-row
workgroups of four wavefronts, one per SIMD, software-pipelined over 32-key sub-tiles
(floneum_amd/csrc/attn_prefill_mfma_rows64.hip).

The library never chooses this form (it is a few per cent slower than the 256-row form of eight wavefronts); a caller
selects it with force_kernel = FHIP_KERNEL_PREFILL_MFMA_ROWS64, and it must then give the results of every other kernel.
Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199; the cases follow those of
tests/test_prefill_rows32_gpu.py.
"""
import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, assert_parity

pytestmark = pytest.mark.gpu

NEG_INF = float("-inf")
TOL_BF16 = dict(max_abs=2e-2, rel_l2=1e-2)
D = 128
FORCE = dict(force_kernel=fa.KERNEL_PREFILL_MFMA_ROWS64)


def rounded(a, dtype):
    if dtype == fa.F16:
        return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)
    return fa.bf16_bits_to_f32(fa.f32_to_bf16_bits(a))


def qkv(seed, B, H, Hkv, Sq, Skv, D, std=1.0):
    rng = np.random.default_rng(seed)
    return (rng.normal(0, std, (B, H, Sq, D)).astype(np.float32), rng.normal(0, std, (B, Hkv, Skv, D)).astype(np.float32),
            rng.normal(0, 1.0, (B, Hkv, Skv, D)).astype(np.float32))


def analytic_mask(Sq, Skv, causal, off, window):
    i = np.arange(Sq)[:, None] + off
    j = np.arange(Skv)[None, :]
    masked = np.zeros((Sq, Skv), bool)
    if causal:
        masked |= j > i
    if window:
        masked |= (j + window) <= i
    return np.where(masked, NEG_INF, 0.0).astype(np.float32)


def reference(q, k, v, D, dtype, mask=None, lens=None):
    outs = []
    for b in range(q.shape[0]):
        n = k.shape[2] if lens is None else int(lens[b])
        outs.append(oracle.flash_attention(rounded(q[b:b + 1], dtype), rounded(k[b:b + 1, :, :n], dtype),
                                           rounded(v[b:b + 1, :, :n], dtype), D ** -0.5, mask,
                                           None if mask is None else "qk"))
    return np.concatenate(outs, 0)



CASES = {
    # name: (Skv - Sq, analytic descriptor as (causal, window) or None, per-sequence key counts or None)
    "causal": (0, (True, 0), None),                  # square prompt: the last sub-tiles of a wavefront's rows are partly visible
    "causal_on_cached_keys": (388, (True, 0), None),  # 15 LDS tiles: every stage is reused several times
    "window": (0, (True, 100), None),                 # a row's first tiles are hidden: rows without a reference yet
    "window_on_cached_keys": (588, (True, 300), None),
    "no_mask": (188, None, None),                     # 700 keys: the last tile ends behind the key axis
    "odd_tiles": (230, (True, 0), None),              # 742 keys: an odd number of 32-key sub-tiles
    "key_counts": (188, None, [333, 41]),             # ragged batch: tiles and rows beyond a sequence's own keys
}


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("case", list(CASES))
def test_masks(device, dtype, case):
    """Every mask form the kernel takes analytically, on a grid of two rounds of workgroups (every LDS stage and register
    is reused by a second workgroup)."""
    B, H, Hkv, Sq = 4, 64, 16, 512
    extra, desc, lens = CASES[case]
    Skv = Sq + extra
    q, k, v = qkv(31, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    kw, mask = dict(FORCE), None
    if desc is not None:
        kw["analytic"] = (desc[0], extra, desc[1])
        mask = analytic_mask(Sq, Skv, desc[0], extra, desc[1])
    if lens is not None:
        kw["kv_lens"] = fa.IntTensor(device, np.array(lens + lens, np.int32))
        lens = lens + lens
    assert tq.selected_kernel(tk, tv, D ** -0.5, **kw) == fa.KERNEL_PREFILL_MFMA_ROWS64
    out = tq.flash_attention(tk, tv, D ** -0.5, **kw).to_numpy()
    ref = reference(q, k, v, D, dtype, mask, lens)
    assert_parity(out, ref, TOL_BF16 if dtype == fa.BF16 else TOL_16, case)


@pytest.mark.parametrize("Sq,Skv", [(300, 300), (77, 1000), (1024, 1024)])
def test_small_grids_and_ragged_query_blocks(device, Sq, Skv):
    """Fewer workgroups than CUs, a last query block whose wavefronts hold rows beyond the prompt, and the result of the
    256-row form of eight wavefronts on the same call (the two differ by rounding only)."""
    B, H, Hkv = 1, 8, 2
    q, k, v = qkv(7 + Sq, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    desc = (True, Skv - Sq, 0)
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=desc, **FORCE).to_numpy()
    ref = reference(q, k, v, D, fa.F16, analytic_mask(Sq, Skv, *desc))
    assert_parity(out, ref, TOL_16, f"{Sq} rows on {Skv} keys")
    other = tq.flash_attention(tk, tv, D ** -0.5, analytic=desc).to_numpy()
    assert_parity(out, other, dict(max_abs=2e-3, rel_l2=5e-4), "against the kernel the library chooses")


@pytest.mark.parametrize("dtype,tol", [(fa.F16, dict(max_abs=2e-3, rel_l2=2e-3)), (fa.BF16, dict(max_abs=2e-2, rel_l2=8e-3))])
@pytest.mark.parametrize("growth", [0.02, 0.3, 3.0, 40.0])
def test_row_maximum_that_keeps_rising(device, dtype, tol, growth):
    """The kernel takes no maximum per tile: a row's reference moves only when a lane's probabilities of a sub-tile sum
    to more than 2^15.  Scores that climb along the keys by `growth` per 32-key sub-tile on top of unit noise walk through
    every regime: never again after the first tile, once in many tiles, every few tiles, and every tile by far more than
    the slack (softmax rows close to one-hot on the last visible key)."""
    B, H, Hkv, Sq, Skv = 1, 32, 8, 1024, 1100
    q, k, v = qkv(5, B, H, Hkv, Sq, Skv, D)
    # (values in [-1, 1]: a row that is one-hot on its last key returns that key's value times a probability rounded to
    # the 16-bit type, which is not exactly 1 when the reference is not the row's own maximum; the gate is absolute)
    v = np.random.default_rng(6).uniform(-1, 1, v.shape).astype(np.float32)
    # dim 0 of every query is sqrt(D), dim 0 of key j is growth * j / 32: the scaled score gains growth per sub-tile
    q[..., 0] = D ** 0.5
    k[..., 0] = (growth / 32.0) * np.arange(Skv, dtype=np.float32)[None, None, :]
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    for desc in ((True, Skv - Sq, 0), (True, Skv - Sq, 300), None):
        kw = dict(FORCE) if desc is None else dict(FORCE, analytic=desc)
        out = tq.flash_attention(tk, tv, D ** -0.5, out_dtype=fa.F32, **kw).to_numpy()
        mask = None if desc is None else analytic_mask(Sq, Skv, *desc)
        ref = reference(q, k, v, D, dtype, mask)
        assert_parity(out, ref, tol, f"growth {growth}, mask {desc}")


@pytest.mark.parametrize("std", [3.0, 8.0, 30.0])
def test_f16_scores_of_large_magnitude(device, std):
    """The scale is applied exactly (its power-of-two part to Q, the rest to the f32 scores), so the error does not grow
    with the scores: queries and keys of standard deviation `std` give scaled scores of deviation std^2.  (Output taken as
    f32: rows this peaked return single values, and some of those exceed 4, where the f16 output's own rounding is as
    large as the gate.)"""
    B, H, Hkv, Sq = 2, 32, 8, 512
    rng = np.random.default_rng(77)
    q = rng.normal(0, std, (B, H, Sq, D)).astype(np.float32)
    k = rng.normal(0, std, (B, Hkv, Sq, D)).astype(np.float32)
    v = rng.normal(0, 1.0, (B, Hkv, Sq, D)).astype(np.float32)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, 0, 0), out_dtype=fa.F32, **FORCE).to_numpy()
    ref = reference(q, k, v, D, fa.F16, analytic_mask(Sq, Sq, True, 0, 0))
    # (std 30: scores of magnitude 2^12 are f32 numbers 2^-11 apart, in any implementation that forms them in f32 as the
    # reference does; on rows that are one-hot on a value of magnitude 5 that alone is a third of the absolute gate)
    assert_parity(out, ref, TOL_16 if std < 30 else dict(max_abs=4e-3, rel_l2=1e-3), f"std {std}")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("kind", ["causal", "window", "batch_key"])
def test_mask_tensors_made_of_intervals(device, dtype, kind):
    """A mask tensor whose rows are intervals of visible keys runs on the same kernel through its interval form (the
    library scans the tensor, or takes the table its owner computed once)."""
    B, H, Hkv, Sq, Skv = 2, 32, 8, 512, 640
    q, k, v = qkv(9, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    if kind == "batch_key":
        m = np.zeros((B, Skv), np.float32)
        m[0, 500:] = NEG_INF
        m[1, :37] = NEG_INF
        m[1, 333:] = NEG_INF
        mk, okind = fa.MaskKind.BatchKeyMask, "batch_key"
    else:
        m = analytic_mask(Sq, Skv, True, Skv - Sq, 0 if kind == "causal" else 200)
        mk, okind = fa.MaskKind.QKMask, "qk"
    tm = fa.Tensor.from_numpy(device, m, dtype)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, m, okind)
    tol = TOL_BF16 if dtype == fa.BF16 else TOL_16
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, mk), **FORCE).to_numpy()
    assert_parity(out, ref, tol, f"{kind}, scanned by the call")
    out2 = tq.flash_attention(tk, tv, D ** -0.5, (tm, mk, fa.MaskIntervals(tm)), **FORCE).to_numpy()
    assert np.array_equal(out, out2), f"{kind}: the call that carries the table differs from the call that scans"


def test_mask_tensor_that_is_not_made_of_intervals(device):
    """A mask with a hole in a row is not of the interval form: the forced kernel steps aside like the chosen one and the
    kernel queued behind it adds the mask values."""
    B, H, Hkv, Sq, Skv = 1, 8, 2, 256, 256
    q, k, v = qkv(13, B, H, Hkv, Sq, Skv, D)
    m = analytic_mask(Sq, Skv, True, 0, 0)
    m[200, 50:60] = NEG_INF
    tq, tk, tv, tm = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v, m))
    out = tq.flash_attention(tk, tv, D ** -0.5, (tm, fa.MaskKind.QKMask), **FORCE).to_numpy()
    ref = oracle.flash_attention(rounded(q, fa.F16), rounded(k, fa.F16), rounded(v, fa.F16), D ** -0.5, m, "qk")
    assert_parity(out, ref, TOL_16, "mask with a hole")


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16])
@pytest.mark.parametrize("layout", ["f32", "seq_major", "unaligned"])
def test_output_types_and_layouts(device, dtype, layout):
    """The output leaves through a transposition in LDS as 16-byte pieces of contiguous rows when its layout allows
    (also as f32, and into a [b, seq, heads * head_dim] buffer, what kalosm-llama's layers take), element by element
    otherwise (rows that start 8 bytes off a 16-byte boundary)."""
    B, H, Hkv, Sq = 3, 32, 8, 300
    q, k, v = qkv(17, B, H, Hkv, Sq, Sq, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    ref = reference(q, k, v, D, dtype, analytic_mask(Sq, Sq, True, 0, 0))
    tol = TOL_BF16 if dtype == fa.BF16 else TOL_16
    if layout == "f32":
        out = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, 0, 0), out_dtype=fa.F32, **FORCE).to_numpy()
    elif layout == "seq_major":
        buf = fa.Tensor.empty(device, (B, Sq, H, D), dtype)
        tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, 0, 0), out=buf.transpose(1, 2), **FORCE)
        out = buf.to_numpy().transpose(0, 2, 1, 3)
    else:
        buf = fa.Tensor.from_numpy(device, np.full((B, H, Sq, D + 8), 7.0, np.float32), dtype)
        tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, 0, 0), out=buf.narrow(3, 4, D), **FORCE)
        full = buf.to_numpy()
        assert (full[..., :4] == 7.0).all() and (full[..., D + 4:] == 7.0).all(), "elements beside the output were written"
        out = full[..., 4:D + 4]
    assert_parity(out, ref, tol, layout)


def test_rows_without_a_visible_key_and_queries_beyond_the_last_block(device):
    """Sq is not a multiple of 256 (the last block's wavefronts hold rows beyond the prompt, one of them none at all),
    and a key count of zero leaves a whole sequence without visible keys: NaN like the reference's 0 / 0."""
    B, H, Hkv, Sq, Skv = 4, 32, 8, 161, 161
    q, k, v = qkv(3, B, H, Hkv, Sq, Skv, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    lens = np.array([161, 0, 5, 100], np.int32)
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=(True, 0, 0), kv_lens=fa.IntTensor(device, lens), **FORCE).to_numpy()
    assert np.isnan(out[1]).all(), "a sequence without keys must give NaN"
    mask = analytic_mask(Sq, Skv, True, 0, 0)
    for b in (0, 2, 3):
        n = int(lens[b])
        ref = oracle.flash_attention(rounded(q[b:b + 1], fa.F16), rounded(k[b:b + 1, :, :n], fa.F16),
                                     rounded(v[b:b + 1, :, :n], fa.F16), D ** -0.5, mask[:, :n], "qk")
        # rows behind the sequence's keys see all of them (causality hides nothing more): still finite
        assert_parity(out[b:b + 1], ref, TOL_16, f"sequence {b} of {n} keys")


def test_forced_on_a_call_it_cannot_run(device):
    """Other head dims, f32 tensors and scales whose power-of-two part Q cannot carry are refused, not served by another
    kernel in silence."""
    q, k, v = qkv(1, 1, 4, 4, 64, 64, 64)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    with pytest.raises(fa.FhipError):
        tq.flash_attention(tk, tv, 0.125, **FORCE)
    q, k, v = qkv(1, 1, 4, 4, 64, 64, D)
    t32 = [fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v)]
    with pytest.raises(fa.FhipError):
        t32[0].flash_attention(t32[1], t32[2], D ** -0.5, **FORCE)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    with pytest.raises(fa.FhipError):
        tq.flash_attention(tk, tv, 4.0, **FORCE)


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_mixed_feature_sweep(device, seed):
    """A seeded sweep with the form forced: both 16-bit types, GQA groups, batches, prompt / chunk-on-cache / few-rows
    shapes and every way of masking the call accepts (a mask that is not made of intervals, or carries finite biases,
    leaves the call to the kernel queued behind this one).  Rows without a visible key must be NaN on both sides."""
    rng = np.random.default_rng(seed)
    gate = {fa.F16: (2e-3, 1e-3), fa.BF16: (2e-2, 8e-3)}
    for it in range(40):
        dtype = [fa.F16, fa.BF16][rng.integers(2)]
        Hkv = int(rng.integers(1, 4))
        H = Hkv * int(rng.choice([1, 2, 4]))
        B = int(rng.integers(1, 4))
        shape = rng.choice(["square", "chunk", "few_rows"])
        if shape == "square":
            Sq = Skv = int(rng.integers(1, 700))
        elif shape == "chunk":
            Sq, Skv = int(rng.integers(1, 300)), int(rng.integers(300, 1500))
        else:
            Sq, Skv = int(rng.integers(1, 70)), int(rng.integers(1000, 3000))
        q, k, v = qkv(int(rng.integers(1 << 30)), B, H, Hkv, Sq, Skv, D)
        mk = rng.choice(["none", "analytic", "get_mask", "bias", "batch_key", "kv_lens"])
        mask = kind = analytic = mt = lens_t = None
        if mk == "analytic":
            w = int(rng.integers(1, Skv + 5)) if rng.random() < 0.5 else 0
            analytic = (True, Skv - Sq, w)
            mask, kind = analytic_mask(Sq, Skv, True, Skv - Sq, w), "qk"
        elif mk == "get_mask":
            w = int(rng.integers(1, 2 * Skv)) if rng.random() < 0.5 else None
            full = oracle.get_mask(Sq, Skv - Sq, w)
            if full.shape == (Sq, Skv):
                mask, kind = full, "qk"
                mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
        elif mk == "bias":
            mask, kind = rng.normal(0, 1, (Sq, Skv)).astype(np.float32), "qk"
            mask[:, rng.integers(1, Skv):] = NEG_INF
            mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.QKMask)
        elif mk == "batch_key":
            mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
            for b in range(B):
                mask[b, int(rng.integers(1, Skv + 1)):] = NEG_INF if rng.random() < 0.7 else -10000.0
            mt = (fa.Tensor.from_numpy(device, mask, dtype), fa.MaskKind.BatchKeyMask)
        elif mk == "kv_lens":
            lens = rng.integers(1, Skv + 1, B).astype(np.int32)
            lens_t = fa.IntTensor(device, lens)
            mask, kind = np.zeros((B, Skv), np.float32), "batch_key"
            for b in range(B):
                mask[b, lens[b]:] = NEG_INF
        what = f"case {it}: dtype {dtype} B {B} H {H} Hkv {Hkv} Sq {Sq} Skv {Skv} {mk} {analytic}"
        tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
        out = tq.flash_attention(tk, tv, D ** -0.5, mt, analytic=analytic, kv_lens=lens_t, out_dtype=fa.F32, **FORCE).to_numpy()
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5,
                                     None if mask is None else rounded(mask, dtype), kind)
        dead_ref = np.isnan(ref).any(-1)
        assert np.array_equal(np.isnan(out).any(-1), dead_ref), f"{what}: rows without a visible key differ"
        live = ~dead_ref
        if live.any():
            assert_parity(out[live], ref[live], dict(max_abs=gate[dtype][0], rel_l2=gate[dtype][1]), what)
