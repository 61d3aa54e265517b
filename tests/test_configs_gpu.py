"""The five benchmark configurations at full size against the CPU checker, plus the KV-cache and
mask-cache flow that produces their inputs in kalosm-llama
(models/kalosm-llama/src/raw/mod.rs:600-652, raw/attention_layer.rs:362-455).

Full-size prefill outputs are compared on a subset of query rows (rows are independent in the
reference algorithm, fusor-ml/fusor/src/composite/flash_attention.rs:141-199) and, over the whole
tensor, through size-independent properties."""
import numpy as np
import pytest

import floneum_amd as fa
import oracle
from floneum_amd import synth
from conftest import TOL_16, TOL_F32, assert_parity

pytestmark = pytest.mark.gpu
SEED = 0xF10E0000


def f32(a):
    return np.asarray(a, np.float32)


def test_c1_llama32_1b_prefill_f32(device):
    # B1 S512 H32/Hkv8 D64 f32 N(0,1), scale 1/8, causal mask from MaskCache (dense tensor, as kalosm-llama passes it)
    B, H, Hkv, S, D = 1, 32, 8, 512, 64
    q, k, v = (synth.normal(SEED + 1, i, s) for i, s in enumerate([(B, H, S, D), (B, Hkv, S, D), (B, Hkv, S, D)]))
    mc = fa.MaskCache(fa.F32)
    am = mc.get_mask(S, 0, None, device)
    assert np.array_equal(am.host, oracle.get_mask(S, 0))  # bit-exact mask
    tq, tk, tv = (fa.Tensor.from_numpy(device, a) for a in (q, k, v))
    ref = oracle.flash_attention(q, k, v, 0.125, am.host, "qk")
    # the reference call: dense QKMask (reduced to intervals on the device, f32 MFMA kernel) ...
    out_dense = tq.flash_attention(tk, tv, 0.125, (am.mask(), fa.MaskKind.QKMask)).to_numpy()
    assert_parity(out_dense, ref, TOL_F32, "C1 dense mask")
    # ... the general kernel on the same tensor ...
    out_gen = tq.flash_attention(tk, tv, 0.125, (am.mask(), fa.MaskKind.QKMask), force_kernel=fa.KERNEL_GENERIC).to_numpy()
    assert_parity(out_gen, ref, TOL_F32, "C1 dense mask, general kernel")
    # ... and the analytic descriptor of the same mask (f32 MFMA kernel): bit-identical to the dense call
    assert tq.selected_kernel(tk, tv, 0.125, analytic=am.analytic) == fa.KERNEL_PREFILL_F32
    out = tq.flash_attention(tk, tv, 0.125, analytic=am.analytic).to_numpy()
    assert_parity(out, ref, TOL_F32, "C1 analytic")
    assert np.array_equal(out, out_dense)
    assert np.array_equal(out[:, :, 0], np.repeat(v, H // Hkv, axis=1)[:, :, 0])  # causal row 0 == V[0]


def test_c2_llama3_8b_decode_f16(device):
    B, H, Hkv, S, D = 16, 32, 8, 4096, 128
    q = synth.normal(SEED + 2, 0, (B, H, 1, D), 0.5, np.float16)
    k = synth.normal(SEED + 2, 1, (B, Hkv, S, D), 0.5, np.float16)
    v = synth.normal(SEED + 2, 2, (B, Hkv, S, D), 0.5, np.float16)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    assert tq.selected_kernel(tk, tv, D ** -0.5) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
    ref = oracle.flash_attention(f32(q), f32(k), f32(v), D ** -0.5)
    assert_parity(out, ref, TOL_16, "C2")
    # the mask kalosm-llama would pass for this step, get_mask(1, 4095, None) = [1, 4096] zeros, changes nothing
    am = fa.MaskCache(fa.F16).get_mask(1, S - 1, None, device)
    assert am.host.shape == (1, S) and not am.host.any()
    out_m = tq.flash_attention(tk, tv, D ** -0.5, (am.mask(), fa.MaskKind.QKMask)).to_numpy()
    assert np.array_equal(out_m, out)


def test_c3_llama3_8b_prefill_f16(device):
    B, H, Hkv, S, D = 1, 32, 8, 8192, 128
    q = synth.normal(SEED + 3, 0, (B, H, S, D), 1.0, np.float16)
    k = synth.normal(SEED + 3, 1, (B, Hkv, S, D), 1.0, np.float16)
    v = synth.normal(SEED + 3, 2, (B, Hkv, S, D), 1.0, np.float16)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    am = fa.CAnalyticMask(1, 1, 0, 0)
    assert tq.selected_kernel(tk, tv, D ** -0.5, analytic=am) == fa.KERNEL_PREFILL_MFMA
    out = tq.flash_attention(tk, tv, D ** -0.5, analytic=am).to_numpy()
    out32 = tq.flash_attention(tk, tv, D ** -0.5, analytic=am, out_dtype=fa.F32).to_numpy()
    rows = np.unique(np.concatenate([np.arange(0, 40), np.arange(250, 262), np.linspace(0, S - 1, 48).astype(int),
                                     np.arange(S - 8, S)])).astype(np.int32)
    mask = np.where(np.arange(S)[None, :] > rows[:, None], -np.inf, 0.0).astype(np.float32)
    ref = oracle.flash_attention(f32(q)[:, :, rows], f32(k), f32(v), D ** -0.5, mask, "qk")
    assert_parity(out[:, :, rows], ref, TOL_16, "C3 f16 out")
    assert_parity(out32[:, :, rows], ref, TOL_16, "C3 f32 out")
    # the call as the reference's caller makes it, with the [8192, 8192] mask tensor of MaskCache (f16, 128 MiB):
    # reduced to intervals on the device, same kernel, same bits
    dense = fa.MaskCache(fa.F16).get_mask(S, 0, None, device)
    out_dense = tq.flash_attention(tk, tv, D ** -0.5, (dense.mask(), fa.MaskKind.QKMask)).to_numpy()
    assert np.array_equal(out_dense, out)
    del dense, out_dense
    # whole-tensor properties: no NaN, row 0 == V[0] exactly, every output inside the range of V (convex combination)
    assert not np.isnan(out).any()
    assert np.array_equal(out[:, :, 0], np.repeat(v, H // Hkv, axis=1)[:, :, 0])
    vmax = np.repeat(np.maximum.accumulate(f32(v), axis=2), H // Hkv, axis=1)
    vmin = np.repeat(np.minimum.accumulate(f32(v), axis=2), H // Hkv, axis=1)
    assert (out32 <= vmax + 2e-3).all() and (out32 >= vmin - 2e-3).all()


def test_c4_mistral_sliding_window_chunk(device):
    # 512 new tokens on a 16384-token cache, W = 4096: the sliding layer's KvCache (max_sequence_len = W)
    # keeps the last 4096 positions and MaskCache gives [512, 4096] = 3584 zero columns + causal block
    B, H, Hkv, D, W, chunk, cached = 4, 32, 8, 128, 4096, 512, 16384
    cache = fa.KvCache(2, W, fa.F16, device)
    ocache = oracle.KvCache(2, W)
    k_all = v_all = ok = ov = None
    # fill the cache in big steps, then append the chunk (the last `W - chunk` cached positions survive)
    for step, n in enumerate([8192, 8192, chunk]):
        kn = synth.normal(SEED + 4, 10 + step, (B, Hkv, n, D), 1.0, np.float16)
        vn = synth.normal(SEED + 4, 20 + step, (B, Hkv, n, D), 1.0, np.float16)
        k_all, v_all = cache.append(device, fa.Tensor.from_numpy(device, kn, fa.F16), fa.Tensor.from_numpy(device, vn, fa.F16))
        ok, ov = ocache.append(kn, vn)
    assert cache.current_seq_len() == W and k_all.shape == (B, Hkv, W, D)
    assert np.array_equal(k_all.to_numpy(), ok) and np.array_equal(v_all.to_numpy(), ov)  # bit-exact cache content
    q = synth.normal(SEED + 4, 0, (B, H, chunk, D), 1.0, np.float16)
    tq = fa.Tensor.from_numpy(device, q, fa.F16)
    am = fa.MaskCache(fa.F16).get_mask(chunk, cached, W, device)
    dense = oracle.get_mask(chunk, cached, W)
    assert am.host.shape == (chunk, W) and np.array_equal(np.isneginf(am.host), np.isneginf(dense))
    assert am.analytic.q_pos_offset == W - chunk and am.analytic.window == W
    out = tq.flash_attention(k_all, v_all, D ** -0.5, analytic=am.analytic).to_numpy()
    rows = np.unique(np.concatenate([np.arange(0, 8), np.linspace(0, chunk - 1, 24).astype(int)])).astype(np.int32)
    ref = oracle.flash_attention(f32(q)[:, :, rows], f32(ok), f32(ov), D ** -0.5, dense[rows], "qk")
    assert_parity(out[:, :, rows], ref, TOL_16, "C4")
    # the dense-mask call (what the reference's caller passes) on one batch entry agrees
    out_d = tq.narrow(0, 0, 1).flash_attention(k_all.narrow(0, 0, 1), v_all.narrow(0, 0, 1), D ** -0.5,
                                               (am.mask(), fa.MaskKind.QKMask)).to_numpy()
    assert_parity(out_d[:, :, rows], ref[:1], TOL_16, "C4 dense mask")


def test_c5_phi3_ragged_decode(device):
    B, H, D = 32, 32, 96
    lens = synth.integers(SEED + 5, 7, B, 128, 32768).astype(np.int32)
    Smax = int(lens.max())
    q = synth.normal(SEED + 5, 0, (B, H, 1, D), 1.0, np.float16)
    # two generated sequences reused across the batch keep host time and memory modest
    base_k = synth.normal(SEED + 5, 1, (2, H, Smax, D), 1.0, np.float16)
    base_v = synth.normal(SEED + 5, 2, (2, H, Smax, D), 1.0, np.float16)
    k = np.empty((B, H, Smax, D), np.float16)
    v = np.empty((B, H, Smax, D), np.float16)
    for b in range(B):
        k[b], v[b] = base_k[b % 2], base_v[(b + 1) % 2]
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    tl = fa.IntTensor(device, lens)
    assert tq.selected_kernel(tk, tv, D ** -0.5, kv_lens=tl) == fa.KERNEL_DECODE_SPLITKV
    out = tq.flash_attention(tk, tv, D ** -0.5, kv_lens=tl).to_numpy()
    assert not np.isnan(out).any()
    for b in list(range(0, B, 5)) + [int(np.argmin(lens)), int(np.argmax(lens))]:
        n = int(lens[b])
        ref = oracle.flash_attention(f32(q[b:b + 1]), f32(k[b:b + 1, :, :n]), f32(v[b:b + 1, :, :n]), D ** -0.5)
        assert_parity(out[b:b + 1], ref, TOL_16, f"C5 sequence {b} (len {n})")


def test_kv_cache_growth_matches_reference_semantics(device):
    # pow-2 growth, in-place row writes, strided sources, truncation (tensor_cache.rs:48-118)
    rng = np.random.default_rng(5)
    for dtype, npdt in ((fa.F32, np.float32), (fa.F16, np.float16)):
        for max_len in (7, 64):
            cache, oc = fa.KvCache(2, max_len, dtype, device), oracle.KvCache(2, max_len)
            for step in range(10):
                n = int(rng.integers(1, 6))
                kn = rng.standard_normal((2, 3, n, 16)).astype(npdt)
                vn = rng.standard_normal((2, 3, n, 16)).astype(npdt)
                # the value tensor arrives as the transposed view of a [B, S, Hkv, D] buffer
                tvn = fa.Tensor.from_numpy(device, np.ascontiguousarray(vn.transpose(0, 2, 1, 3)), dtype).transpose(1, 2)
                ka, va = cache.append(device, fa.Tensor.from_numpy(device, kn, dtype), tvn)
                ok, ov = oc.append(kn, vn)
                assert ka.shape == ok.shape and cache.current_seq_len() == oc.current_seq_len()
                assert cache.allocated_seq_len() == oc.key.allocated_seq_len
                # the view keeps the buffer's stride: the allocation while it grows, twice max_len once it slides
                assert ka.strides[1] in (cache.allocated_seq_len() * 16, 2 * max_len * 16)
                assert np.array_equal(ka.to_numpy(), ok) and np.array_equal(va.to_numpy(), ov)
            cache.reset()
            assert cache.current_seq_len() == 0


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16])
def test_full_kv_cache_slides_without_recopying(device, dtype):
    """Once max_sequence_len rows are cached every append drops the oldest rows (tensor_cache.rs:55-78).  The device
    cache slides a window through a buffer of twice that length, so the values and the order the caller sees are the
    reference's, through many wrap-arounds and with blocks of every size up to beyond the window."""
    rng = np.random.default_rng(9)
    W, B, Hkv, D = 16, 2, 2, 32
    cache, oc = fa.KvCache(2, W, dtype, device), oracle.KvCache(2, W)
    npdt = np.float32 if dtype == fa.F32 else np.float16
    sizes = [5, 9, 3] + [1] * 40 + [7, 1, 16, 1, 1, 15, 2, 40, 1, 1, 1, 17, 1] + [2] * 20
    pos = 0
    q = rng.standard_normal((B, 4, 1, D)).astype(np.float32)
    tq = fa.Tensor.from_numpy(device, q, dtype)
    for step, n in enumerate(sizes):
        kn = rng.standard_normal((B, Hkv, n, D)).astype(npdt)
        vn = rng.standard_normal((B, Hkv, n, D)).astype(npdt)
        ka, va = cache.append(device, fa.Tensor.from_numpy(device, kn, dtype), fa.Tensor.from_numpy(device, vn, dtype))
        ok, ov = oc.append(kn, vn)
        assert ka.shape == ok.shape and cache.current_seq_len() == oc.current_seq_len(), f"step {step}"
        assert cache.allocated_seq_len() == oc.key.allocated_seq_len, f"step {step}"
        assert np.array_equal(ka.to_numpy(), ok) and np.array_equal(va.to_numpy(), ov), f"step {step}"
        pos += n
        if step % 7 == 0:  # the moving view feeds the attention call as it is
            out = tq.flash_attention(ka, va, D ** -0.5).to_numpy()
            ref = oracle.flash_attention(np.asarray(q, np.float32).astype(npdt).astype(np.float32), ok.astype(np.float32),
                                         ov.astype(np.float32), D ** -0.5)
            assert_parity(out, ref, TOL_F32 if dtype == fa.F32 else TOL_16, f"attention over the window, step {step}")
