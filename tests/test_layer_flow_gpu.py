"""The whole per-layer flow kalosm-llama runs around the attention call, on the device, against the CPU checker.

models/kalosm-llama/src/raw/attention_layer.rs: the projections arrive as [b, seq, heads, hd] and are viewed as
[b, heads, seq, hd] (:226-229), q and k go through their RMS norms when the block has them (:229-257), both are
rotated (:272-278), k and v join the layer's KvCache (:400-420; sliding layers hold the last W positions,
raw/cache.rs:27-39), MaskCache::get_mask gives the mask of the step (raw/mod.rs:618-620), the attention runs, and
its output is transposed back to [b, seq, heads * hd] for the output projection (:450-454).

Here: a prompt, then token-by-token steps, each compared with the same flow on the CPU restatements.
"""
import ctypes

import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, TOL_F32, assert_parity
from test_attention_gpu import rounded

pytestmark = pytest.mark.gpu


def _cpu_layer(state, q, k, v, pos, cfg):
    """One call of the layer on the CPU restatements; state = oracle.KvCache."""
    D = q.shape[-1]
    qh, kh, vh = (a.transpose(0, 2, 1, 3) for a in (q, k, v))  # [b, heads, seq, hd]
    if cfg["norm"]:
        qh = rounded(oracle.rms_norm(qh, cfg["qw"], None, 1e-6), cfg["dtype"])
        kh = rounded(oracle.rms_norm(kh, cfg["kw"], None, 1e-6), cfg["dtype"])
    qr = rounded(oracle.rope(qh, cfg["cos"], cfg["sin"], pos), cfg["dtype"])
    kr = rounded(oracle.rope(kh, cfg["cos"], cfg["sin"], pos), cfg["dtype"])
    ka, va = state.append(kr, rounded(vh, cfg["dtype"]))
    n = q.shape[1]
    mask = oracle.get_mask(n, pos, cfg["window"])
    assert mask.shape == (n, ka.shape[2])
    out = oracle.flash_attention(qr, np.ascontiguousarray(ka), np.ascontiguousarray(va), D ** -0.5, mask, "qk")
    return out.transpose(0, 2, 1, 3).reshape(q.shape[0], n, -1)


@pytest.mark.parametrize("dtype,window,norm,D", [(fa.F32, None, False, 64), (fa.F32, 24, True, 128), (fa.F16, None, True, 128),
                                                 (fa.F32, 16, False, 256), (fa.F16, 20, False, 96)])
def test_prompt_then_decode_steps(device, dtype, window, norm, D):
    B, H, Hkv = 2, 4, 2
    rng = np.random.default_rng(3)
    rc = fa.RopeCache(D, 256, 10000.0, device)
    cfg = dict(dtype=dtype, window=window, norm=norm, cos=rc.cos_host, sin=rc.sin_host,
               qw=rounded(rng.normal(1, 0.2, D).astype(np.float32), dtype), kw=rounded(rng.normal(1, 0.2, D).astype(np.float32), dtype))
    qn = fa.RmsNorm(cfg["qw"], None, 1e-6, dtype, device) if norm else None
    kn = fa.RmsNorm(cfg["kw"], None, 1e-6, dtype, device) if norm else None
    max_len = window if window is not None else 4096   # raw/cache.rs:27-39
    cache, ocache = fa.KvCache(2, max_len, dtype, device), oracle.KvCache(2, max_len)
    masks = fa.MaskCache(dtype)
    tol = TOL_F32 if dtype == fa.F32 else TOL_16
    pos = 0
    # (a prompt longer than the window is not a case the reference can run: its cache would return W keys for a
    # [n, n] mask and the operator's shape assert would fire)
    prompt = 37 if window is None else window - 3
    for step, n in enumerate([prompt] + [1] * 12 + [5] + [1] * 6):
        q = rounded(rng.normal(0, 1, (B, n, H, D)).astype(np.float32), dtype)     # [b, seq, heads, hd] projections
        k = rounded(rng.normal(0, 1, (B, n, Hkv, D)).astype(np.float32), dtype)
        v = rounded(rng.normal(0, 1, (B, n, Hkv, D)).astype(np.float32), dtype)
        tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype).transpose(1, 2) for a in (q, k, v))
        q_rot, k_all, v_all = cache.qkv_rope_append(rc, tq, tk, tv, pos, False, qn, kn)
        mask = masks.get_mask(n, pos, window, device)
        out_buf = fa.Tensor.empty(device, (B, n, H, D), dtype)                      # what attention_wo multiplies
        out = q_rot.flash_attention(k_all, v_all, D ** -0.5, (mask.mask(), fa.MaskKind.QKMask), out=out_buf.transpose(1, 2))
        got = out_buf.to_numpy().reshape(B, n, H * D)
        ref = _cpu_layer(ocache, q, k, v, pos, cfg)
        assert k_all.shape[2] == ocache.current_seq_len()
        assert_parity(got, ref, tol, f"step {step} (pos {pos}, {n} new tokens)")
        pos += n
