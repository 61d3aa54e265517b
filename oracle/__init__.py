"""CPU checker for the attention path -- TEST INFRASTRUCTURE, not part of the shipped library.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package.
It restates fusor-ml's CPU attention composite (C, ``fusor_cpu_attention.c``), its mask builders,
its growable KV cache, its rotary embedding and its RMS norm (numpy, this file), and carries float64
textbook twins used to pin the restatements.

Parity status: everything here is pinned by the checks in tests/test_oracle.py,
tests/test_rope_oracle.py and tests/test_rms_norm_oracle.py except two bit-level details, which are PARITY UNPINNED: the summation order
of the `gemm` 0.18.2 micro-kernels inside the two matrix products (value-level parity is pinned, three
orders of magnitude inside the 1e-5 tolerance), and the last bit of cos/sin in ``rope_tables`` (libm
dependent; the rotation takes the tables as inputs, so no op result depends on it).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

MASK_NONE, MASK_QK, MASK_BATCH_KEY = 0, 1, 2


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    so = os.path.join(_HERE, "liboracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        L = ctypes.CDLL(so)
        fp = ctypes.POINTER(ctypes.c_float)
        ip = ctypes.POINTER(ctypes.c_int32)
        L.oracle_flash_attention_f32.restype = ctypes.c_int
        L.oracle_flash_attention_f32.argtypes = [fp, fp, fp, fp, ctypes.c_int] + [ctypes.c_int] * 6 + [
            ctypes.c_float, ip, ctypes.c_int, fp, ctypes.c_int]
        L.oracle_flash_attention_naive_f32.restype = ctypes.c_int
        L.oracle_flash_attention_naive_f32.argtypes = [fp, fp, fp, fp, ctypes.c_int] + [ctypes.c_int] * 6 + [
            ctypes.c_float, fp]
        L.oracle_mask_causal_f32.argtypes = [ctypes.c_int, fp]
        L.oracle_mask_sliding_f32.argtypes = [ctypes.c_int, ctypes.c_long, fp]
        L.oracle_get_mask_offset.restype = ctypes.c_long
        L.oracle_get_mask_offset.argtypes = [ctypes.c_long, ctypes.c_long, ctypes.c_int, ctypes.c_long]
        L.oracle_get_mask_f32.argtypes = [ctypes.c_int, ctypes.c_long, ctypes.c_int, ctypes.c_long, fp]
        _LIB = L
    return _LIB


def _f32c(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _mask_args(mask, kind, B, Sq, Skv):
    if mask is None:
        return None, None, MASK_NONE
    kind = {"qk": MASK_QK, "batch_key": MASK_BATCH_KEY}.get(kind, kind)
    want = (Sq, Skv) if kind == MASK_QK else (B, Skv)
    # the reference asserts on the mask shape (fusor flash_attention.rs:153-172)
    if tuple(mask.shape) != want:
        raise AssertionError(f"mask shape {tuple(mask.shape)} does not match expected {list(want)}")
    m, mp = _f32c(mask)
    return m, mp, kind


def flash_attention(q, k, v, scale, mask=None, mask_kind=None, rows=None, nthreads=0, naive=False):
    """fusor CPU attention on f32 values (f16 inputs are upcast exactly by the caller or here).

    q [B,H,Sq,D]; k, v [B,Hkv,Skv,D]; mask [Sq,Skv] ('qk') or [B,Skv] ('batch_key').
    rows: optional query-row subset -> output [B,H,len(rows),D].
    """
    q, qp = _f32c(q)
    k, kp = _f32c(k)
    v, vp = _f32c(v)
    B, H, Sq, D = q.shape
    Bk, Hkv, Skv, Dk = k.shape
    assert v.shape == k.shape and Bk == B and Dk == D
    m, mp, kind = _mask_args(mask, mask_kind, B, Sq, Skv)
    L = lib()
    if naive:
        assert rows is None
        out = np.empty((B, H, Sq, D), np.float32)
        rc = L.oracle_flash_attention_naive_f32(qp, kp, vp, mp, kind, B, H, Hkv, Sq, Skv, D,
                                                np.float32(scale), out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)))
    else:
        if rows is not None:
            rows = np.ascontiguousarray(rows, dtype=np.int32)
            assert rows.size == 0 or (rows.min() >= 0 and rows.max() < Sq)
            rp, nr = rows.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), int(rows.size)
        else:
            rp, nr = None, 0
        out = np.empty((B, H, nr if rows is not None else Sq, D), np.float32)
        rc = L.oracle_flash_attention_f32(qp, kp, vp, mp, kind, B, H, Hkv, Sq, Skv, D, np.float32(scale),
                                          rp, nr, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), nthreads)
    if rc == -1:
        raise AssertionError(f"Number of Q heads ({H}) must be divisible by number of K/V heads ({Hkv})")
    if rc != 0:
        raise MemoryError("oracle allocation failed")
    return out


def flash_attention_f64(q, k, v, scale, mask=None, mask_kind=None):
    """Textbook softmax attention in float64 -- the referee used to pin the f32 restatement.

    Shares nothing with the C code except the definition of the operator: GQA by kv = h // G,
    additive mask, softmax over keys, weighted sum of V.
    """
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    B, H, Sq, D = q.shape
    Hkv, Skv = k.shape[1], k.shape[2]
    G = H // Hkv
    assert G * Hkv == H
    ke = np.repeat(k, G, axis=1)
    ve = np.repeat(v, G, axis=1)
    s = np.einsum("bhid,bhjd->bhij", q, ke) * np.float64(np.float32(scale))
    if mask is not None:
        m = np.asarray(mask, np.float64)
        kind = {"qk": MASK_QK, "batch_key": MASK_BATCH_KEY}.get(mask_kind, mask_kind)
        s = s + (m[None, None, :, :] if kind == MASK_QK else m[:, None, None, :])
    with np.errstate(invalid="ignore"):
        s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    p = e / e.sum(axis=-1, keepdims=True)
    return np.einsum("bhij,bhjd->bhid", p, ve)


# ---- masks (numpy restatement; the C file holds an independent one) -----------------------------

def mask_causal(n, dtype=np.float32):
    """AttentionMask::causal -- fusor-ml/fusor/src/cache/attention_mask.rs:26-34."""
    i = np.arange(n)[:, None]
    j = np.arange(n)[None, :]
    return np.where(j > i, -np.inf, 0.0).astype(dtype)


def mask_sliding(n, window, dtype=np.float32):
    """MaskCache::create_sliding_window_mask -- fusor-ml/fusor/src/cache/mask_cache.rs:88-103."""
    i = np.arange(n)[:, None]
    j = np.arange(n)[None, :]
    return np.where((i < j) | (j + window <= i), -np.inf, 0.0).astype(dtype)


def get_mask(seq_len, seqlen_offset, window=None, dtype=np.float32):
    """MaskCache::get_mask -- fusor-ml/fusor/src/cache/mask_cache.rs:36-86."""
    if window is not None:
        off = min(seqlen_offset, max(window - seq_len, 0))  # saturating_sub (:45)
        base = mask_sliding(seq_len, window, dtype)
    else:
        off = seqlen_offset
        base = mask_causal(seq_len, dtype)
    if off > 0:
        out = np.zeros((seq_len, off + seq_len), dtype)
        out[:, off:] = base
        return out
    return base


def get_mask_c(seq_len, seqlen_offset, window=None):
    """The C restatement of get_mask (independent of the numpy one above)."""
    L = lib()
    hw, w = (1, int(window)) if window is not None else (0, 0)
    off = L.oracle_get_mask_offset(seq_len, seqlen_offset, hw, w)
    out = np.empty((seq_len, off + seq_len), np.float32)
    L.oracle_get_mask_f32(seq_len, seqlen_offset, hw, w, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)))
    return out


# ---- growable KV cache (numpy restatement) -------------------------------------------------------

class TensorCache:
    """TensorCache::append -- fusor-ml/fusor/src/cache/tensor_cache.rs:48-118.

    parity: PINNED by the reference's tests (tensor_cache.rs:130-186, kv_cache.rs:74-157) and by
    brute force against plain concatenation + truncation.
    """

    def __init__(self, concat_dim, max_sequence_len):
        self.all_data = None
        self.current_seq_len = 0
        self.allocated_seq_len = 0
        self.concat_dim = concat_dim
        self.max_sequence_len = max_sequence_len

    def reset(self):
        self.all_data = None
        self.current_seq_len = 0
        self.allocated_seq_len = 0

    def current_data(self):
        return self.all_data

    def _narrow(self, a, start, length):
        idx = [slice(None)] * a.ndim
        idx[self.concat_dim] = slice(start, start + length)
        return a[tuple(idx)]

    def append(self, v):
        v = np.asarray(v)
        seq_len = v.shape[self.concat_dim]
        required = self.current_seq_len + seq_len
        if required > self.max_sequence_len:  # :55-78
            mx = self.max_sequence_len
            new_start = required - mx
            parts = []
            if self.all_data is not None:
                parts.append(self._narrow(self.all_data, new_start, self.current_seq_len - new_start))
            parts.append(v)
            cat = np.concatenate(parts, axis=self.concat_dim)
            n = cat.shape[self.concat_dim]
            self.all_data = np.ascontiguousarray(self._narrow(cat, n - mx, mx))
            self.current_seq_len = mx
            self.allocated_seq_len = mx
            return self.all_data
        if self.all_data is not None:  # :80-110
            if required > self.allocated_seq_len:
                new_alloc = 1 << (required - 1).bit_length()  # next_power_of_two
                self.allocated_seq_len = new_alloc
                shp = list(v.shape)
                shp[self.concat_dim] = new_alloc - self.current_seq_len
                self.all_data = np.concatenate([self.all_data, np.zeros(shp, v.dtype)], axis=self.concat_dim)
            self._narrow(self.all_data, self.current_seq_len, seq_len)[...] = v
            self.current_seq_len = required
            return self._narrow(self.all_data, 0, self.current_seq_len)
        self.all_data = v.copy()  # :111-116
        self.current_seq_len = seq_len
        self.allocated_seq_len = seq_len
        return self.all_data


class KvCache:
    """KvCache -- fusor-ml/fusor/src/cache/kv_cache.rs:13-68."""

    def __init__(self, concat_dim, max_sequence_len):
        self.key = TensorCache(concat_dim, max_sequence_len)
        self.value = TensorCache(concat_dim, max_sequence_len)

    def reset(self):
        self.key.reset()
        self.value.reset()

    def append(self, k, v):
        return self.key.append(k), self.value.append(v)

    def current_seq_len(self):
        return self.key.current_seq_len


# ---- rotary position embedding (fusor-ml/fusor/src/composite/rope.rs) --------------------------------
# numpy float32 arithmetic rounds once per operation, exactly like the reference's CPU tensor ops
# (mul_, add_, sub_ are separate passes there), so these restatements are bit-level statements of it.

def rope_tables(head_dim, context_length, theta):
    """RopeCache::new (rope.rs:198-221): outer product of positions and 1/theta^(i/dim), then cos/sin, in f32.
    The last bit of cos/sin depends on the libm in use; the rotation itself takes the tables as inputs."""
    th = np.float32(theta)
    inv = np.array([np.float32(1.0) / np.power(th, np.float32(i) / np.float32(head_dim), dtype=np.float32)
                    for i in range(0, head_dim, 2)], np.float32)
    outer = (np.arange(context_length, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float32)
    return np.cos(outer).astype(np.float32), np.sin(outer).astype(np.float32)


def rope(x, cos, sin, start_pos=0):
    """Tensor::rope (rope.rs:46-79) on rows start_pos.. of the tables: x*cos + rotate_half(x)*sin."""
    x = np.asarray(x, np.float32)
    n, d = x.shape[2], x.shape[3]
    c = np.concatenate([cos, cos], 1)[start_pos:start_pos + n][None, None].astype(np.float32)
    s = np.concatenate([sin, sin], 1)[start_pos:start_pos + n][None, None].astype(np.float32)
    h = d // 2
    rot = np.concatenate([-x[..., h:], x[..., :h]], -1)  # rotate_half (rope.rs:10-21)
    return (x * c).astype(np.float32) + (rot * s).astype(np.float32)


def rope_interleaved(x, cos, sin, start_pos=0):
    """Tensor::rope_interleaved (rope.rs:81-137): pairs (2i, 2i+1)."""
    x = np.asarray(x, np.float32)
    n = x.shape[2]
    c = cos[start_pos:start_pos + n][None, None].astype(np.float32)
    s = sin[start_pos:start_pos + n][None, None].astype(np.float32)
    x0, x1 = x[..., 0::2], x[..., 1::2]
    y0 = (x0 * c).astype(np.float32) - (x1 * s).astype(np.float32)
    y1 = (x0 * s).astype(np.float32) + (x1 * c).astype(np.float32)
    out = np.empty_like(x)
    out[..., 0::2], out[..., 1::2] = y0, y1
    return out


def rope_f64(x, cos, sin, start_pos=0, interleaved=False):
    """The same rotation written from the textbook (complex multiplication) in float64."""
    x = np.asarray(x, np.float64)
    n, d = x.shape[2], x.shape[3]
    ang_c = np.asarray(cos, np.float64)[start_pos:start_pos + n][None, None]
    ang_s = np.asarray(sin, np.float64)[start_pos:start_pos + n][None, None]
    z = (x[..., 0::2] + 1j * x[..., 1::2]) if interleaved else (x[..., :d // 2] + 1j * x[..., d // 2:])
    w = z * (ang_c + 1j * ang_s)
    out = np.empty_like(x)
    if interleaved:
        out[..., 0::2], out[..., 1::2] = w.real, w.imag
    else:
        out[..., :d // 2], out[..., d // 2:] = w.real, w.imag
    return out


def rms_norm(x, weight, bias=None, eps=1e-5):
    """RmsNorm::forward_generic_4d -> rms_norm_fused_cpu_impl (fusor-ml/fusor/src/layers/rms_norm.rs:122-133,
    fusor-ml/fusor/src/composite/normalization.rs:351-407) over the last axis, f32, one rounding per op:
    x*x; sum folded left to right from 0 (cpu/src/reduce.rs:752-757); / n; + eps; sqrt; x / rms; * weight; (+ bias).
    The caller rounds the result to the tensor's element type (the cast at rms_norm.rs:132)."""
    x = np.asarray(x, np.float32)
    w = np.asarray(weight, np.float32)
    n = x.shape[-1]
    ss = np.zeros(x.shape[:-1], np.float32)
    for i in range(n):
        ss = (ss + (x[..., i] * x[..., i]).astype(np.float32)).astype(np.float32)
    mean = (ss / np.float32(n)).astype(np.float32)
    rms = np.sqrt((mean + np.float32(eps)).astype(np.float32)).astype(np.float32)
    out = ((x / rms[..., None]).astype(np.float32) * w).astype(np.float32)
    if bias is not None:
        out = (out + np.asarray(bias, np.float32)).astype(np.float32)
    return out


def rms_norm_f64(x, weight, bias=None, eps=1e-5):
    """The textbook definition in float64: x / sqrt(mean(x^2) + eps) * weight + bias."""
    x = np.asarray(x, np.float64)
    out = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + np.float64(np.float32(eps))) * np.asarray(weight, np.float64)
    return out if bias is None else out + np.asarray(bias, np.float64)
