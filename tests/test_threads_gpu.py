"""Two host threads, two streams, one GPU: the threading contract of the boundary.

The reference runs one model per thread and shares the device between them
(models/kalosm-llama/src/lib.rs:128-139,213-250: a session's work is spawned onto its own thread).  The header
promises that calls on different streams may be made concurrently from different threads, that the only mutable
state lives in the handles, and that the error text is per thread.  Here two threads share one device handle, each
with its own stream, KV cache and workspace, and run interleaved cache appends and attention calls (prompt, decode
steps, a multi-token step) through the C ABI; every result is compared with the CPU checker and a thread stops at
its first mismatch.  Between steps each thread makes a call that the reference would panic on and checks that the
message it reads back is its own.
"""
import ctypes
import threading

import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, TOL_F32, assert_parity
from test_attention_gpu import rounded

pytestmark = pytest.mark.gpu


def _session(dev, dtype, D, H, Hkv, seed, bad_heads, start, errors, log):
    """One chat session: prompt, then decode steps; appends into its own cache and attends over it."""
    try:
        rng = np.random.default_rng(seed)
        B = 2
        tol = TOL_F32 if dtype == fa.F32 else TOL_16
        cache, ocache = fa.KvCache(2, 4096, dtype, dev), oracle.KvCache(2, 4096)
        masks = fa.MaskCache(dtype)
        pos = 0
        for step, n in enumerate([96] + [1] * 10 + [3] + [1] * 10):
            start.wait()  # both sessions enter every step together: their calls overlap in time
            q = rounded(rng.normal(0, 1, (B, H, n, D)).astype(np.float32), dtype)
            k = rounded(rng.normal(0, 1, (B, Hkv, n, D)).astype(np.float32), dtype)
            v = rounded(rng.normal(0, 1, (B, Hkv, n, D)).astype(np.float32), dtype)
            tq, tk, tv = (fa.Tensor.from_numpy(dev, a, dtype) for a in (q, k, v))
            k_all, v_all = cache.append(dev, tk, tv)
            mask = masks.get_mask(n, pos, None, dev)
            out = tq.flash_attention(k_all, v_all, D ** -0.5, (mask.mask(), fa.MaskKind.QKMask))
            # an invalid call in between: its message must be this thread's, whatever the other thread is doing
            bad_q = fa.Tensor.empty(dev, (B, bad_heads, n, D), dtype)
            try:
                bad_q.flash_attention(k_all, v_all, 1.0)
                raise RuntimeError("the invalid call was accepted")
            except fa.InvalidArgument as e:
                want = f"Number of Q heads ({bad_heads}) must be divisible by number of K/V heads ({Hkv})"
                assert want in str(e), f"thread with {bad_heads} heads read: {e}"
                text = fa.lib().fhip_last_error().decode()
                assert want in text, f"fhip_last_error() on this thread: {text!r}"
            got = out.to_numpy()
            ka, va = ocache.append(k, v)
            ref = oracle.flash_attention(q, np.ascontiguousarray(ka), np.ascontiguousarray(va), D ** -0.5,
                                         oracle.get_mask(n, pos, None), "qk")
            assert_parity(got, ref, tol, f"seed {seed} step {step} (pos {pos}, {n} new rows)")
            pos += n
            log.append((seed, step))
    except BaseException as e:  # noqa: BLE001 - handed to the main thread
        if not isinstance(e, threading.BrokenBarrierError):
            errors.append((seed, e))
        start.abort()


def test_two_threads_two_streams_interleaved_sessions(device):
    second = device.with_new_stream()
    assert second.handle is device.handle and second.stream.value != device.stream.value
    errors, log = [], []
    start = threading.Barrier(2)
    threads = [
        threading.Thread(target=_session, args=(device, fa.F16, 128, 8, 2, 11, 3, start, errors, log)),
        threading.Thread(target=_session, args=(second, fa.F32, 64, 4, 4, 12, 5, start, errors, log)),
    ]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
        assert not t.is_alive(), "a session did not finish"
    assert not errors, f"session with seed {errors[0][0]}: {errors[0][1]!r}"
    assert not start.broken
    # both sessions ran all their steps, and their steps interleaved in time (neither ran start to end alone)
    assert sum(1 for s, _ in log if s == 11) == 22 and sum(1 for s, _ in log if s == 12) == 22
    for i in range(0, 44, 2):  # step by step, in either order
        assert {log[i][0], log[i + 1][0]} == {11, 12} and log[i][1] == log[i + 1][1] == i // 2


def test_error_text_is_per_thread(device):
    """A failure on one thread leaves the other thread's error text alone."""
    L = fa.lib()
    seen = {}

    def fail():
        q = fa.Tensor.empty(device, (1, 3, 4, 32), fa.F32)
        kv = fa.Tensor.empty(device, (1, 2, 4, 32), fa.F32)
        args = q._attn_args(kv, kv, 1.0, None, None, None, None, fa.KERNEL_AUTO, None)
        seen["rc"] = L.fhip_flash_attention_validate(ctypes.byref(args))
        seen["own"] = L.fhip_last_error().decode()

    q = fa.Tensor.empty(device, (1, 4, 4, 32), fa.F32)
    kv = fa.Tensor.empty(device, (1, 2, 4, 32), fa.F32)
    good = q._attn_args(kv, kv, 1.0, None, None, None, None, fa.KERNEL_AUTO, None)
    assert L.fhip_flash_attention_validate(ctypes.byref(good)) == fa.OK
    before = L.fhip_last_error().decode()
    t = threading.Thread(target=fail)
    t.start()
    t.join()
    assert seen["rc"] == fa.ERR_INVALID_ARG and "Number of Q heads (3)" in seen["own"]
    assert L.fhip_last_error().decode() == before
