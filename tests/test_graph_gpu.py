"""GPU tests of stream capture: library calls recorded into a graph and replayed.

A serving loop is bound by launch cost (a batch-1 decode step is a few launches of ~10 us), so the calls of a
step are meant to be recorded once and replayed.  What changes between replays is the content of device
memory only: the query rows, the int32 key counts a ragged decode call reads, the cache.  Every replay is
checked against the same calls made eagerly on the same state, with eager work and synchronisation between
the replays.
"""
import ctypes

import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, TOL_F32, assert_parity
from test_attention_gpu import _normal_qkv, rounded

pytestmark = pytest.mark.gpu


def _upload(device, t, host):
    host = np.ascontiguousarray(host)
    fa.check(fa.lib().fhip_memcpy_h2d(device.stream, ctypes.c_void_p(t.buffer.ptr), host.ctypes.data_as(ctypes.c_void_p),
                                      host.nbytes))


def _bound_args(device, q, k, v, scale, out, **kw):
    args = q._attn_args(k, v, scale, kw.get("mask"), kw.get("analytic"), kw.get("kv_lens"), None, fa.KERNEL_AUTO, out)
    need = ctypes.c_size_t()
    fa.check(fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(args), device.compute_units, ctypes.byref(need)))
    if need.value:
        ws = fa.Buffer(device, need.value)
        args.workspace, args.workspace_bytes = ws.ptr, need.value
        args._keep.append(ws)
    return args


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16])
def test_decode_step_replayed_with_growing_key_counts(device, dtype):
    """rope(q) + ragged split-KV decode over a fixed cache buffer, recorded once; the key counts and the query change
    between replays."""
    B, H, Hkv, D, Smax = 3, 8, 2, 128, 700
    _, k, v = _normal_qkv(51, B, H, Hkv, 1, Smax, D, 0.5)
    tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (k, v))
    rc = fa.RopeCache(D, 1024, 10000.0, device)
    q_in = fa.Tensor.empty(device, (B, H, 1, D), fa.F32)
    q_rot = fa.Tensor.empty(device, (B, H, 1, D), dtype)
    out = fa.Tensor.empty(device, (B, H, 1, D), dtype)
    lens_t = fa.IntTensor(device, np.array([1, 1, 1], np.int32))
    args = _bound_args(device, q_rot, tk, tv, D ** -0.5, out, kv_lens=lens_t)
    tables = rc._tables(5, False)
    cq, cr = q_in._c4(), q_rot._c4()

    def step():
        fa.check(fa.lib().fhip_rope(device.stream, ctypes.byref(tables), ctypes.byref(cq), fa.F32, ctypes.byref(cr), dtype))
        fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))

    with device.capture() as cap:
        step()
    graph = cap.graph
    tol = TOL_F32 if dtype == fa.F32 else TOL_16
    for it, lens in enumerate(([5, 700, 333], [6, 1, 334], [700, 700, 700], [129, 64, 2])):
        q = _normal_qkv(60 + it, B, H, Hkv, 1, 1, D, 0.5)[0]
        _upload(device, q_in, q)
        _upload(device, lens_t, np.array(lens, np.int32))
        graph.launch()
        replayed = out.to_numpy()
        step()                                    # the same calls, eagerly, on the same state
        eager = out.to_numpy()
        assert np.array_equal(replayed.view(np.uint8), eager.view(np.uint8)), f"replay {it}"
        q_r = rounded(oracle.rope(q, rc.cos_host, rc.sin_host, 5), dtype)
        for b in range(B):
            ref = oracle.flash_attention(q_r[b:b + 1], rounded(k[b:b + 1, :, :lens[b]], dtype),
                                         rounded(v[b:b + 1, :, :lens[b]], dtype), D ** -0.5)
            assert_parity(replayed[b:b + 1], ref, tol, f"replay {it} sequence {b}")


@pytest.mark.parametrize("D", [64, 128])
def test_masked_prefill_replayed(device, D):
    """A prefill call with a mask tensor is several launches: the interval scan and the tiled kernel (which at
    head_dim 64 holds both mask forms), at head_dim 128 also the kernel for masks that are not intervals, plus, under
    capture, a kernel that clears the word the scan marks.  All of it is recorded, and the mask content may change
    between replays, from the interval form to a bias and back.  A replay whose mask is made of intervals again must
    run on the interval form again (a mark left behind by the bias replay would send every later replay to the
    mask-adding form): its result equals the eager call's bit for bit, and the analytic call's."""
    B, H, Hkv, S = 1, 4, 2, 200
    q, k, v = _normal_qkv(52, B, H, Hkv, S, S, D)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F32) for a in (q, k, v))
    tm = fa.Tensor.empty(device, (S, S), fa.F32)
    out = fa.Tensor.empty(device, (B, H, S, D), fa.F32)
    args = _bound_args(device, tq, tk, tv, D ** -0.5, out, mask=(tm, fa.MaskKind.QKMask))
    _upload(device, tm, oracle.get_mask(S, 0))
    with device.capture() as cap:
        fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))
    rng = np.random.default_rng(1)
    bias = rng.normal(0, 1, (S, S)).astype(np.float32)
    bias[:, 150:] = float("-inf")
    causal, window = oracle.get_mask(S, 0), oracle.get_mask(S, 0, 40)
    analytic = {id(causal): (True, 0, 0), id(window): (True, 0, 40)}
    for it, mask in enumerate((causal, bias, window, bias * 2, causal, causal)):
        _upload(device, tm, mask)
        cap.graph.launch()
        got = out.to_numpy()
        ref = oracle.flash_attention(q, k, v, D ** -0.5, mask, "qk")
        assert_parity(got, ref, TOL_F32, f"replay {it}")
        fa.check(fa.lib().fhip_flash_attention(device.stream, ctypes.byref(args)))  # the same call, eagerly
        eager = out.to_numpy()
        assert np.array_equal(got.view(np.uint8), eager.view(np.uint8)), f"replay {it} differs from the eager call"
        if id(mask) in analytic:
            same = tq.flash_attention(tk, tv, D ** -0.5, analytic=analytic[id(mask)]).to_numpy()
            assert np.array_equal(got.view(np.uint8), same.view(np.uint8)), f"replay {it} did not run on the interval form"
        _ = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()   # unrelated eager work between the replays


def test_memset_is_a_kernel_and_replays(device):
    """fhip_memset at odd addresses and sizes, eagerly and recorded into a graph that is replayed over dirtied memory
    (a memset node in a captured graph is not reliable on these machines; the library fills with a kernel)."""
    L = fa.lib()
    n = 5000
    buf = fa.Buffer(device, n)
    host = np.empty(n, np.uint8)

    def dirty():
        src = np.full(n, 0xEE, np.uint8)
        fa.check(L.fhip_memcpy_h2d(device.stream, ctypes.c_void_p(buf.ptr), src.ctypes.data_as(ctypes.c_void_p), n))

    def read():
        fa.check(L.fhip_memcpy_d2h(device.stream, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(buf.ptr), n))
        return host.copy()

    cases = [(0, n, 0x00), (1, 1, 0x7F), (3, 11, 0xAB), (13, 4099, 0x01), (16, 4096, 0xFF), (7, 0, 0x55), (4990, 10, 0x33)]
    for off, size, val in cases:
        dirty()
        fa.check(L.fhip_memset(device.stream, ctypes.c_void_p(buf.ptr + off), val, size))
        want = np.full(n, 0xEE, np.uint8)
        want[off:off + size] = val
        assert np.array_equal(read(), want), (off, size, val)

    with device.capture() as cap:
        for off, size, val in cases[1:5]:
            fa.check(L.fhip_memset(device.stream, ctypes.c_void_p(buf.ptr + off), val, size))
    want = np.full(n, 0xEE, np.uint8)
    for off, size, val in cases[1:5]:
        want[off:off + size] = val
    for _ in range(3):
        dirty()
        device.synchronize()
        cap.graph.launch()
        assert np.array_equal(read(), want)


def test_blocks_freed_after_capture_are_not_reused_while_the_graph_lives(device):
    """The Python mirror caches freed device blocks by size.  A graph holds the pointers its calls recorded, not the
    buffers: a tensor freed after the capture must not be handed to a new tensor while the graph can still be
    replayed (the replay would write into the new owner's memory), and the device's workspace must neither be
    recycled nor grow inside a capture."""
    device = device.with_new_stream()  # a stream, block cache and workspace of its own: no state from other tests
    B, H, Hkv, S, D = 2, 8, 2, 1500, 128
    q, k, v = _normal_qkv(77, B, H, Hkv, 1, S, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    first = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()  # eager: sizes the device's workspace
    ws_before = device.workspace(0)
    with device.capture() as cap:
        out = tq.flash_attention(tk, tv, D ** -0.5)            # the mirror's convenience call: output from the pool
    out_ptr, nbytes = out.buffer.ptr, out.buffer.nbytes
    del out                                                    # back to the mirror, but not for reuse yet
    squatter = fa.Tensor.empty(device, (B, H, 1, D), fa.F16)   # same size: would have received the freed block
    assert squatter.buffer.nbytes == nbytes and squatter.buffer.ptr != out_ptr
    pattern = np.full((B, H, 1, D), 7.0, np.float16)
    _upload(device, squatter, pattern)
    cap.graph.launch()
    device.synchronize()
    assert np.array_equal(squatter.to_numpy(), pattern), "a replay wrote into a tensor allocated after the capture"
    # the replay's own output is still where the graph put it
    host = np.empty((B, H, 1, D), np.float16)
    fa.check(fa.lib().fhip_memcpy_d2h(device.stream, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(out_ptr), host.nbytes))
    assert np.array_equal(host.view(np.uint8), first.view(np.uint8))
    # a block allocated AND freed after the capture was never recorded: it goes back to the cache and is handed out again
    # (a serving loop that keeps one recorded step alive must not grow by what it allocates eagerly per step)
    late = fa.Tensor.empty(device, (3, 5, 7, 64), fa.F16)
    late_ptr, parked_before = late.buffer.ptr, len(device._parked)
    del late
    assert len(device._parked) == parked_before
    again = fa.Tensor.empty(device, (3, 5, 7, 64), fa.F16)
    assert again.buffer.ptr == late_ptr
    del again
    # a larger call while the graph lives: the old workspace is parked, not reused; the replay still works
    k2, v2 = (fa.Tensor.from_numpy(device, np.concatenate([a, a, a, a], 2), fa.F16) for a in (k, v))
    _ = tq.flash_attention(k2, v2, D ** -0.5).to_numpy()
    assert ws_before[0] in device._parked or device.workspace(0)[0] == ws_before[0]
    cap.graph.launch()
    fa.check(fa.lib().fhip_memcpy_d2h(device.stream, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(out_ptr), host.nbytes))
    assert np.array_equal(host.view(np.uint8), first.view(np.uint8))
    # growing the workspace inside a capture is refused (it would allocate and synchronise)
    k3, v3 = (fa.Tensor.from_numpy(device, np.concatenate([a] * 16, 2), fa.F16) for a in (k, v))
    out3 = fa.Tensor.empty(device, (B, H, 1, D), fa.F16)
    with pytest.raises(fa.FhipError, match="inside a capture"):
        with device.capture():
            tq.flash_attention(k3, v3, D ** -0.5, out=out3)
    parked = len(device._parked)
    del cap                                                    # the last graph goes: parked blocks return to the cache
    import gc
    gc.collect()
    assert device._graphs_alive == 0 and (parked == 0 or len(device._parked) < parked)
