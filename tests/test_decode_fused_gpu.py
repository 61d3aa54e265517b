"""The split-KV decode step that merges its splits inside the main kernel (one launch instead of two).

With 2 to 8 splits per (batch, kv head) and equal lengths, the matrix-core decode kernels number their workgroups so
that the splits of a unit share one XCD's L2; each parks its partial (acc, m, l) there and the last one to arrive merges
them with the arithmetic of the separate merge kernel.  Checked here: the plan says one launch; the result equals the
two-launch form bit for bit (forced by passing the same lengths as a per-sequence array, which that form serves) and
the CPU checker within the gate; unit counts that are not a multiple of the 8 XCDs; calls of different shapes in a row
on one workspace (the arrival counters are never cleared); replays of a recorded call.
"""
import ctypes

import numpy as np
import pytest

import floneum_amd as fa
import oracle
from conftest import TOL_16, TOL_F32, assert_parity
from test_attention_gpu import _analytic_mask, rounded

pytestmark = pytest.mark.gpu


def _normal_qkv(seed, B, H, Hkv, Sq, Skv, D, scale=1.0):
    """Seeded normals (numpy's generator: these caches are tens of millions of elements)."""
    rng = np.random.default_rng(seed)
    return tuple(rng.standard_normal(shp, dtype=np.float32) * np.float32(scale)
                 for shp in ((B, H, Sq, D), (B, Hkv, Skv, D), (B, Hkv, Skv, D)))


def _tol(dtype):
    return TOL_F32 if dtype == fa.F32 else (dict(max_abs=1e-2, rel_l2=5e-3) if dtype == fa.BF16 else TOL_16)


def _fused_and_two_launch(device, dtype, q, k, v, scale, analytic=None, what="", two_launch=True):
    B, Skv = q.shape[0], k.shape[2]
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
    kw = {} if analytic is None else {"analytic": analytic}
    plan = tq.decode_plan(tk, tv, scale, **kw)
    assert plan["is_decode"] == 1 and 2 <= plan["nsplit"] <= 8, f"{what}: {plan}"
    assert plan["kernels"] == 1, f"{what}: the merge was not fused: {plan}"
    out = tq.flash_attention(tk, tv, scale, **kw).to_numpy()
    if two_launch:
        # the same lengths as a per-sequence array: served by the two-launch form, same split
        lens = fa.IntTensor(device, np.full(B, Skv, np.int32))
        plan2 = tq.decode_plan(tk, tv, scale, kv_lens=lens, **kw)
        assert plan2["kernels"] == 2 and (plan2["nsplit"], plan2["chunk"]) == (plan["nsplit"], plan["chunk"]), f"{what}: {plan2}"
        two = tq.flash_attention(tk, tv, scale, kv_lens=lens, **kw).to_numpy()
        assert np.array_equal(out.view(np.uint8), two.view(np.uint8)), f"{what}: fused merge differs from the merge kernel"
    mask = None if analytic is None else _analytic_mask(q.shape[2], Skv, *analytic)
    ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale, mask,
                                 None if mask is None else "qk")
    assert_parity(out, ref, _tol(dtype), what)
    return out


@pytest.mark.parametrize("dtype", [fa.F16, fa.BF16, fa.F32])
@pytest.mark.parametrize("B,H,Hkv,Sq,Skv,D", [
    (16, 32, 8, 1, 4096, 128),    # the benchmark's decode step: 128 units, 4 splits
    (12, 32, 8, 1, 3000, 128),    # 96 units, 6 splits
    (25, 6, 3, 1, 2500, 64),      # 75 units: not a multiple of the 8 XCDs (padding workgroups leave at once)
    (16, 16, 4, 1, 2048, 256),    # one workgroup per CU above head_dim 128
    (16, 32, 8, 4, 4096, 128),    # a multi-token step: 16 columns per unit
    (40, 4, 4, 2, 1100, 96),      # 160 units, 2 columns each
])
def test_fused_merge_equals_the_two_launch_form_and_the_checker(device, dtype, B, H, Hkv, Sq, Skv, D):
    if dtype == fa.F32 and D == 256:
        pytest.skip("f32 at head_dim 256 with four columns per KV head runs on the vector variant (two launches)")
    q, k, v = _normal_qkv(500 + D + B, B, H, Hkv, Sq, Skv, D, 0.5)
    analytic = (True, Skv - Sq, 0) if Sq > 1 else None
    _fused_and_two_launch(device, dtype, q, k, v, D ** -0.5, analytic, f"B{B} H{H}/{Hkv} Sq{Sq} Skv{Skv} D{D}")


def test_fused_merge_with_a_sliding_window_inside_a_longer_cache(device):
    """The visible stretch of the cache is what gets split: a window of 3000 keys at the end of 8192.  (With
    per-sequence lengths the whole cache is planned, so there is no two-launch twin with the same split.)"""
    B, H, Hkv, Skv, D = 16, 16, 4, 8192, 128
    q, k, v = _normal_qkv(520, B, H, Hkv, 1, Skv, D, 0.5)
    _fused_and_two_launch(device, fa.F16, q, k, v, D ** -0.5, (True, Skv - 1, 3000), "window 3000 of 8192", two_launch=False)


def test_fused_merge_calls_of_different_shapes_in_a_row_on_one_workspace(device):
    """The arrival counters in the workspace are never cleared: they carry a mark unique to the call.  Calls with
    different unit counts and split counts follow each other on the device's one workspace, each twice."""
    shapes = [(16, 32, 8, 4096, 128), (24, 8, 4, 1500, 64), (16, 32, 8, 2048, 128), (9, 8, 8, 3333, 128), (16, 32, 8, 4096, 128)]
    first = {}
    for rnd in range(2):
        for i, (B, H, Hkv, Skv, D) in enumerate(shapes):
            q, k, v = _normal_qkv(530 + i, B, H, Hkv, 1, Skv, D, 0.5)
            tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
            assert tq.decode_plan(tk, tv, D ** -0.5)["kernels"] == 1
            out = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
            if rnd == 0:
                ref = oracle.flash_attention(rounded(q, fa.F16), rounded(k, fa.F16), rounded(v, fa.F16), D ** -0.5)
                assert_parity(out, ref, TOL_16, f"shape {i}")
                first[i] = out
            else:
                assert np.array_equal(out.view(np.uint8), first[i].view(np.uint8)), f"shape {i}: second round differs"


def test_fused_merge_replayed_from_a_graph(device):
    """A recorded call is replayed with the mark it was recorded with: the counters of the previous replay hold that
    mark and a finished count, which restarts them.  Every replay equals the eager call, with other decode calls on the
    same workspace in between."""
    device = device.with_new_stream()
    B, H, Hkv, Skv, D = 16, 32, 8, 4096, 128
    q, k, v = _normal_qkv(540, B, H, Hkv, 1, Skv, D, 0.5)
    tq, tk, tv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q, k, v))
    q2, k2, v2 = _normal_qkv(541, 8, 8, 2, 1, 2048, D, 0.5)
    uq, uk, uv = (fa.Tensor.from_numpy(device, a, fa.F16) for a in (q2, k2, v2))
    assert tq.decode_plan(tk, tv, D ** -0.5)["kernels"] == 1
    eager = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
    out = fa.Tensor.empty(device, q.shape, fa.F16)
    with device.capture() as cap:
        tq.flash_attention(tk, tv, D ** -0.5, out=out)
    for rep in range(4):
        fa.check(fa.lib().fhip_memset(device.stream, ctypes.c_void_p(out.buffer.ptr), 0, out.buffer.nbytes))
        cap.graph.launch()
        device.synchronize()
        assert np.array_equal(out.to_numpy().view(np.uint8), eager.view(np.uint8)), f"replay {rep}"
        _ = uq.flash_attention(uk, uv, D ** -0.5).to_numpy()  # another call's marks in the same workspace


def test_fused_merge_on_two_streams_at_once(device):
    """Two host threads, two streams of one device handle, each with a workspace of its own, queue decode steps whose
    splits are merged inside the kernel, back to back and at the same time: the workgroups of both launches share the
    chip.  Every result equals the one computed alone, bit for bit, and later decode calls still succeed (a workgroup
    that found its unit spread over several XCDs would have failed them)."""
    import threading
    second = device.with_new_stream()
    shapes = {0: (16, 32, 8, 4096, 128), 1: (24, 8, 4, 3000, 64)}
    alone, tensors = {}, {}
    for i, dev in ((0, device), (1, second)):
        B, H, Hkv, Skv, D = shapes[i]
        q, k, v = _normal_qkv(560 + i, B, H, Hkv, 1, Skv, D, 0.5)
        tq, tk, tv = (fa.Tensor.from_numpy(dev, a, fa.F16) for a in (q, k, v))
        assert tq.decode_plan(tk, tv, D ** -0.5)["kernels"] == 1
        out = tq.flash_attention(tk, tv, D ** -0.5).to_numpy()
        ref = oracle.flash_attention(rounded(q, fa.F16), rounded(k, fa.F16), rounded(v, fa.F16), D ** -0.5)
        assert_parity(out, ref, TOL_16, f"stream {i}, alone")
        alone[i], tensors[i] = out, (tq, tk, tv, D)
    errors = []
    start = threading.Barrier(2)

    def work(i, dev):
        try:
            tq, tk, tv, D = tensors[i]
            outs = [fa.Tensor.empty(dev, tq.shape, fa.F16) for _ in range(40)]
            start.wait()
            for o in outs:                                   # queued without waiting: the two streams' kernels overlap
                tq.flash_attention(tk, tv, D ** -0.5, out=o)
            for n, o in enumerate(outs):
                if not np.array_equal(o.to_numpy().view(np.uint8), alone[i].view(np.uint8)):
                    raise AssertionError(f"stream {i}, call {n}: differs from the call made alone")
        except BaseException as e:  # noqa: BLE001 - handed to the main thread
            errors.append((i, e))
            start.abort()

    threads = [threading.Thread(target=work, args=(0, device)), threading.Thread(target=work, args=(1, second))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
        assert not t.is_alive()
    assert not errors, f"stream {errors[0][0]}: {errors[0][1]!r}"
    for i, dev in ((0, device), (1, second)):                # the form is still on, and still right
        tq, tk, tv, D = tensors[i]
        assert tq.decode_plan(tk, tv, D ** -0.5)["kernels"] == 1
        assert np.array_equal(tq.flash_attention(tk, tv, D ** -0.5).to_numpy().view(np.uint8), alone[i].view(np.uint8))


def test_fused_merge_seeded_sweep(device):
    """Shapes drawn from a fixed seed among those the merge inside the kernel serves (2 to 8 splits): unit counts that
    are and are not multiples of 8, GQA groups 1 to 8, one to four new rows, head dims of both matrix-core variants,
    all three element types, with and without a sliding window."""
    rng = np.random.default_rng(0xFD5E)
    fused = 0
    for it in range(30):
        dtype = [fa.F16, fa.BF16, fa.F32][it % 3]
        D = int(rng.choice([32, 64, 96, 128, 192, 256]))
        Hkv = int(rng.choice([1, 2, 3, 4, 8]))
        G = int(rng.choice([1, 2, 4, 8]))
        rows = int(rng.choice([1, 1, 2, 4]))
        B = int(rng.integers(64 // Hkv + 1, 160 // Hkv + 2))
        Skv = int(rng.integers(600, 3500))
        window = int(rng.integers(200, Skv)) if it % 4 == 3 else 0
        q, k, v = (rng.standard_normal(shp, dtype=np.float32) * np.float32(0.5)
                   for shp in ((B, Hkv * G, rows, D), (B, Hkv, Skv, D), (B, Hkv, Skv, D)))
        tq, tk, tv = (fa.Tensor.from_numpy(device, a, dtype) for a in (q, k, v))
        analytic = (True, Skv - rows, window) if (rows > 1 or window) else None
        kw = {} if analytic is None else {"analytic": analytic}
        plan = tq.decode_plan(tk, tv, D ** -0.5, **kw)
        if not (plan["is_decode"] and plan["kernels"] == 1 and plan["nsplit"] > 1):
            continue
        fused += 1
        out = tq.flash_attention(tk, tv, D ** -0.5, **kw).to_numpy()
        mask = None if analytic is None else _analytic_mask(rows, Skv, *analytic)
        ref = oracle.flash_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), D ** -0.5, mask,
                                     None if mask is None else "qk")
        assert_parity(out, ref, _tol(dtype), f"it{it} B{B} H{Hkv * G}/{Hkv} rows{rows} Skv{Skv} D{D} window{window} {plan}")
    assert fused >= 12, fused
