"""The benchmark's calibration entry point: a register-only matrix-core loop that reports the clock it ran at."""
import ctypes

import numpy as np
import pytest

import floneum_amd as fa

pytestmark = pytest.mark.gpu


def test_mfma_calibration_runs_and_reports_clocks(device):
    L = fa.lib()
    cus = device.compute_units
    nbytes = cus * (256 * 4 + 16)
    scratch = fa.Buffer(device, nbytes)
    host = np.zeros(nbytes, np.uint8)
    for dtype, rand, duty in ((fa.F16, 1, 100), (fa.BF16, 1, 67), (fa.F16, 0, 100)):
        fa.check(L.fhip_memset(device.stream, ctypes.c_void_p(scratch.ptr), 0, nbytes))
        fa.check(L.fhip_calibration_mfma(device.stream, dtype, rand, duty, 200, ctypes.c_void_p(scratch.ptr), nbytes))
        fa.check(L.fhip_memcpy_d2h(device.stream, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(scratch.ptr), nbytes))
        ticks = host[cus * 1024:].view(np.uint64).reshape(cus, 2).astype(np.float64)
        assert (ticks > 0).all(), "every workgroup reports cycles and wall ticks"
        ghz = ticks[:, 0] / ticks[:, 1] * 0.1
        assert ((ghz > 0.3) & (ghz < 2.6)).all(), f"shader clock out of range: {ghz.min():.2f}..{ghz.max():.2f} GHz"
        # 200 rounds of 32 matrix instructions of 32 cycles each, plus the sleeps: at least that many cycles
        assert (ticks[:, 0] >= 200 * 32 * 32).all()
        sink = host[:cus * 1024].view(np.float32)
        assert np.isfinite(sink).all() and (rand or not sink.any())


def test_mfma_calibration_rejects_bad_arguments(device):
    L = fa.lib()
    nbytes = device.compute_units * (256 * 4 + 16)
    scratch = fa.Buffer(device, nbytes)
    p = ctypes.c_void_p(scratch.ptr)
    assert L.fhip_calibration_mfma(device.stream, fa.F32, 1, 100, 10, p, nbytes) == fa.ERR_UNSUPPORTED
    assert L.fhip_calibration_mfma(device.stream, fa.F16, 1, 20, 10, p, nbytes) == fa.ERR_INVALID_ARG
    assert L.fhip_calibration_mfma(device.stream, fa.F16, 1, 100, 0, p, nbytes) == fa.ERR_INVALID_ARG
    assert L.fhip_calibration_mfma(device.stream, fa.F16, 1, 100, 10, p, nbytes - 16) == fa.ERR_WORKSPACE
    assert L.fhip_calibration_mfma(device.stream, fa.F16, 1, 100, 10, None, nbytes) == fa.ERR_INVALID_ARG


def test_read_calibration_runs_and_rejects_bad_arguments(device):
    L = fa.lib()
    n = 8 << 20
    buf, sink = fa.Buffer(device, n), fa.Buffer(device, device.compute_units * 32)
    fa.check(L.fhip_memset(device.stream, ctypes.c_void_p(buf.ptr), 1, n))
    for nbytes in (n, n - 4096 + 16, 16, 0):
        fa.check(L.fhip_calibration_read(device.stream, ctypes.c_void_p(buf.ptr), nbytes, ctypes.c_void_p(sink.ptr),
                                         device.compute_units * 32))
    device.synchronize()
    assert L.fhip_calibration_read(device.stream, ctypes.c_void_p(buf.ptr + 8), n - 16, ctypes.c_void_p(sink.ptr),
                                   device.compute_units * 32) == fa.ERR_WORKSPACE
    assert L.fhip_calibration_read(device.stream, ctypes.c_void_p(buf.ptr), n, ctypes.c_void_p(sink.ptr), 16) == fa.ERR_WORKSPACE
    assert L.fhip_calibration_read(device.stream, None, n, ctypes.c_void_p(sink.ptr), 1 << 20) == fa.ERR_INVALID_ARG


def test_issue_calibration_runs_every_mix_and_rejects_bad_arguments(device):
    """fhip_calibration_issue: steps of one matrix instruction and companions, one wavefront per SIMD.  A step cannot
    take fewer cycles than the matrix pipe is busy with its instruction (32), and companions do not make it shorter."""
    L = fa.lib()
    cus = device.compute_units
    nbytes = cus * (256 * 4 + 16)
    scratch = fa.Buffer(device, nbytes)
    p = ctypes.c_void_p(scratch.ptr)
    host = np.zeros(nbytes, np.uint8)
    rounds = 300
    cycles = []
    for mix in range(13):
        fa.check(L.fhip_memset(device.stream, p, 0, nbytes))
        fa.check(L.fhip_calibration_issue(device.stream, mix, rounds, p, nbytes))
        fa.check(L.fhip_memcpy_d2h(device.stream, host.ctypes.data_as(ctypes.c_void_p), p, nbytes))
        ticks = host[cus * 1024:].view(np.uint64).reshape(cus, 2).astype(np.float64)
        assert (ticks > 0).all(), f"mix {mix}: every workgroup reports cycles and wall ticks"
        assert (ticks[:, 0] >= 0.85 * rounds * 16 * 32).all(), f"mix {mix}: fewer cycles than the matrix instructions take"
        cycles.append(float(np.median(ticks[:, 0])) / (rounds * 16))
    assert cycles[3] > cycles[2] - 2 and cycles[10] > cycles[0], cycles
    assert L.fhip_calibration_issue(device.stream, 13, 10, p, nbytes) == fa.ERR_INVALID_ARG
    assert L.fhip_calibration_issue(device.stream, -1, 10, p, nbytes) == fa.ERR_INVALID_ARG
    assert L.fhip_calibration_issue(device.stream, 0, 0, p, nbytes) == fa.ERR_INVALID_ARG
    assert L.fhip_calibration_issue(device.stream, 0, 10, p, nbytes - 16) == fa.ERR_WORKSPACE
    assert L.fhip_calibration_issue(device.stream, 0, 10, None, nbytes) == fa.ERR_INVALID_ARG
