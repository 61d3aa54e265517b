"""floneum_amd -- MI355X (gfx950) attention backend for fusor-ml, bound through its C ABI.

This module is a thin ctypes binding of ``libfusor_hip.so`` (declared in ``include/fusor_hip.h``)
plus a host-side mirror of the fusor API that sits on the attention path, with the reference's
names and argument meaning:

    Tensor.flash_attention(k, v, scale, mask=(mask, MaskKind.QKMask))
        -> fusor::Tensor<4,D>::flash_attention   fusor-ml/fusor/src/composite/flash_attention.rs:52-73
    MaskKind.{QKMask, BatchKeyMask}               flash_attention.rs:11-19
    AttentionMask.causal(device, seq_len)         fusor-ml/fusor/src/cache/attention_mask.rs:26-46
    MaskCache.get_mask(seq_len, seqlen_offset, sliding_window_size, device)
                                                  fusor-ml/fusor/src/cache/mask_cache.rs:36-86
    KvCache(concat_dim, max_sequence_len).append(device, k, v)
                                                  fusor-ml/fusor/src/cache/kv_cache.rs:13-68

All arithmetic happens in the HIP library; there is no CPU fallback.  If the shared library is
missing the import of :func:`lib` raises.
"""
import ctypes
import enum
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfusor_hip.so")

F32, F16, BF16 = 0, 1, 2
_DTYPE_BYTES = {F32: 4, F16: 2, BF16: 2}

KERNEL_AUTO, KERNEL_GENERIC, KERNEL_PREFILL_MFMA, KERNEL_PREFILL_F32, KERNEL_DECODE_SPLITKV = 0, 1, 2, 3, 4
KERNEL_PREFILL_MFMA_ROWS64 = 5  # only as force_kernel: the tiled 16-bit kernel's 64-rows-per-wavefront form at head_dim 128
KERNEL_NAMES = {1: "generic", 2: "prefill_mfma", 3: "prefill_f32", 4: "decode_splitkv", 5: "prefill_mfma_rows64"}

OK, ERR_INVALID_ARG, ERR_UNSUPPORTED, ERR_HIP, ERR_WORKSPACE = 0, 1, 2, 3, 4
NOALLOC_WORKSPACE_BYTES = 32 << 20  # FHIP_NOALLOC_WORKSPACE_BYTES


class FhipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"fusor_hip status {code}: {message}")
        self.code = code
        self.message = message


class InvalidArgument(FhipError, AssertionError):
    """What the reference raises as an `assert!` panic (shape / divisibility errors)."""


class CTensor4(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("offset", ctypes.c_uint64), ("shape", ctypes.c_uint32 * 4),
                ("stride", ctypes.c_int64 * 4)]


class CTensor2(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("offset", ctypes.c_uint64), ("shape", ctypes.c_uint32 * 2),
                ("stride", ctypes.c_int64 * 2)]


class CAnalyticMask(ctypes.Structure):
    _fields_ = [("enabled", ctypes.c_int32), ("causal", ctypes.c_int32), ("q_pos_offset", ctypes.c_int64),
                ("window", ctypes.c_int64)]


class CAttnArgs(ctypes.Structure):
    _fields_ = [("q", CTensor4), ("k", CTensor4), ("v", CTensor4), ("out", CTensor4),
                ("dtype", ctypes.c_int), ("out_dtype", ctypes.c_int), ("scale", ctypes.c_float),
                ("mask_kind", ctypes.c_int), ("mask", CTensor2), ("analytic", CAnalyticMask),
                ("kv_lens", ctypes.c_void_p), ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
                ("force_kernel", ctypes.c_int32), ("main_kernel_done", ctypes.c_void_p),
                ("main_kernel_start", ctypes.c_void_p), ("mask_intervals", ctypes.c_void_p)]


class CDecodePlanInfo(ctypes.Structure):
    _fields_ = [("is_decode", ctypes.c_int32), ("nsplit", ctypes.c_int32), ("chunk", ctypes.c_int32),
                ("wavefronts", ctypes.c_int32), ("kernels", ctypes.c_int32)]


class CDeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 64), ("compute_units", ctypes.c_int32),
                ("wavefront_size", ctypes.c_int32), ("clock_khz", ctypes.c_int32),
                ("memory_clock_khz", ctypes.c_int32), ("memory_bus_bits", ctypes.c_int32),
                ("total_memory", ctypes.c_uint64), ("lds_per_cu", ctypes.c_uint64), ("l2_bytes", ctypes.c_uint64)]


# every symbol include/fusor_hip.h declares: name -> (restype, argtypes)
_P = ctypes.c_void_p
_PP = ctypes.POINTER(ctypes.c_void_p)
class CRopeTables(ctypes.Structure):
    _fields_ = [("cos", ctypes.c_void_p), ("sin", ctypes.c_void_p), ("table_rows", ctypes.c_uint64),
                ("start_pos", ctypes.c_uint64), ("interleaved", ctypes.c_int32)]


class CRmsNorm(ctypes.Structure):
    _fields_ = [("weight", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("dtype", ctypes.c_int), ("eps", ctypes.c_float)]


SYMBOLS = {
    "fhip_last_error": (ctypes.c_char_p, []),
    "fhip_version": (ctypes.c_char_p, []),
    "fhip_device_count": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int32)]),
    "fhip_device_create": (ctypes.c_int, [ctypes.c_int32, _PP]),
    "fhip_device_destroy": (ctypes.c_int, [_P]),
    "fhip_device_get_info": (ctypes.c_int, [_P, ctypes.POINTER(CDeviceInfo)]),
    "fhip_stream_create": (ctypes.c_int, [_P, _PP]),
    "fhip_stream_destroy": (ctypes.c_int, [_P]),
    "fhip_stream_synchronize": (ctypes.c_int, [_P]),
    "fhip_malloc": (ctypes.c_int, [_P, ctypes.c_size_t, _PP]),
    "fhip_free": (ctypes.c_int, [_P, _P]),
    "fhip_memcpy_h2d": (ctypes.c_int, [_P, _P, _P, ctypes.c_size_t]),
    "fhip_memcpy_d2h": (ctypes.c_int, [_P, _P, _P, ctypes.c_size_t]),
    "fhip_memcpy_d2d": (ctypes.c_int, [_P, _P, _P, ctypes.c_size_t]),
    "fhip_memset": (ctypes.c_int, [_P, _P, ctypes.c_int, ctypes.c_size_t]),
    "fhip_event_create": (ctypes.c_int, [_P, _PP]),
    "fhip_event_destroy": (ctypes.c_int, [_P]),
    "fhip_event_record": (ctypes.c_int, [_P, _P]),
    "fhip_event_synchronize": (ctypes.c_int, [_P]),
    "fhip_event_elapsed_ms": (ctypes.c_int, [_P, _P, ctypes.POINTER(ctypes.c_float)]),
    "fhip_flash_attention_validate": (ctypes.c_int, [ctypes.POINTER(CAttnArgs)]),
    "fhip_flash_attention_select": (ctypes.c_int, [ctypes.POINTER(CAttnArgs), ctypes.POINTER(ctypes.c_int32)]),
    "fhip_flash_attention_workspace_bytes": (ctypes.c_int, [ctypes.POINTER(CAttnArgs), ctypes.c_int32,
                                                            ctypes.POINTER(ctypes.c_size_t)]),
    "fhip_flash_attention_decode_plan": (ctypes.c_int, [_P, ctypes.POINTER(CAttnArgs), ctypes.POINTER(CDecodePlanInfo)]),
    "fhip_flash_attention": (ctypes.c_int, [_P, ctypes.POINTER(CAttnArgs)]),
    "fhip_flash_attention_noalloc": (ctypes.c_int, [_P, ctypes.POINTER(CAttnArgs)]),
    "fhip_calibration_mfma": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, _P, ctypes.c_size_t]),
    "fhip_calibration_issue": (ctypes.c_int, [_P, ctypes.c_int32, ctypes.c_int32, _P, ctypes.c_size_t]),
    "fhip_calibration_xcd_map": (ctypes.c_int, [_P, ctypes.c_uint32, _P, ctypes.c_size_t]),
    "fhip_calibration_read": (ctypes.c_int, [_P, _P, ctypes.c_size_t, _P, ctypes.c_size_t]),
    "fhip_mask_causal": (ctypes.c_int, [ctypes.c_int, ctypes.c_uint32, _P]),
    "fhip_mask_sliding_window": (ctypes.c_int, [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64, _P]),
    "fhip_mask_get_mask_shape": (ctypes.c_int, [ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int32, ctypes.c_uint64,
                                                ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint64)]),
    "fhip_mask_get_mask": (ctypes.c_int, [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int32,
                                          ctypes.c_uint64, _P]),
    "fhip_mask_intervals_bytes": (ctypes.c_int, [ctypes.c_uint32, ctypes.POINTER(ctypes.c_size_t)]),
    "fhip_mask_intervals": (ctypes.c_int, [_P, ctypes.POINTER(CTensor2), ctypes.c_int, _P, ctypes.c_size_t]),
    "fhip_mask_get_analytic": (ctypes.c_int, [ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int32, ctypes.c_uint64,
                                              ctypes.POINTER(CAnalyticMask)]),
    "fhip_kv_cache_create": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_uint64, _PP]),
    "fhip_kv_cache_destroy": (ctypes.c_int, [_P]),
    "fhip_kv_cache_reset": (ctypes.c_int, [_P]),
    "fhip_kv_cache_current_seq_len": (ctypes.c_int, [_P, ctypes.POINTER(ctypes.c_uint64)]),
    "fhip_kv_cache_allocated_seq_len": (ctypes.c_int, [_P, ctypes.POINTER(ctypes.c_uint64)]),
    "fhip_kv_cache_append": (ctypes.c_int, [_P, _P, ctypes.POINTER(CTensor4), ctypes.POINTER(CTensor4),
                                            ctypes.POINTER(CTensor4), ctypes.POINTER(CTensor4)]),
    "fhip_rope": (ctypes.c_int, [_P, ctypes.POINTER(CRopeTables), ctypes.POINTER(CTensor4), ctypes.c_int,
                                 ctypes.POINTER(CTensor4), ctypes.c_int]),
    "fhip_kv_cache_rope_append": (ctypes.c_int, [_P, _P, ctypes.POINTER(CRopeTables), ctypes.POINTER(CTensor4),
                                                 ctypes.POINTER(CTensor4), ctypes.c_int, ctypes.POINTER(CTensor4),
                                                 ctypes.POINTER(CTensor4)]),
    "fhip_kv_cache_qkv_rope_append": (ctypes.c_int, [_P, _P, ctypes.POINTER(CRmsNorm), ctypes.POINTER(CRmsNorm),
                                                     ctypes.POINTER(CRopeTables), ctypes.POINTER(CTensor4), ctypes.c_int,
                                                     ctypes.POINTER(CTensor4), ctypes.c_int, ctypes.POINTER(CTensor4),
                                                     ctypes.POINTER(CTensor4), ctypes.c_int, ctypes.POINTER(CTensor4),
                                                     ctypes.POINTER(CTensor4)]),
    "fhip_stream_begin_capture": (ctypes.c_int, [_P]),
    "fhip_stream_end_capture": (ctypes.c_int, [_P, _PP]),
    "fhip_graph_launch": (ctypes.c_int, [_P, _P]),
    "fhip_graph_destroy": (ctypes.c_int, [_P]),
    "fhip_mask_get_mask_device": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int32,
                                                 ctypes.c_uint64, _P]),
    "fhip_norm_rope": (ctypes.c_int, [_P, ctypes.POINTER(CRmsNorm), ctypes.POINTER(CRopeTables), ctypes.POINTER(CTensor4),
                                      ctypes.c_int, ctypes.POINTER(CTensor4), ctypes.c_int]),
    "fhip_kv_cache_norm_rope_append": (ctypes.c_int, [_P, _P, ctypes.POINTER(CRmsNorm), ctypes.POINTER(CRopeTables),
                                                      ctypes.POINTER(CTensor4), ctypes.POINTER(CTensor4), ctypes.c_int,
                                                      ctypes.POINTER(CTensor4), ctypes.POINTER(CTensor4)]),
}

_LIB = None


def lib():
    """The loaded C-ABI library.  Raises if it has not been built: there is no fallback path."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: run `python -m floneum_amd.build` "
                              "(or __graft_entry__.build()) first; there is no CPU fallback")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = L
    return _LIB


def check(code):
    if code != OK:
        msg = lib().fhip_last_error().decode("utf-8", "replace")
        if code == ERR_INVALID_ARG:
            raise InvalidArgument(code, msg)
        raise FhipError(code, msg)


# ---- numpy <-> element types -----------------------------------------------------------------------

def np_dtype(dtype):
    return {F32: np.float32, F16: np.float16, BF16: np.uint16}[dtype]


def f32_to_bf16_bits(a):
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, (u >> 16) | 0x40, rounded).astype(np.uint16)


def bf16_bits_to_f32(a):
    return (np.ascontiguousarray(a, np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---- device / stream / buffers ---------------------------------------------------------------------

class Device:
    """A HIP device plus one stream.  Mirrors what fusor's `Device::Gpu` carries for WGPU
    (fusor-ml/fusor/src/device.rs:39-45, fusor-ml/core/src/device.rs)."""

    _default = None

    def __init__(self, ordinal=0, handle=None):
        L = lib()
        if handle is None:
            handle = ctypes.c_void_p()
            check(L.fhip_device_create(ordinal, ctypes.byref(handle)))
        self.handle = handle
        s = ctypes.c_void_p()
        check(L.fhip_stream_create(self.handle, ctypes.byref(s)))
        self.stream = s
        info = CDeviceInfo()
        check(L.fhip_device_get_info(self.handle, ctypes.byref(info)))
        self.info = info
        self.compute_units = info.compute_units
        self.name = info.name.decode()
        self.arch = info.arch.decode()
        self._workspace = None
        self._workspace_bytes = 0
        self._pool, self._sizes, self._pooled = {}, {}, 0  # cached free blocks by size, block sizes, bytes cached
        # A recorded graph keeps the POINTERS of the buffers and of the workspace its calls used, not the buffers.
        # The blocks a capture may have recorded (those alive when it opened or allocated while it was open) are
        # `_pinned`: freed while a capture is open or a Graph of this device is alive, they are parked instead of
        # being handed out again (a replay would overwrite their new owner's data).  Blocks allocated after the
        # capture closed are not pinned and return to the cache as usual.  The workspace is neither recycled nor
        # grown under a capture.
        self._capturing, self._graphs_alive, self._parked = False, 0, []
        self._live, self._pinned = set(), set()

    @classmethod
    def default(cls):
        if cls._default is None:
            cls._default = cls(0)
        return cls._default

    def with_new_stream(self):
        """The same device handle with a stream, allocation cache and workspace of its own: what a second host
        thread uses (one stream and one workspace belong to one thread at a time)."""
        return Device(handle=self.handle)

    @staticmethod
    def count():
        n = ctypes.c_int32()
        rc = lib().fhip_device_count(ctypes.byref(n))
        return n.value if rc == OK else 0

    # Freed blocks are kept by size and handed out again, as the reference's device keeps an allocation cache
    # (fusor-ml/core/src/device.rs:305-354): hipMalloc / hipFree cost tens of microseconds and hipFree waits for
    # the device.  Safe because this object has a single stream: a reused block is only touched by work queued
    # after the work of its previous owner.
    _CACHE_LIMIT = 1 << 30

    def malloc(self, nbytes):
        size = (max(int(nbytes), 1) + 255) & ~255
        free_list = self._pool.get(size)
        if free_list:
            self._pooled -= size
            ptr = free_list.pop()
        else:
            p = ctypes.c_void_p()
            check(lib().fhip_malloc(self.handle, size, ctypes.byref(p)))
            self._sizes[p.value] = size
            ptr = p.value
        self._live.add(ptr)
        if self._capturing:
            self._pinned.add(ptr)
        return ptr

    def free(self, ptr):
        if self._capturing or (self._graphs_alive > 0 and ptr in self._pinned):
            self._parked.append(ptr)
            return
        self._live.discard(ptr)
        size = self._sizes.get(ptr)
        if size is not None and self._pooled + size <= self._CACHE_LIMIT:
            self._pool.setdefault(size, []).append(ptr)
            self._pooled += size
            return
        self._sizes.pop(ptr, None)
        check(lib().fhip_free(self.handle, ctypes.c_void_p(ptr)))

    def _graph_gone(self):
        self._graphs_alive -= 1
        if self._graphs_alive == 0 and not self._capturing:
            parked, self._parked = self._parked, []
            self._pinned = set()
            for ptr in parked:
                self.free(ptr)

    def release_cached_memory(self):
        """Give the cached blocks back to the driver."""
        for ptrs in self._pool.values():
            for ptr in ptrs:
                self._sizes.pop(ptr, None)
                check(lib().fhip_free(self.handle, ctypes.c_void_p(ptr)))
        self._pool, self._pooled = {}, 0

    def synchronize(self):
        check(lib().fhip_stream_synchronize(self.stream))

    def capture(self):
        """Context manager: library calls made inside are recorded into a Graph instead of running."""
        return _Capture(self)

    def workspace(self, nbytes):
        """A grow-only scratch buffer owned by the device object (the caller of the C ABI owns the
        workspace; this is the Python caller's)."""
        if nbytes > self._workspace_bytes:
            if self._capturing:
                raise FhipError(ERR_WORKSPACE, f"the workspace would have to grow to {nbytes} bytes inside a capture "
                                "(allocation and synchronisation are not recordable): run the call once eagerly first")
            if self._workspace:
                if self._graphs_alive == 0:
                    self.synchronize()
                self.free(self._workspace)  # parked while a graph that recorded it is alive
            self._workspace = self.malloc(nbytes)
            self._workspace_bytes = nbytes
        return self._workspace, self._workspace_bytes


class Graph:
    """A recorded sequence of library calls (fhip_graph): launch() replays it with one submission."""

    def __init__(self, device, handle):
        self.device, self.handle = device, handle
        device._graphs_alive += 1

    def launch(self):
        check(lib().fhip_graph_launch(self.handle, self.device.stream))

    def __del__(self):
        try:
            if self.handle:
                lib().fhip_graph_destroy(self.handle)
                self.handle = None
                self.device._graph_gone()
        except Exception:
            pass


class _Capture:
    def __init__(self, device):
        self.device, self.graph = device, None

    def __enter__(self):
        check(lib().fhip_stream_begin_capture(self.device.stream))
        self.device._capturing = True
        self.device._pinned |= self.device._live
        return self

    def __exit__(self, exc_type, exc, tb):
        h = ctypes.c_void_p()
        rc = lib().fhip_stream_end_capture(self.device.stream, ctypes.byref(h))
        self.device._capturing = False
        if exc_type is None:
            check(rc)
            self.graph = Graph(self.device, h)
        else:
            if rc == OK and h:
                lib().fhip_graph_destroy(h)  # the body raised: what was recorded so far is dropped
            if self.device._graphs_alive == 0:
                self.device._graphs_alive = 1  # hand the blocks parked during the failed capture back
                self.device._graph_gone()
        return False


class Buffer:
    """Owning handle of one device allocation (freed with the last tensor that views it)."""

    def __init__(self, device, nbytes):
        self.device = device
        self.nbytes = nbytes
        self.ptr = device.malloc(max(nbytes, 1))

    def __del__(self):
        try:
            if self.ptr:
                self.device.free(self.ptr)
                self.ptr = None
        except Exception:
            pass


class _View:
    """Non-owning device memory (e.g. KV-cache storage owned by the C library)."""

    def __init__(self, device, ptr, keepalive=None):
        self.device = device
        self.ptr = ptr
        self.keepalive = keepalive


def _contig_strides(shape):
    st, acc = [], 1
    for n in reversed(shape):
        st.append(acc)
        acc *= n
    return tuple(reversed(st))


class MaskKind(enum.IntEnum):
    """fusor::MaskKind (flash_attention.rs:11-19)."""
    QKMask = 1
    BatchKeyMask = 2


class Tensor:
    """A strided view of device memory: {buffer, offset, shape, strides} in element units, the
    layout contract of fusor tensors (fusor-ml/types/src/layout.rs:88-129)."""

    def __init__(self, buffer, dtype, shape, strides=None, offset=0):
        self.buffer = buffer
        self.dtype = dtype
        self.shape = tuple(int(x) for x in shape)
        self.strides = tuple(int(x) for x in (strides if strides is not None else _contig_strides(self.shape)))
        self.offset = int(offset)

    # -- construction / readback ------------------------------------------------------------------
    @property
    def device(self):
        return self.buffer.device

    @classmethod
    def empty(cls, device, shape, dtype):
        n = int(np.prod(shape)) if len(shape) else 1
        return cls(Buffer(device, n * _DTYPE_BYTES[dtype]), dtype, shape)

    @classmethod
    def from_numpy(cls, device, array, dtype=None):
        """Uploads a host array.  float32 -> F32, float16 -> F16, uint16 + dtype=BF16 -> bf16 bits;
        a float32 array with dtype=F16/BF16 is rounded to nearest even first."""
        a = np.asarray(array)
        if dtype is None:
            dtype = {np.dtype(np.float32): F32, np.dtype(np.float16): F16}[a.dtype]
        if dtype == F32:
            host = np.ascontiguousarray(a, np.float32)
        elif dtype == F16:
            host = np.ascontiguousarray(a.astype(np.float16))
        else:
            host = np.ascontiguousarray(a if a.dtype == np.uint16 else f32_to_bf16_bits(a))
        t = cls.empty(device, host.shape, dtype)
        if host.nbytes:
            check(lib().fhip_memcpy_h2d(device.stream, ctypes.c_void_p(t.buffer.ptr),
                                        host.ctypes.data_as(ctypes.c_void_p), host.nbytes))
        return t

    def _span(self):
        lo = hi = self.offset
        for n, s in zip(self.shape, self.strides):
            if n == 0:
                return self.offset, self.offset
            if s >= 0:
                hi += (n - 1) * s
            else:
                lo += (n - 1) * s
        return lo, hi + 1

    def to_numpy(self):
        """Readback (the reference's `as_slice().await`): synchronises the stream.  bf16 comes back
        widened to float32."""
        eb = _DTYPE_BYTES[self.dtype]
        lo, hi = self._span()
        raw = np.empty(hi - lo, np_dtype(self.dtype))
        if raw.size:
            check(lib().fhip_memcpy_d2h(self.device.stream, raw.ctypes.data_as(ctypes.c_void_p),
                                        ctypes.c_void_p(self.buffer.ptr + lo * eb), raw.nbytes))
        view = np.lib.stride_tricks.as_strided(raw[self.offset - lo:], self.shape, tuple(s * eb for s in self.strides))
        out = np.array(view)
        return bf16_bits_to_f32(out) if self.dtype == BF16 else out

    # -- layout ops: never copy (fusor-ml/core/src/map_layout.rs:34-51) ----------------------------
    def transpose(self, a, b):
        shp, st = list(self.shape), list(self.strides)
        shp[a], shp[b] = shp[b], shp[a]
        st[a], st[b] = st[b], st[a]
        return Tensor(self.buffer, self.dtype, shp, st, self.offset)

    def narrow(self, dim, start, length):
        assert 0 <= start and start + length <= self.shape[dim]
        shp = list(self.shape)
        shp[dim] = length
        return Tensor(self.buffer, self.dtype, shp, self.strides, self.offset + start * self.strides[dim])

    def broadcast_to(self, shape):
        """Layout::broadcast_to (fusor-ml/types/src/layout.rs): dimensions of size 1 repeat with stride 0."""
        assert len(shape) == len(self.shape)
        st = []
        for have, want, stride in zip(self.shape, shape, self.strides):
            assert have == want or have == 1, f"cannot broadcast {self.shape} to {tuple(shape)}"
            st.append(stride if have == want else 0)
        return Tensor(self.buffer, self.dtype, shape, st, self.offset)

    def is_contiguous(self):
        return self.strides == _contig_strides(self.shape)

    def reshape(self, shape):
        assert self.is_contiguous(), "reshape of a strided view would copy; not part of this path"
        assert int(np.prod(shape)) == int(np.prod(self.shape))
        return Tensor(self.buffer, self.dtype, shape, None, self.offset)

    def _c4(self):
        assert len(self.shape) == 4
        t = CTensor4()
        t.ptr = self.buffer.ptr
        t.offset = self.offset
        t.shape[:] = self.shape
        t.stride[:] = self.strides
        return t

    def _c2(self):
        assert len(self.shape) == 2
        t = CTensor2()
        t.ptr = self.buffer.ptr
        t.offset = self.offset
        t.shape[:] = self.shape
        t.stride[:] = self.strides
        return t

    # -- the operator -------------------------------------------------------------------------------
    def flash_attention(self, k, v, scale, mask=None, *, analytic=None, kv_lens=None, out_dtype=None,
                        force_kernel=KERNEL_AUTO, out=None):
        """fusor::Tensor<4,D>::flash_attention(&self, k, v, scale, mask) -> Self.

        self [B,H,Sq,D]; k, v [B,Hkv,Skv,D]; mask = None or (Tensor<2>, MaskKind).  Keyword-only
        arguments are the C ABI's extensions: `analytic` = (causal, q_pos_offset, window) or an
        AnalyticMask from MaskCache.get_analytic; `kv_lens` = device int32 [B] tensor of valid key
        counts; `out_dtype` F32 for 16-bit inputs.  Raises InvalidArgument (an AssertionError)
        where the reference panics."""
        args = self._attn_args(k, v, scale, mask, analytic, kv_lens, out_dtype, force_kernel, out)
        L = lib()
        dev = self.device
        need = ctypes.c_size_t()
        check(L.fhip_flash_attention_workspace_bytes(ctypes.byref(args), dev.compute_units, ctypes.byref(need)))
        if need.value:
            ws, nb = dev.workspace(need.value)
            args.workspace = ws
            args.workspace_bytes = nb
        check(L.fhip_flash_attention(dev.stream, ctypes.byref(args)))
        return args._out_tensor

    def flash_attention_noalloc(self, k, v, scale, out, mask=None, *, analytic=None, kv_lens=None,
                                force_kernel=KERNEL_AUTO):
        """flash_attention into `out` on the library's own fixed workspace (fhip_flash_attention_noalloc): nothing
        is allocated by the call, here or in the library."""
        args = self._attn_args(k, v, scale, mask, analytic, kv_lens, out.dtype, force_kernel, out)
        check(lib().fhip_flash_attention_noalloc(self.device.stream, ctypes.byref(args)))
        return out

    def _attn_args(self, k, v, scale, mask, analytic, kv_lens, out_dtype, force_kernel, out):
        if not (k.device is self.device and v.device is self.device):
            raise AssertionError("Cannot mix tensors of different devices")  # fusor lib.rs:265
        if len(self.shape) != 4 or len(k.shape) != 4 or len(v.shape) != 4:
            raise InvalidArgument(ERR_INVALID_ARG, "flash_attention takes rank-4 tensors")
        if not (k.dtype == self.dtype and v.dtype == self.dtype):
            raise InvalidArgument(ERR_INVALID_ARG, "q, k, v must share one element type")
        odt = self.dtype if out_dtype is None else out_dtype
        if out is None:
            out = Tensor.empty(self.device, self.shape, odt)  # fresh, contiguous, Q's shape (core :505-507)
        args = CAttnArgs()
        args.q, args.k, args.v, args.out = self._c4(), k._c4(), v._c4(), out._c4()
        args.dtype, args.out_dtype = self.dtype, odt
        args.scale = float(np.float32(scale))
        keep = [out]
        if mask is not None:
            m, kind, *table = mask  # (tensor, kind) or (tensor, kind, MaskIntervals of that tensor)
            if table:
                args.mask_intervals = table[0].buffer.ptr
                keep.append(table[0])
            if m.device is not self.device:
                raise AssertionError("Mask must be on the same device as other tensors")  # fusor :64
            if m.dtype != self.dtype:
                raise InvalidArgument(ERR_INVALID_ARG, "mask must have the element type of q")
            args.mask = m._c2()
            args.mask_kind = int(kind)
            keep.append(m)
        if analytic is not None:
            if isinstance(analytic, CAnalyticMask):
                args.analytic = analytic
            else:
                causal, off, window = analytic
                args.analytic.enabled = 1
                args.analytic.causal = 1 if causal else 0
                args.analytic.q_pos_offset = int(off)
                args.analytic.window = int(window or 0)
        if kv_lens is not None:
            assert kv_lens.dtype == "i32" and kv_lens.shape == (self.shape[0],)
            args.kv_lens = kv_lens.buffer.ptr + kv_lens.offset * 4
            keep.append(kv_lens)
        args.force_kernel = int(force_kernel)
        args._out_tensor = out
        args._keep = keep
        return args

    def selected_kernel(self, k, v, scale, mask=None, **kw):
        args = self._attn_args(k, v, scale, mask, kw.get("analytic"), kw.get("kv_lens"), kw.get("out_dtype"),
                               kw.get("force_kernel", KERNEL_AUTO), kw.get("out"))
        kid = ctypes.c_int32()
        check(lib().fhip_flash_attention_select(ctypes.byref(args), ctypes.byref(kid)))
        return kid.value


    def decode_plan(self, k, v, scale, mask=None, **kw):
        """How the call would run on the split-KV decode kernels: dict(is_decode, nsplit, chunk, wavefronts, kernels)."""
        args = self._attn_args(k, v, scale, mask, kw.get("analytic"), kw.get("kv_lens"), kw.get("out_dtype"),
                               kw.get("force_kernel", KERNEL_AUTO), kw.get("out"))
        info = CDecodePlanInfo()
        check(lib().fhip_flash_attention_decode_plan(self.buffer.device.stream, ctypes.byref(args), ctypes.byref(info)))
        return {name: getattr(info, name) for name, _ in CDecodePlanInfo._fields_}


class IntTensor:
    """Device int32 vector (per-batch key counts)."""
    dtype = "i32"

    def __init__(self, device, values):
        host = np.ascontiguousarray(values, np.int32)
        self.buffer = Buffer(device, host.nbytes)
        self.shape = host.shape
        self.offset = 0
        check(lib().fhip_memcpy_h2d(device.stream, ctypes.c_void_p(self.buffer.ptr),
                                    host.ctypes.data_as(ctypes.c_void_p), host.nbytes))


# ---- masks --------------------------------------------------------------------------------------------

def _host_mask(fn, dtype, rows, cols, *a):
    host = np.empty((rows, cols), np_dtype(dtype))
    check(fn(dtype, *a, host.ctypes.data_as(ctypes.c_void_p)))
    return host


class MaskIntervals:
    """The interval form of a mask tensor (fhip_mask_intervals), computed once for a mask that does not change and
    passed with it as the third element of flash_attention's mask tuple: the call then skips its scan of the mask."""

    def __init__(self, mask):
        need = ctypes.c_size_t()
        check(lib().fhip_mask_intervals_bytes(mask.shape[0], ctypes.byref(need)))
        self.buffer = Buffer(mask.device, need.value)
        cm = mask._c2()
        check(lib().fhip_mask_intervals(mask.device.stream, ctypes.byref(cm), mask.dtype, ctypes.c_void_p(self.buffer.ptr),
                                        need.value))
        self.mask = mask  # the table describes this view and lives no longer than it


class AttentionMask:
    """fusor::cache::AttentionMask (attention_mask.rs:9-83): wraps the 2-D additive mask tensor."""

    def __init__(self, mask, host=None, analytic=None):
        self._mask = mask
        self.host = host          # the same values on the host (numpy), kept for inspection
        self.analytic = analytic  # CAnalyticMask equal to this mask, when it was built by MaskCache
        self._intervals = None

    def intervals(self):
        """The mask's interval table, computed on first use and kept with the mask (which never changes)."""
        if self._intervals is None:
            self._intervals = MaskIntervals(self._mask)
        return self._intervals

    @classmethod
    def causal(cls, device, seq_len, dtype=F32):
        host = _host_mask(lib().fhip_mask_causal, dtype, seq_len, seq_len, seq_len)
        am = CAnalyticMask(1, 1, 0, 0)
        return cls(Tensor.from_numpy(device, host, dtype) if device is not None else None, host, am)

    def mask(self):
        return self._mask


class MaskCache:
    """fusor::cache::MaskCache (mask_cache.rs:9-116): base masks cached by (seq_len, window)."""

    def __init__(self, dtype=F32):
        self.dtype = dtype
        self.masks = {}

    def get_mask(self, seq_len, seqlen_offset, sliding_window_size, device):
        L = lib()
        has_w = sliding_window_size is not None
        w = int(sliding_window_size) if has_w else 0
        rows, cols = ctypes.c_uint32(), ctypes.c_uint64()
        check(L.fhip_mask_get_mask_shape(seq_len, seqlen_offset, int(has_w), w, ctypes.byref(rows), ctypes.byref(cols)))
        off = cols.value - seq_len
        key = (seq_len, sliding_window_size)
        base = self.masks.get(key)
        if base is None:
            if has_w:
                host = _host_mask(L.fhip_mask_sliding_window, self.dtype, seq_len, seq_len, seq_len, w)
            else:
                host = _host_mask(L.fhip_mask_causal, self.dtype, seq_len, seq_len, seq_len)
            base = AttentionMask(Tensor.from_numpy(device, host, self.dtype) if device is not None else None, host)
            self.masks[key] = base
        am = CAnalyticMask()
        rc = L.fhip_mask_get_analytic(seq_len, seqlen_offset, int(has_w), w, ctypes.byref(am))
        analytic = am if rc == OK else None
        if off > 0:
            host = np.empty((seq_len, cols.value), np_dtype(self.dtype))
            check(L.fhip_mask_get_mask(self.dtype, seq_len, seqlen_offset, int(has_w), w,
                                       host.ctypes.data_as(ctypes.c_void_p)))
            t = Tensor.from_numpy(device, host, self.dtype) if device is not None else None
            return AttentionMask(t, host, analytic)
        return AttentionMask(base._mask, base.host, analytic)

    def get_mask_on_device(self, seq_len, seqlen_offset, sliding_window_size, device):
        """The same tensor written by a kernel: no host loop over seq_len^2 elements, no upload."""
        L = lib()
        has_w = sliding_window_size is not None
        w = int(sliding_window_size) if has_w else 0
        rows, cols = ctypes.c_uint32(), ctypes.c_uint64()
        check(L.fhip_mask_get_mask_shape(seq_len, seqlen_offset, int(has_w), w, ctypes.byref(rows), ctypes.byref(cols)))
        t = Tensor.empty(device, (rows.value, cols.value), self.dtype)
        check(L.fhip_mask_get_mask_device(device.stream, self.dtype, seq_len, seqlen_offset, int(has_w), w,
                                          ctypes.c_void_p(t.buffer.ptr)))
        am = CAnalyticMask()
        rc = L.fhip_mask_get_analytic(seq_len, seqlen_offset, int(has_w), w, ctypes.byref(am))
        return AttentionMask(t, None, am if rc == OK else None)


# ---- KV cache -----------------------------------------------------------------------------------------

class KvCache:
    """fusor::cache::KvCache over device memory (kv_cache.rs:13-68, tensor_cache.rs:9-124)."""

    def __init__(self, concat_dim, max_sequence_len, dtype=F32, device=None):
        if concat_dim != 2:
            raise FhipError(ERR_UNSUPPORTED, "the device KV cache concatenates along dim 2 ([B,Hkv,seq,D]), "
                                             "the layout kalosm-llama uses")
        self.device = device or Device.default()
        self.dtype = dtype
        h = ctypes.c_void_p()
        check(lib().fhip_kv_cache_create(self.device.handle, dtype, max_sequence_len, ctypes.byref(h)))
        self.handle = h

    def __del__(self):
        try:
            if self.handle:
                lib().fhip_kv_cache_destroy(self.handle)
                self.handle = None
        except Exception:
            pass

    def reset(self):
        check(lib().fhip_kv_cache_reset(self.handle))

    def current_seq_len(self):
        n = ctypes.c_uint64()
        check(lib().fhip_kv_cache_current_seq_len(self.handle, ctypes.byref(n)))
        return n.value

    def allocated_seq_len(self):
        n = ctypes.c_uint64()
        check(lib().fhip_kv_cache_allocated_seq_len(self.handle, ctypes.byref(n)))
        return n.value

    def append(self, device, k, v):
        assert k.dtype == self.dtype and v.dtype == self.dtype
        ck, cv = k._c4(), v._c4()
        ka, va = CTensor4(), CTensor4()
        check(lib().fhip_kv_cache_append(self.handle, self.device.stream, ctypes.byref(ck), ctypes.byref(cv),
                                         ctypes.byref(ka), ctypes.byref(va)))

        def wrap(c):
            return Tensor(_View(self.device, c.ptr, self), self.dtype, tuple(c.shape), tuple(c.stride), c.offset)

        return wrap(ka), wrap(va)

    def append_rope(self, rope, k, v, start_pos, interleaved=False, k_norm=None):
        """append(rope(k), v) in one pass: the keys are rotated (RopeCache.forward semantics) and both
        tensors converted from their own element type to the cache's on the way into the cache.  With
        k_norm (an RmsNorm) the keys are normalised before the rotation (attention_k_norm)."""
        assert k.dtype == v.dtype
        ck, cv = k._c4(), v._c4()
        ka, va = CTensor4(), CTensor4()
        tables = rope._tables(start_pos, interleaved)
        if k_norm is None:
            check(lib().fhip_kv_cache_rope_append(self.handle, self.device.stream, ctypes.byref(tables), ctypes.byref(ck),
                                                  ctypes.byref(cv), k.dtype, ctypes.byref(ka), ctypes.byref(va)))
        else:
            cn = k_norm._c()
            check(lib().fhip_kv_cache_norm_rope_append(self.handle, self.device.stream, ctypes.byref(cn),
                                                       ctypes.byref(tables), ctypes.byref(ck), ctypes.byref(cv), k.dtype,
                                                       ctypes.byref(ka), ctypes.byref(va)))

        def wrap(c):
            return Tensor(_View(self.device, c.ptr, self), self.dtype, tuple(c.shape), tuple(c.stride), c.offset)

        return wrap(ka), wrap(va)


def _kv_step(self, rope, q, k, v, start_pos, interleaved=False, q_norm=None, k_norm=None, q_out_dtype=None):
    """rope(norm(q)) and append(rope(norm(k)), v) in one launch; returns (q_rotated, k_all, v_all)."""
    assert k.dtype == v.dtype
    q_out = Tensor.empty(self.device, q.shape, q_out_dtype if q_out_dtype is not None else q.dtype)
    cq, co, ck, cv = q._c4(), q_out._c4(), k._c4(), v._c4()
    ka, va = CTensor4(), CTensor4()
    tables = rope._tables(start_pos, interleaved)
    qn = q_norm._c() if q_norm is not None else None
    kn = k_norm._c() if k_norm is not None else None
    check(lib().fhip_kv_cache_qkv_rope_append(self.handle, self.device.stream, ctypes.byref(qn) if qn is not None else None,
                                              ctypes.byref(kn) if kn is not None else None, ctypes.byref(tables),
                                              ctypes.byref(cq), q.dtype, ctypes.byref(co), q_out.dtype, ctypes.byref(ck),
                                              ctypes.byref(cv), k.dtype, ctypes.byref(ka), ctypes.byref(va)))

    def wrap(c):
        return Tensor(_View(self.device, c.ptr, self), self.dtype, tuple(c.shape), tuple(c.stride), c.offset)

    return q_out, wrap(ka), wrap(va)


KvCache.qkv_rope_append = _kv_step


def base_inverse_frequency(dim, rope_theta):
    """fusor::base_inverse_frequency (rope.rs:188-196): 1 / theta^(i / dim) for even i, in f32."""
    theta = np.float32(rope_theta)
    return np.array([np.float32(1.0) / np.power(theta, np.float32(i) / np.float32(dim), dtype=np.float32)
                     for i in range(0, dim, 2)], np.float32)


class RopeCache:
    """fusor::RopeCache (rope.rs:180-265): [context_length, head_dim/2] f32 cos/sin tables on the device."""

    def __init__(self, head_dim, context_length, rope_theta, device=None, inverse_frequency=None):
        self.device = device or Device.default()
        inv = base_inverse_frequency(head_dim, rope_theta) if inverse_frequency is None \
            else np.asarray(inverse_frequency, np.float32)
        pos = np.arange(context_length, dtype=np.float32)[:, None]
        outer = (pos * inv[None, :]).astype(np.float32)  # a [n,1] x [1,h] matmul: one product per element
        self.cos_host, self.sin_host = np.cos(outer).astype(np.float32), np.sin(outer).astype(np.float32)
        self.cos = Tensor.from_numpy(self.device, self.cos_host, F32)
        self.sin = Tensor.from_numpy(self.device, self.sin_host, F32)
        self.rows = context_length

    @classmethod
    def from_parts(cls, cos, sin, device=None):
        self = cls.__new__(cls)
        self.device = device or Device.default()
        self.cos_host, self.sin_host = np.asarray(cos, np.float32), np.asarray(sin, np.float32)
        self.cos = Tensor.from_numpy(self.device, self.cos_host, F32)
        self.sin = Tensor.from_numpy(self.device, self.sin_host, F32)
        self.rows = self.cos_host.shape[0]
        return self

    def _tables(self, start_pos, interleaved):
        return CRopeTables(self.cos.buffer.ptr, self.sin.buffer.ptr, self.rows, start_pos, 1 if interleaved else 0)

    def apply(self, x, start_pos, interleaved=False, out_dtype=None, norm=None):
        """Tensor::rope_normal_fused / rope_fused with the tables narrowed to start_pos.. (rope.rs:139-175);
        with norm (an RmsNorm) the rows are normalised first, in the same pass."""
        out = Tensor.empty(self.device, x.shape, out_dtype if out_dtype is not None else x.dtype)
        cx, co = x._c4(), out._c4()
        tables = self._tables(start_pos, interleaved)
        if norm is None:
            check(lib().fhip_rope(self.device.stream, ctypes.byref(tables), ctypes.byref(cx), x.dtype, ctypes.byref(co),
                                  out.dtype))
        else:
            cn = norm._c()
            check(lib().fhip_norm_rope(self.device.stream, ctypes.byref(cn), ctypes.byref(tables), ctypes.byref(cx),
                                       x.dtype, ctypes.byref(co), out.dtype))
        return out

    def forward(self, q, k, start_pos):
        return self.apply(q, start_pos), self.apply(k, start_pos)

    def forward_interleaved(self, q, k, start_pos):
        return self.apply(q, start_pos, True), self.apply(k, start_pos, True)


class RmsNorm:
    """fusor::layers::RmsNorm<1, T> over the last dimension (fusor-ml/fusor/src/layers/rms_norm.rs:11-133): the
    q / k norm of blocks that have attention_q_norm / attention_k_norm."""

    def __init__(self, weight, bias=None, eps=1e-5, dtype=F32, device=None):
        self.device = device or Device.default()
        self.dtype = dtype
        self.eps = float(eps)
        self.weight = Tensor.from_numpy(self.device, np.asarray(weight, np.float32).reshape(1, -1), dtype)
        self.bias = None if bias is None else Tensor.from_numpy(self.device, np.asarray(bias, np.float32).reshape(1, -1), dtype)

    def _c(self):
        return CRmsNorm(self.weight.buffer.ptr, self.bias.buffer.ptr if self.bias is not None else None, self.dtype,
                        self.eps)

    def forward_generic_4d(self, x, out_dtype=None):
        """RmsNorm::forward_generic_4d (rms_norm.rs:122-133): the norm alone."""
        out = Tensor.empty(self.device, x.shape, out_dtype if out_dtype is not None else x.dtype)
        cx, co, cn = x._c4(), out._c4(), self._c()
        check(lib().fhip_norm_rope(self.device.stream, ctypes.byref(cn), None, ctypes.byref(cx), x.dtype,
                                   ctypes.byref(co), out.dtype))
        return out
