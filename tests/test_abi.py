"""Host-only checks of the C-ABI library: it loads, exports every symbol include/fusor_hip.h
declares, rejects what the reference panics on with the reference's messages, selects kernels as
documented, and builds masks bit-exactly.  No GPU is touched."""
import ctypes
import os
import re

import numpy as np
import pytest

import floneum_amd as fa
import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = 0x10000  # a non-null, 16-byte aligned stand-in for a device pointer; never dereferenced on the host


def declared_functions():
    text = open(os.path.join(ROOT, "include", "fusor_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 35
    L = ctypes.CDLL(fa.LIB_PATH)
    for n in names:
        assert hasattr(L, n), f"{n} is declared in include/fusor_hip.h but not exported"
    assert sorted(fa.SYMBOLS) == names, "the ctypes binding table and the header disagree"
    assert b"gfx950" in fa.lib().fhip_version()


def test_struct_layout_matches_header():
    # natural C layout of the header's structs on x86-64
    assert ctypes.sizeof(fa.CTensor4) == 8 + 8 + 16 + 32
    assert ctypes.sizeof(fa.CTensor2) == 8 + 8 + 8 + 16
    assert ctypes.sizeof(fa.CAnalyticMask) == 24
    assert ctypes.sizeof(fa.CAttnArgs) == 4 * 64 + 16 + 40 + 24 + 8 + 8 + 8 + 8 + 8 + 8 + 8


def t4(shape, strides=None, ptr=FAKE, offset=0):
    t = fa.CTensor4()
    t.ptr, t.offset = ptr, offset
    t.shape[:] = shape
    st, acc = [], 1
    for n in reversed(shape):
        st.append(acc)
        acc *= n
    t.stride[:] = strides if strides is not None else list(reversed(st))
    return t


def make_args(B=1, H=4, Hkv=2, Sq=8, Skv=8, D=64, dtype=fa.F16, **kw):
    a = fa.CAttnArgs()
    a.q, a.k, a.v, a.out = t4([B, H, Sq, D]), t4([B, Hkv, Skv, D]), t4([B, Hkv, Skv, D]), t4([B, H, Sq, D])
    a.dtype = a.out_dtype = dtype
    a.scale = 0.125
    for k, v in kw.items():
        setattr(a, k, v)
    return a


def status(a):
    rc = fa.lib().fhip_flash_attention_validate(ctypes.byref(a))
    return rc, fa.lib().fhip_last_error().decode()


def test_validate_accepts_good_arguments():
    assert status(make_args())[0] == fa.OK
    assert status(make_args(dtype=fa.F32))[0] == fa.OK
    a = make_args()
    a.out_dtype = fa.F32
    assert status(a)[0] == fa.OK


def test_validate_reference_panics():
    # fusor flash_attention.rs:94-99
    rc, msg = status(make_args(H=3, Hkv=2))
    assert rc == fa.ERR_INVALID_ARG and msg == "Number of Q heads (3) must be divisible by number of K/V heads (2)"
    # fusor flash_attention.rs:153-160
    a = make_args(Sq=8, Skv=16)
    a.mask_kind = fa.MaskKind.QKMask
    a.mask.ptr = FAKE
    a.mask.shape[:] = [8, 8]
    rc, msg = status(a)
    assert rc == fa.ERR_INVALID_ARG and msg == "QKMask shape [8, 8] does not match expected [8, 16]"
    # fusor flash_attention.rs:165-172
    a.mask_kind = fa.MaskKind.BatchKeyMask
    rc, msg = status(a)
    assert rc == fa.ERR_INVALID_ARG and msg == "BatchKeyMask shape [8, 8] does not match expected [1, 16]"
    a.mask.shape[:] = [1, 16]
    assert status(a)[0] == fa.OK


def test_validate_other_errors():
    a = make_args()
    a.v.shape[2] = 9
    assert status(a)[0] == fa.ERR_INVALID_ARG
    a = make_args()
    a.out.shape[3] = 32
    assert status(a)[0] == fa.ERR_INVALID_ARG
    a = make_args()
    a.q.ptr = None
    assert status(a)[0] == fa.ERR_INVALID_ARG
    a = make_args()
    a.scale = float("nan")
    assert status(a)[0] == fa.ERR_INVALID_ARG
    a = make_args()
    a.out_dtype = fa.BF16
    assert status(a)[0] == fa.ERR_INVALID_ARG
    a = make_args()
    a.analytic.enabled = 1
    a.mask_kind = fa.MaskKind.QKMask
    a.mask.ptr = FAKE
    a.mask.shape[:] = [8, 8]
    assert status(a)[0] == fa.ERR_INVALID_ARG
    a = make_args(D=1024)
    assert status(a)[0] == fa.ERR_UNSUPPORTED
    assert fa.lib().fhip_flash_attention_validate(None) == fa.ERR_INVALID_ARG
    assert fa.lib().fhip_flash_attention(None, ctypes.byref(make_args())) == fa.ERR_INVALID_ARG


def test_validate_accepts_tensors_without_elements():
    # no keys, no queries, no batch: valid calls (the result is all zeros, or has no element); no memory needed
    for kw in (dict(Skv=0), dict(Sq=0), dict(B=0), dict(H=0, Hkv=0)):
        a = make_args(**kw)
        assert status(a)[0] == fa.OK, kw
        need = ctypes.c_size_t(99)
        assert fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(a), 256, ctypes.byref(need)) == fa.OK
        assert need.value == 0
    a = make_args(Sq=0)
    a.q.ptr = a.out.ptr = None
    assert status(a)[0] == fa.OK
    # u32::is_multiple_of(0) holds for 0 only (fusor flash_attention.rs:94-99)
    rc, msg = status(make_args(H=4, Hkv=0))
    assert rc == fa.ERR_INVALID_ARG and "divisible" in msg


def selected(a):
    kid = ctypes.c_int32()
    rc = fa.lib().fhip_flash_attention_select(ctypes.byref(a), ctypes.byref(kid))
    return rc, kid.value


def test_kernel_selection():
    assert selected(make_args(Sq=512, Skv=512, D=128))[1] == fa.KERNEL_PREFILL_MFMA
    assert selected(make_args(Sq=512, Skv=512, D=64, dtype=fa.F32))[1] == fa.KERNEL_PREFILL_F32
    assert selected(make_args(Sq=1, Skv=4096, D=128))[1] == fa.KERNEL_DECODE_SPLITKV
    assert selected(make_args(Sq=1, Skv=4096, D=96, dtype=fa.BF16))[1] == fa.KERNEL_DECODE_SPLITKV
    # f32 decode (kalosm-llama's cache is f32, attention_layer.rs:400-403) streams through the split-KV kernel too
    assert selected(make_args(Sq=1, Skv=4096, D=128, dtype=fa.F32))[1] == fa.KERNEL_DECODE_SPLITKV
    assert selected(make_args(Sq=7, Skv=9, D=33))[1] == fa.KERNEL_GENERIC
    # a dense additive mask without the scratch its interval form needs: the f32-arithmetic tiled kernel adds the mask
    # element by element (16-bit rows are widened on load), up to head_dim 128; beyond that the general kernel
    a = make_args(Sq=64, Skv=64, D=128)
    a.mask_kind = fa.MaskKind.QKMask
    a.mask.ptr = FAKE
    a.mask.shape[:] = [64, 64]
    a.mask.stride[:] = [64, 1]
    assert selected(a)[1] == fa.KERNEL_PREFILL_F32
    a = make_args(Sq=64, Skv=64, D=256)
    a.mask_kind = fa.MaskKind.QKMask
    a.mask.ptr = FAKE
    a.mask.shape[:] = [64, 64]
    a.mask.stride[:] = [64, 1]
    assert selected(a)[1] == fa.KERNEL_GENERIC
    # 16-bit head dims: every multiple of 8 up to 256 runs on the 16-bit matrix cores (64 / 96 / 128 on the 256-row kernel,
    # the others, padded with zeros to the next multiple of 32, on the wide-head one) ...
    assert selected(make_args(Sq=64, Skv=64, D=80))[1] == fa.KERNEL_PREFILL_MFMA
    assert selected(make_args(Sq=64, Skv=64, D=200, dtype=fa.BF16))[1] == fa.KERNEL_PREFILL_MFMA
    assert selected(make_args(Sq=64, Skv=64, D=8))[1] == fa.KERNEL_PREFILL_MFMA
    assert selected(make_args(Sq=64, Skv=64, D=256, dtype=fa.BF16))[1] == fa.KERNEL_PREFILL_MFMA
    # ... and the other multiples of 4 on the f32-arithmetic kernel (rows widened on load)
    assert selected(make_args(Sq=64, Skv=64, D=100))[1] == fa.KERNEL_PREFILL_F32
    assert selected(make_args(Sq=64, Skv=64, D=12, dtype=fa.BF16))[1] == fa.KERNEL_PREFILL_F32
    assert selected(make_args(Sq=64, Skv=64, D=256, dtype=fa.F32))[1] == fa.KERNEL_PREFILL_F32
    assert selected(make_args(Sq=64, Skv=64, D=264))[1] == fa.KERNEL_GENERIC
    # innermost stride != 1 or a misaligned base pointer -> generic
    a = make_args(Sq=64, Skv=64, D=128)
    a.k.stride[:] = [2 * 64 * 128, 1, 128 * 2, 64]
    assert selected(a)[1] == fa.KERNEL_GENERIC
    a = make_args(Sq=64, Skv=64, D=128)
    a.q.offset = 3
    assert selected(a)[1] == fa.KERNEL_GENERIC
    # narrowed cache view (stride[1] = allocated * D) keeps the tiled kernel
    a = make_args(Sq=64, Skv=100, D=128)
    a.k.stride[:] = [2 * 128 * 128, 128 * 128, 128, 1]
    a.v.stride[:] = [2 * 128 * 128, 128 * 128, 128, 1]
    assert selected(a)[1] == fa.KERNEL_PREFILL_MFMA
    # forcing a kernel that cannot run the arguments is an error, not a silent fallback
    a = make_args(Sq=7, Skv=9, D=33)
    a.force_kernel = fa.KERNEL_PREFILL_MFMA
    assert selected(a)[0] == fa.ERR_UNSUPPORTED
    # the id that is never chosen: the tiled 16-bit kernel's 64-rows-per-wavefront form, head_dim 128 only, keys never
    # split over workgroups (no partials in the workspace it asks for)
    a = make_args(Sq=128, Skv=8192, D=128)
    need = ctypes.c_size_t()
    assert fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(a), 256, ctypes.byref(need)) == fa.OK and need.value > 0
    a.force_kernel = fa.KERNEL_PREFILL_MFMA_ROWS64
    assert selected(a) == (fa.OK, fa.KERNEL_PREFILL_MFMA_ROWS64)
    assert fa.lib().fhip_flash_attention_workspace_bytes(ctypes.byref(a), 256, ctypes.byref(need)) == fa.OK and need.value == 0
    for kw in (dict(D=64), dict(D=256), dict(D=128, dtype=fa.F32)):
        a = make_args(Sq=64, Skv=64, **kw)
        a.force_kernel = fa.KERNEL_PREFILL_MFMA_ROWS64
        assert selected(a)[0] == fa.ERR_UNSUPPORTED, kw


def test_workspace_bytes():
    need = ctypes.c_size_t()
    L = fa.lib()
    a = make_args(B=16, H=32, Hkv=8, Sq=1, Skv=4096, D=128)
    assert L.fhip_flash_attention_workspace_bytes(ctypes.byref(a), 256, ctypes.byref(need)) == fa.OK
    # (partials of D + 2 floats per (batch, head, split); up to 8 splits a little more: every split's partials start on a
    # 128-byte line and every (batch, kv head) has an arrival counter, for the merge inside the main kernel)
    per = 16 * 32 * (128 + 2) * 4
    nsplit = need.value // per
    assert 2 <= nsplit <= 16 and need.value - nsplit * per <= 16 * 8 * (nsplit * 128 + 4) + 256
    a = make_args(Sq=512, Skv=512, D=128)
    assert L.fhip_flash_attention_workspace_bytes(ctypes.byref(a), 256, ctypes.byref(need)) == fa.OK and need.value == 0
    # a decode call without the workspace it needs must fail before any launch (stream is checked first)
    assert L.fhip_flash_attention(None, ctypes.byref(a)) == fa.ERR_INVALID_ARG


def test_decode_split_planning_on_256_cus():
    """How many key splits the planner asks a workspace for (partials of D + 2 floats per (batch, head, split)):
    1024-key chunks for a batch that fills the chip, down to one workgroup step per split for one chat stream
    (128 keys for the matrix-core variant, 64 for the vector variant at head_dim 128), unsplit up to 256 keys."""
    need = ctypes.c_size_t()
    L = fa.lib()

    def splits(B, H, Hkv, Skv, D, dtype):
        a = make_args(B=B, H=H, Hkv=Hkv, Sq=1, Skv=Skv, D=D, dtype=dtype)
        assert L.fhip_flash_attention_workspace_bytes(ctypes.byref(a), 256, ctypes.byref(need)) == fa.OK
        per = B * H * (D + 2) * 4
        ns = need.value // per
        # more than 8 splits: the partials exactly; up to 8 the padding and counters of the merge inside the main kernel
        assert need.value == ns * per if ns > 8 or ns == 0 else need.value - ns * per <= B * Hkv * (ns * 128 + 4) + 256
        return ns

    assert splits(16, 32, 8, 4096, 128, fa.F16) == 4     # C2
    assert splits(1, 32, 8, 4096, 128, fa.F16) == 32     # one stream, 128-key steps
    assert splits(1, 32, 8, 32768, 128, fa.F16) == 64
    assert splits(1, 32, 8, 4096, 128, fa.F32) == 64     # vector variant: 64-key steps
    assert splits(1, 32, 8, 1024, 128, fa.F32) == 16
    assert splits(1, 32, 8, 256, 128, fa.F16) == 0       # unsplit: no partials, no second launch


def test_prefill_key_split_planning_on_256_cus():
    """Few query rows on a long cache: the keys are split over workgroups (partials of D + 2 floats per row and share
    for the f32-arithmetic kernel, D + 4 for the 16-bit one); a square causal prompt is not split."""
    need = ctypes.c_size_t()
    L = fa.lib()

    def shares(Sq, Skv, dtype, pitch, analytic=True, D=128, H=32, Hkv=8):
        a = make_args(B=1, H=H, Hkv=Hkv, Sq=Sq, Skv=Skv, D=D, dtype=dtype)
        if analytic:
            a.analytic.enabled, a.analytic.causal, a.analytic.q_pos_offset = 1, 1, Skv - Sq
        assert L.fhip_flash_attention_workspace_bytes(ctypes.byref(a), 256, ctypes.byref(need)) == fa.OK
        per = H * Sq * pitch * 4
        assert need.value % per == 0
        return need.value // per

    assert shares(128, 8192, fa.F32, 130) == 4    # a new chat turn: 4 query blocks x 32 heads x 4 shares of 2048 keys
    assert shares(128, 8192, fa.F16, 132) == 8    # one 128-row block per head x 8 shares of 1024 keys
    assert shares(32, 32768, fa.F16, 132) == 32   # packed: 8 head quads x 32 shares of 1024 keys (unpacked it was 32 heads x 16)
    assert shares(512, 512, fa.F32, 130) == 0     # square causal prompts are left alone
    assert shares(2048, 2048, fa.F16, 132) == 0
    # a few rows on a short cache: shorter shares while CUs would stay without a workgroup
    assert shares(20, 2048, fa.F16, 132) == 8     # 256 keys (up to 64 rows)
    assert shares(128, 2048, fa.F16, 132) == 4    # 512 keys
    assert shares(128, 1024, fa.F16, 132) == 0    # two shares of 512 keys lose there
    assert shares(20, 2048, fa.F32, 130) == 8     # 256 keys fill the chip (32 thirty-two-row workgroups x 8)
    assert shares(20, 1024, fa.F32, 130) == 8     # 128 keys
    # head_dim 256: two query heads per workgroup in f32 arithmetic (8 workgroups before the split)
    assert shares(20, 2048, fa.F32, 258, D=256, H=16, Hkv=4) == 16   # 128 keys
    assert shares(48, 8192, fa.F32, 258, D=256, H=16, Hkv=4) == 16   # unpacked above 32 rows: 512 keys
    assert shares(20, 8192, fa.F16, 260, D=256, H=16, Hkv=4) == 8    # the wide-head 16-bit kernel, four heads per workgroup
    assert shares(64, 8192, fa.F16, 260, D=256, H=16, Hkv=4) == 8    # 64-row workgroups, two per CU


# ---- masks: bit-exact against the checker and the reference's vectors -----------------------------------

NEG_BITS = {fa.F32: 0xFF800000, fa.F16: 0xFC00, fa.BF16: 0xFF80}


def lib_get_mask(dtype, n, off, w):
    L = fa.lib()
    rows, cols = ctypes.c_uint32(), ctypes.c_uint64()
    assert L.fhip_mask_get_mask_shape(n, off, int(w is not None), w or 0, ctypes.byref(rows), ctypes.byref(cols)) == 0
    out = np.empty((rows.value, cols.value), np.uint32 if dtype == fa.F32 else np.uint16)
    assert L.fhip_mask_get_mask(dtype, n, off, int(w is not None), w or 0, out.ctypes.data_as(ctypes.c_void_p)) == 0
    return out


@pytest.mark.parametrize("dtype", [fa.F32, fa.F16, fa.BF16])
def test_masks_bit_exact(dtype):
    for n in (1, 2, 3, 4, 7, 33):
        for off in (0, 1, 5, 100):
            for w in (None, 1, 2, 4, 9, 64):
                want = np.isneginf(oracle.get_mask(n, off, w))
                got = lib_get_mask(dtype, n, off, w)
                assert got.shape == want.shape, (n, off, w)
                assert np.array_equal(got, np.where(want, NEG_BITS[dtype], 0).astype(got.dtype)), (n, off, w)
    L = fa.lib()
    n = 5
    out = np.empty((n, n), np.uint32 if dtype == fa.F32 else np.uint16)
    assert L.fhip_mask_causal(dtype, n, out.ctypes.data_as(ctypes.c_void_p)) == 0
    assert np.array_equal(out != 0, np.isneginf(oracle.mask_causal(n)))
    assert L.fhip_mask_sliding_window(dtype, n, 2, out.ctypes.data_as(ctypes.c_void_p)) == 0
    assert np.array_equal(out != 0, np.isneginf(oracle.mask_sliding(n, 2)))


def test_masks_reference_goldens_through_the_host_mirror():
    import json
    g = json.load(open(os.path.join(ROOT, "tests", "golden", "masks.json")))
    cache = fa.MaskCache(fa.F32)
    for name in ("causal_3", "causal_4", "sliding_4_w2"):
        c = g[name]
        m = cache.get_mask(c["seq_len"], c["offset"], c["window"], None)  # device None: host values only
        assert np.array_equal(np.isneginf(m.host), np.array(c["masked"]) == 1), name
        assert set(np.unique(m.host.view(np.uint32))) <= {0, 0xFF800000}
    c = g["offset_shape"]
    assert list(cache.get_mask(c["seq_len"], c["offset"], c["window"], None).host.shape) == c["shape"]
    assert np.array_equal(np.isneginf(fa.AttentionMask.causal(None, 3).host), np.array(g["causal_3"]["masked"]) == 1)


def test_analytic_descriptor_equals_dense_mask():
    L = fa.lib()
    for n in (1, 3, 8, 40):
        for off in (0, 2, 17, 500):
            for w in (None, 1, 3, 8, 64):
                am = fa.CAnalyticMask()
                assert L.fhip_mask_get_analytic(n, off, int(w is not None), w or 0, ctypes.byref(am)) == 0
                dense = np.isneginf(oracle.get_mask(n, off, w))
                i = np.arange(n)[:, None] + am.q_pos_offset
                j = np.arange(dense.shape[1])[None, :]
                rule = (j > i) if am.causal else np.zeros_like(dense)
                if am.window:
                    rule = rule | ((j + am.window) <= i)
                assert am.enabled == 1 and np.array_equal(rule, dense), (n, off, w)
