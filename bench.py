#!/usr/bin/env python3
"""Benchmark of the attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2|C3|C1|C4|C5] [--no-cpu] [--no-extra]

A step is one attention call through the C ABI on synthetic, seeded inputs that are resident in
HBM before the timed region.  The default workload is C2 (Llama-3-8B-shaped decode, batch 16, 4096
f16 KV tokens per sequence): `value` is its KV-streaming rate in GB/s (algorithmic bytes per call /
time per call, combine pass included).

Output: one JSON object per line.  Lines that start with {"detail": ...} come first and hold every workload's
complete record (roofline of its dominant kernel from HIP events carried by that kernel's dispatch on the launch
stream, the CPU checker timed on the host cores as "cpu_baseline", a spot check against it) and the two
calibrations.  The LAST line is the result line: C2 in full contract form with "roofline" and "cpu_baseline",
the C3 prefill figure (TFLOP/s, MFMA roofline, its own cpu_baseline) under "prefill", and one short entry per
other workload under "configs" (C1, C1M, C4, C5, F2, M1, L1, L2, W2, W3); it stays under 4 KB.
"""
import argparse
import ctypes
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "attn prefill TFLOP/s + decode KV GB/s, % of roofline, 1xMI355X"
PEAK_HBM_GBS = 8000.0
PEAK_MFMA_F16_TFLOPS = 2500.0
PEAK_MFMA_F32_TFLOPS = 157.3
SEED = 0xF10E0000
# HBM bytes per launch of the dominant kernel, from two rocprofv3 --pmc runs of this file (FETCH_SIZE, then
# WRITE_SIZE), each scaled by what the same counter reads for a 256 MiB copy in the same run.  The record holds,
# per configuration, the bytes and the SHA-256 of the kernel source they were measured on; a figure whose source
# has changed since is not reported.  Written by --record-traffic from the counter CSVs.
TRAFFIC_RECORD = os.path.join(ROOT, "profiles", "traffic.json")
KERNEL_SOURCES = {"decode_splitkv": "attn_decode.hip", "prefill_mfma": "attn_prefill_mfma.hip",
                  "prefill_f32": "attn_prefill_f32.hip", "generic": "attn_generic.hip"}


def source_hash(kernel, source=None):
    path = os.path.join(ROOT, "floneum_amd", "csrc", source or KERNEL_SOURCES[kernel])
    return hashlib.sha256(open(path, "rb").read()).hexdigest()


def measured_traffic(name, kernel):
    """(bytes per launch or None, note) from the committed counter record."""
    try:
        rec = json.load(open(TRAFFIC_RECORD)).get(name)
    except (OSError, ValueError):
        rec = None
    if not rec:
        return None, "no counter record for this configuration"
    if rec.get("kernel") != kernel or rec.get("source_sha256") != source_hash(kernel, rec.get("source")):
        return None, "the kernel source has changed since the counters were read"
    return float(rec["fetch_bytes"]) + float(rec["write_bytes"]), \
        f"FETCH_SIZE {rec['fetch_bytes']:.4g} B + WRITE_SIZE {rec['write_bytes']:.4g} B per launch"


def configs():
    # name -> description of the synthetic workload (the benchmark configurations, in order)
    return {
        "C1": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=512, Skv=512, D=64, dtype="f32", std=1.0, causal=True),
        "C2": dict(kind="decode", B=16, H=32, Hkv=8, Sq=1, Skv=4096, D=128, dtype="f16", std=0.5, causal=False),
        "C3": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=8192, Skv=8192, D=128, dtype="f16", std=1.0, causal=True),
        # reference-faithful sliding-window continuation: K/V are the last 4096 cached positions and the
        # mask is get_mask(512, 16384, Some(4096)) = 3584 visible columns + a causal 512x512 block
        "C4": dict(kind="prefill", B=4, H=32, Hkv=8, Sq=512, Skv=4096, D=128, dtype="f16", std=1.0, causal=True,
                   q_pos_offset=3584, window=4096),
        # absolute-position form of the same chunk (not a parity claim against the reference's truncating cache): the
        # whole 16896-key cache is passed and the analytic window leaves every query exactly 4096 keys
        "C4B": dict(kind="prefill", B=4, H=32, Hkv=8, Sq=512, Skv=16896, D=128, dtype="f16", std=1.0, causal=True,
                    q_pos_offset=16384, window=4096),
        # C3 and C4 on the form of the tiled kernel the library never chooses (force_kernel 5: four wavefronts of 64 query
        # rows per workgroup, one per SIMD; half the LDS operand reads per matrix instruction, everything issued in order)
        "C3R": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=8192, Skv=8192, D=128, dtype="f16", std=1.0, causal=True,
                    force_kernel=5),
        "C4R": dict(kind="prefill", B=4, H=32, Hkv=8, Sq=512, Skv=4096, D=128, dtype="f16", std=1.0, causal=True,
                    q_pos_offset=3584, window=4096, force_kernel=5),
        "C5": dict(kind="decode", B=32, H=32, Hkv=32, Sq=1, Skv=32768, D=96, dtype="f16", std=1.0, causal=False,
                   ragged=(128, 32768)),
        # not a headline configuration: a new chat turn, 128 query rows on 8192 cached keys (the shape at which the
        # prefill kernels split the keys over workgroups), in the reference's f32 and in f16
        "T1": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=128, Skv=8192, D=128, dtype="f32", std=1.0, causal=True,
                   q_pos_offset=8064),
        "T2": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=128, Skv=8192, D=128, dtype="f16", std=1.0, causal=True,
                   q_pos_offset=8064),
        # short prompts (latency-bound grids that do not fill the chip): 1024 tokens in f16, 512 tokens in f32
        "P1": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=1024, Skv=1024, D=128, dtype="f16", std=1.0, causal=True),
        "P2": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=512, Skv=512, D=128, dtype="f32", std=1.0, causal=True),
        # not headline configurations either: one chat stream, i.e. a batch-1 decode step on 4096 cached keys in the
        # reference's f32 and in f16, and in f16 on 32768 keys (latency-bound: two dependent launches)
        "S1": dict(kind="decode", B=1, H=32, Hkv=8, Sq=1, Skv=4096, D=128, dtype="f32", std=0.5, causal=False),
        "S2": dict(kind="decode", B=1, H=32, Hkv=8, Sq=1, Skv=4096, D=128, dtype="f16", std=0.5, causal=False),
        "S3": dict(kind="decode", B=1, H=32, Hkv=8, Sq=1, Skv=32768, D=128, dtype="f16", std=0.5, causal=False),
        # C1 as kalosm-llama really calls it: the mask comes as the [512, 512] tensor MaskCache::get_mask builds, not as
        # a formula.  Timed as a model calls it layer after layer: the mask tensor comes with the interval table its owner computed
        # when it built the mask (fhip_mask_intervals; MaskCache keeps both), so the calls run no scan of the mask.
        # C1S: the same call without the table (scan of the mask in every call).
        "C1M": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=512, Skv=512, D=64, dtype="f32", std=1.0, causal=True,
                    mask_tensor=True, mask_table=True),
        "C1S": dict(kind="prefill", B=1, H=32, Hkv=8, Sq=512, Skv=512, D=64, dtype="f32", std=1.0, causal=True,
                    mask_tensor=True),
        # C2 with its lengths given as a per-sequence array (all 4096): the same split, merged by a second kernel, which is
        # how every split-KV decode call ran before the merge moved into the main kernel for equal-length batches
        "C2K": dict(kind="decode", B=16, H=32, Hkv=8, Sq=1, Skv=4096, D=128, dtype="f16", std=0.5, causal=False,
                    ragged=(4096, 4096)),
        # C2's batch with the f32 cache kalosm-llama really keeps (attention_layer.rs:400-403): the f32 matrix-core
        # variant of the decode kernel; and a 16-bit cache with Gemma-3's key length 256 (the 16-bit matrix-core variant
        # with one workgroup per CU)
        "F2": dict(kind="decode", B=16, H=32, Hkv=8, Sq=1, Skv=4096, D=128, dtype="f32", std=0.5, causal=False),
        "W2": dict(kind="decode", B=16, H=16, Hkv=4, Sq=1, Skv=4096, D=256, dtype="f16", std=0.5, causal=False),
        # a 4096-token prompt at that key length in 16-bit (the four-wavefront tiled kernel for head dims 160 ... 256)
        "W3": dict(kind="prefill", B=1, H=16, Hkv=4, Sq=4096, Skv=4096, D=256, dtype="f16", std=1.0, causal=True),
        # a multi-token decode step: C2's batch with four new rows per sequence at the end of the cache, causal among
        # themselves (a draft being verified); the rows ride beside the heads of a GQA group, the cache is read once
        "M1": dict(kind="decode", B=16, H=32, Hkv=8, Sq=4, Skv=4096, D=128, dtype="f16", std=0.5, causal=True),
        # eight new rows per sequence: 32 columns per KV head, two column blocks per workgroup of the decode kernel
        "M2": dict(kind="decode", B=16, H=32, Hkv=8, Sq=8, Skv=4096, D=128, dtype="f16", std=0.5, causal=True),
    }


def visible_pairs(c, lens=None):
    """Number of (query, key) pairs per (batch, head) that the mask leaves visible, summed over batch."""
    if lens is not None:
        return int(np.sum(lens)) * c["Sq"]
    if not c["causal"]:
        return c["B"] * c["Sq"] * c["Skv"]
    off = c.get("q_pos_offset", c["Skv"] - c["Sq"])
    w = c.get("window", 0)
    i = np.arange(c["Sq"], dtype=np.int64) + off
    hi = np.minimum(i + 1, c["Skv"])
    lo = np.maximum(i - w + 1, 0) if w else np.zeros_like(i)
    return c["B"] * int(np.sum(np.maximum(hi - lo, 0)))


def algorithmic(c, lens=None):
    """FLOPs = 4 D x visible pairs x heads; bytes = |Q| + |K| + |V| + |O| with K/V once per KV head."""
    eb = 4 if c["dtype"] == "f32" else 2
    pairs = visible_pairs(c, lens)
    flops = 4 * c["D"] * pairs * c["H"]
    kv_rows = int(np.sum(lens)) if lens is not None else c["B"] * c["Skv"]
    byts = eb * (2 * c["B"] * c["H"] * c["Sq"] * c["D"] + 2 * kv_rows * c["Hkv"] * c["D"])
    return flops, byts


class Event:
    def __init__(self, fa, dev):
        self.fa, self.h = fa, ctypes.c_void_p()
        fa.check(fa.lib().fhip_event_create(dev.handle, ctypes.byref(self.h)))

    def record(self, dev):
        self.fa.check(self.fa.lib().fhip_event_record(self.h, dev.stream))

    def sync(self):
        self.fa.check(self.fa.lib().fhip_event_synchronize(self.h))

    def ms_since(self, start):
        ms = ctypes.c_float()
        self.fa.check(self.fa.lib().fhip_event_elapsed_ms(start.h, self.h, ctypes.byref(ms)))
        return ms.value


def _big_normal(synth, seed, tid, shape, std, npdt, max_batches=2):
    """Normals for shape [B, ...]: the first `max_batches` batch entries are generated, the rest
    repeat them with alternating sign (timing needs distinct memory, not distinct statistics)."""
    B = shape[0]
    if B <= max_batches:
        return synth.normal(seed, tid, shape, std, npdt)
    base = synth.normal(seed, tid, (max_batches,) + tuple(shape[1:]), std, npdt)
    out = np.empty(shape, npdt)
    for b in range(B):
        out[b] = base[b % max_batches] if (b // max_batches) % 2 == 0 else -base[b % max_batches]
    return out


def make_inputs(fa, synth, dev, c, cfg_id, n_sets):
    """n_sets rotating (Q, K, V) sets so a decode step never finds its KV in the 256 MB Infinity
    Cache.  Set 0 is the seeded workload (and the one spot-checked); sets 1.. are rolled, sign-flipped
    copies of it, which cost no generator time."""
    dt = {"f32": fa.F32, "f16": fa.F16}[c["dtype"]]
    npdt = np.float32 if dt == fa.F32 else np.float16
    seed = SEED + cfg_id
    big = c["B"] * c["Hkv"] * c["Skv"] * c["D"] > (1 << 28)
    gen = (lambda tid, shp: _big_normal(synth, seed, tid, shp, c["std"], npdt)) if big else \
          (lambda tid, shp: synth.normal(seed, tid, shp, c["std"], npdt))
    q = gen(0, (c["B"], c["H"], c["Sq"], c["D"]))
    k = gen(1, (c["B"], c["Hkv"], c["Skv"], c["D"]))
    v = gen(2, (c["B"], c["Hkv"], c["Skv"], c["D"]))
    sets = []
    for s in range(n_sets):
        if s == 0:
            arrs = (q, k, v)
        else:
            sg = npdt(-1.0 if s % 2 else 1.0)
            arrs = (q * sg, np.roll(k, s, axis=2) * sg, np.roll(v, s, axis=2))
        sets.append(tuple(fa.Tensor.from_numpy(dev, a, dt) for a in arrs))
    return dt, sets, (q, k, v)


def prepare(fa, dev, c, sets, lens_t):
    """Argument blocks (one per input set) with output and workspace bound once, outside the timed region."""
    L = fa.lib()
    blocks = []
    mask = None
    if c.get("mask_tensor"):
        # the tensor the reference's MaskCache builds for this call, written on the device
        dt = {"f32": fa.F32, "f16": fa.F16}[c["dtype"]]
        off = c.get("q_pos_offset", c["Skv"] - c["Sq"])
        am = fa.MaskCache(dt).get_mask_on_device(c["Sq"], off, c.get("window") or None, dev)
        mask = (am.mask(), fa.MaskKind.QKMask, am.intervals()) if c.get("mask_table") else (am.mask(), fa.MaskKind.QKMask)
    for (q, k, v) in sets:
        analytic = None
        if c["causal"] and mask is None:
            analytic = (True, c.get("q_pos_offset", c["Skv"] - c["Sq"]), c.get("window", 0))
        args = q._attn_args(k, v, c["D"] ** -0.5, mask, analytic, lens_t, None, c.get("force_kernel", fa.KERNEL_AUTO), None)
        need = ctypes.c_size_t()
        fa.check(L.fhip_flash_attention_workspace_bytes(ctypes.byref(args), dev.compute_units, ctypes.byref(need)))
        if need.value:
            ws = fa.Buffer(dev, need.value)
            args.workspace, args.workspace_bytes = ws.ptr, need.value
            args._keep.append(ws)
        blocks.append(args)
    kid = ctypes.c_int32()
    fa.check(L.fhip_flash_attention_select(ctypes.byref(blocks[0]), ctypes.byref(kid)))
    return blocks, fa.KERNEL_NAMES[kid.value]


def time_config(fa, dev, c, blocks, steps, warmup):
    """Wall-clock over exactly `steps` calls (sync on both sides), then a second instrumented pass of `steps`
    calls in which the dispatch of every call's main kernel carries a pair of HIP events: their interval is the
    kernel's own duration as the command processor stamps it (what a profiler's kernel trace reports)."""
    L = fa.lib()
    n = len(blocks)
    for i in range(warmup):
        fa.check(L.fhip_flash_attention(dev.stream, ctypes.byref(blocks[i % n])))
    dev.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fa.check(L.fhip_flash_attention(dev.stream, ctypes.byref(blocks[i % n])))
    dev.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps

    starts = [Event(fa, dev) for _ in range(steps)]
    dones = [Event(fa, dev) for _ in range(steps)]
    for i in range(steps):
        a = blocks[i % n]
        a.main_kernel_start, a.main_kernel_done = starts[i].h, dones[i].h
        fa.check(L.fhip_flash_attention(dev.stream, ctypes.byref(a)))
        a.main_kernel_start = a.main_kernel_done = None
    dev.synchronize()
    kernel_ms = np.array([dones[i].ms_since(starts[i]) for i in range(steps)])
    for e in starts + dones:
        L.fhip_event_destroy(e.h)
    return wall_ms, kernel_ms


def _decode_rows_mask(c, n):
    """[Sq, n] mask of a multi-token decode step (row r sits at position n - Sq + r); None for a plain step."""
    if not c["causal"]:
        return None
    i = np.arange(c["Sq"])[:, None] + (n - c["Sq"])
    return np.where(np.arange(n)[None, :] > i, -np.inf, 0.0).astype(np.float32)


def parity_spot_check(fa, oracle, c, out_t, host, lens):
    """A few output rows of the timed workload against the CPU checker (cheap: rows are independent)."""
    q, k, v = host
    f32 = lambda a: np.asarray(a, np.float32)  # noqa: E731  (slices are widened, never the whole cache)
    out = np.asarray(out_t.to_numpy(), np.float32)
    if c["kind"] == "decode":
        bs = [0, c["B"] - 1]
        worst = 0.0
        for b in bs:
            n = int(lens[b]) if lens is not None else c["Skv"]
            mask = _decode_rows_mask(c, n)
            ref = oracle.flash_attention(f32(q[b:b + 1]), f32(k[b:b + 1, :, :n]), f32(v[b:b + 1, :, :n]),
                                         c["D"] ** -0.5, mask, None if mask is None else "qk")
            worst = max(worst, float(np.abs(out[b:b + 1] - ref).max()))
        return worst
    q, k, v = f32(q), f32(k), f32(v)
    rows = np.unique(np.linspace(0, c["Sq"] - 1, 16).astype(np.int32))
    off = c.get("q_pos_offset", c["Skv"] - c["Sq"])
    mask = None
    if c["causal"]:
        i = rows[:, None].astype(np.int64) + off
        j = np.arange(c["Skv"])[None, :]
        masked = j > i
        if c.get("window", 0):
            masked |= (j + c["window"]) <= i
        mask = np.where(masked, -np.inf, 0.0).astype(np.float32)
    # the checker takes a [Sq, Skv] mask: evaluate the selected rows as their own Sq
    ref = oracle.flash_attention(q[:, :, rows], k, v, c["D"] ** -0.5, mask, "qk" if mask is not None else None)
    return float(np.abs(out[:, :, rows] - ref).max())


def cpu_baseline(oracle, c, host, lens, flops, byts):
    """The CPU checker (a C port of fusor's CPU composite) on the host cores, bounded to ~10-30 s."""
    q, k, v = host
    f32 = lambda a: np.asarray(a, np.float32)  # noqa: E731
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    scale = c["D"] ** -0.5
    if c["kind"] == "decode":
        if lens is not None:
            # ragged: one un-padded call per sequence on a subset of sequences (upcast outside the clock,
            # as kalosm-llama keeps its cache in f32)
            pick = list(range(min(4, c["B"])))
            reps, dts = 3, []
            seqs = [(f32(q[b:b + 1]), f32(k[b:b + 1, :, :int(lens[b])]), f32(v[b:b + 1, :, :int(lens[b])])) for b in pick]
            for _ in range(reps):
                t0 = time.perf_counter()
                for qb, kb, vb in seqs:
                    oracle.flash_attention(qb, kb, vb, scale)
                dts.append(time.perf_counter() - t0)
            frac = float(np.sum(lens[pick])) / float(np.sum(lens))
            sample = f"sequences {pick} of the batch, un-padded, f16 upcast to f32, median of {reps} passes"
            return dict(value=byts * frac / float(np.median(dts)) / 1e9, unit="GB/s", cores=threads, kind="port",
                        sample=sample)
        reps, dts = 3, []
        q, k, v = f32(q), f32(k), f32(v)
        mask = _decode_rows_mask(c, c["Skv"])
        kind = None if mask is None else "qk"
        oracle.flash_attention(q, k, v, scale, mask, kind)
        for _ in range(reps):
            t0 = time.perf_counter()
            oracle.flash_attention(q, k, v, scale, mask, kind)
            dts.append(time.perf_counter() - t0)
        return dict(value=byts / float(np.median(dts)) / 1e9, unit="GB/s", cores=threads, kind="port",
                    sample=f"the full step (all {c['B']} sequences), f16 upcast to f32 first, median of {reps} passes "
                           "after one warm-up pass")
    # prefill: a subset of query rows of every head (rows are independent in the reference algorithm)
    q, k, v = f32(q), f32(k), f32(v)
    target_flops = 2e11
    stride = max(1, int(np.ceil(flops / target_flops)))
    rows = np.arange(stride - 1, c["Sq"], stride, dtype=np.int32)
    off = c.get("q_pos_offset", c["Skv"] - c["Sq"])
    i = rows[:, None].astype(np.int64) + off
    j = np.arange(c["Skv"])[None, :]
    masked = j > i if c["causal"] else np.zeros((len(rows), c["Skv"]), bool)
    if c.get("window", 0):
        masked |= (j + c["window"]) <= i
    mask = np.where(masked, -np.inf, 0.0).astype(np.float32)
    reps, dts = 3, []
    qs = np.ascontiguousarray(q[:, :, rows])
    for _ in range(reps):
        t0 = time.perf_counter()
        oracle.flash_attention(qs, k, v, scale, mask, "qk")
        dts.append(time.perf_counter() - t0)
    dt = float(np.median(dts))
    # the CPU path has no tile skipping: it computes every (row, key) pair and masks afterwards, but
    # it is credited, like the GPU, with the visible pairs only
    sample_flops = 4 * c["D"] * c["H"] * c["B"] * int((~masked).sum())
    return dict(value=sample_flops / dt / 1e12, unit="TFLOP/s", cores=threads, kind="port",
                sample=f"every {stride}th query row of every head ({len(rows)} of {c['Sq']} rows), dense "
                       f"[rows, Skv] scores then mask, as the reference does; median of {reps} passes")


def run_config(name, steps, warmup, with_cpu=True):
    import floneum_amd as fa
    from floneum_amd import synth
    import oracle

    c = configs()[name]
    cfg_id = int(name[1])
    dev = fa.Device.default()
    lens = lens_t = None
    if "ragged" in c:
        lens = synth.integers(SEED + cfg_id, 7, c["B"], *c["ragged"]).astype(np.int32)
        lens_t = fa.IntTensor(dev, lens)
    flops, byts = algorithmic(c, lens)
    # decode streams the KV cache from HBM: rotate enough distinct sets to exceed the 256 MB MALL
    kv_bytes = byts
    n_sets = 1 if c["kind"] == "prefill" else max(2, min(8, int(np.ceil(1.2e9 / max(kv_bytes, 1)))))
    if name == "C5":
        n_sets = 1  # 6.5 GB per step already dwarfs the cache; one padded set is 13 GB of HBM
    dt, sets, host = make_inputs(fa, synth, dev, c, cfg_id, n_sets)
    blocks, kernel = prepare(fa, dev, c, sets, lens_t)
    wall_ms, main_ms = time_config(fa, dev, c, blocks, steps, warmup)
    main_ms_mean, main_ms_med = float(main_ms.mean()), float(np.median(main_ms))
    err = parity_spot_check(fa, oracle, c, blocks[0]._out_tensor, host, lens)

    if c["kind"] == "decode":
        value, unit = byts / (wall_ms * 1e-3) / 1e9, "GB/s"
        roof = dict(bound="hbm", achieved=byts / (main_ms_mean * 1e-3) / 1e9, peak=PEAK_HBM_GBS, unit="GB/s")
    else:
        peak = PEAK_MFMA_F32_TFLOPS if c["dtype"] == "f32" else PEAK_MFMA_F16_TFLOPS
        value, unit = flops / (wall_ms * 1e-3) / 1e12, "TFLOP/s"
        roof = dict(bound="mfma", achieved=flops / (main_ms_mean * 1e-3) / 1e12, peak=peak, unit="TFLOP/s")
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"], roof["traffic_note"] = measured_traffic(name, kernel)
    roof["kernel"] = kernel
    roof["kernel_ms_mean"] = main_ms_mean
    roof["kernel_ms_median"] = main_ms_med
    roof["kernel_ms_min"] = float(main_ms.min())
    res = dict(value=value, unit=unit, ms_per_step=wall_ms, roofline=roof,
               config=dict(workload=name, kind=c["kind"], batch=c["B"], q_heads=c["H"], kv_heads=c["Hkv"],
                           q_len=c["Sq"], kv_len=c["Skv"], head_dim=c["D"], causal=c["causal"],
                           q_pos_offset=c.get("q_pos_offset"), window=c.get("window"),
                           ragged_lens=c.get("ragged"), kv_sets_rotated=n_sets,
                           algorithmic_flops=flops, algorithmic_bytes=byts),
               dtype=c["dtype"], frac_of_roofline=value / roof["peak"], spot_check_max_abs_err=err)
    if lens is not None:
        # what the ragged lengths cost: the same call with every sequence at the mean length (same buffers,
        # the same bytes to within rounding), so any difference in GB/s is load imbalance between workgroups
        eq = np.full(c["B"], int(round(float(lens.mean()))), np.int32)
        eq_t = fa.IntTensor(dev, eq)
        _, eq_byts = algorithmic(c, eq)
        eq_blocks, _ = prepare(fa, dev, c, sets, eq_t)
        eq_wall_ms, _ = time_config(fa, dev, c, eq_blocks, max(5, steps // 2), min(warmup, 5))
        eq_value = eq_byts / (eq_wall_ms * 1e-3) / 1e9
        res["imbalance"] = dict(lens_min=int(lens.min()), lens_mean=float(lens.mean()), lens_max=int(lens.max()),
                                equal_lengths_value=eq_value, unit=unit, ragged_over_equal=value / eq_value,
                                note="same call with every sequence at the mean length; 1.0 = the ragged batch "
                                     "streams as fast as an even one")
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(oracle, c, host, lens, flops, byts)
    return res


# ---- a whole attention layer step around the call -----------------------------------------------------------------
# What kalosm-llama runs per layer (models/kalosm-llama/src/raw/attention_layer.rs:217-280,400-455, raw/mod.rs:618-620):
# q / k RMS-norm (blocks that have them), rotary embedding, KvCache::append, the mask tensor of the step from
# MaskCache::get_mask, attention, output as [b, seq, heads * hd].  Here: fhip_kv_cache_qkv_rope_append (one launch) and
# fhip_flash_attention with the mask TENSOR, through the C ABI, everything but the two calls prepared outside the clock.
LAYER_STEPS = {
    # one decode step at batch 1 on the f32 cache kalosm-llama keeps, about 4096 keys (the cache grows by one per step)
    "L1": dict(kind="layer_decode", B=1, H=32, Hkv=8, n=1, start=4090, D=128, dtype="f32", norm=False),
    # a 512-token prompt (C1's shape) into an empty cache, with q / k norms
    "L2": dict(kind="layer_prompt", B=1, H=32, Hkv=8, n=512, start=0, D=64, dtype="f32", norm=True),
}


def run_layer_step(name, steps, warmup, with_cpu=True):
    import floneum_amd as fa
    from floneum_amd import synth
    import oracle

    c = LAYER_STEPS[name]
    L = fa.lib()
    dev = fa.Device.default()
    B, H, Hkv, n, D = c["B"], c["H"], c["Hkv"], c["n"], c["D"]
    decode = c["kind"] == "layer_decode"
    seed = SEED + 0x100 + int(name[1])
    eb = 4
    # the projections as the reference holds them: [b, seq, heads, hd], viewed as [b, heads, seq, hd]
    qh = synth.normal(seed, 0, (B, n, H, D), 1.0, np.float32)
    kh = synth.normal(seed, 1, (B, n, Hkv, D), 1.0, np.float32)
    vh = synth.normal(seed, 2, (B, n, Hkv, D), 1.0, np.float32)
    tq, tk, tv = (fa.Tensor.from_numpy(dev, a, fa.F32).transpose(1, 2) for a in (qh, kh, vh))
    ctx = 8192
    rope = fa.RopeCache(D, ctx, 10000.0, dev)
    qw = kw = None
    qn = kn = None
    if c["norm"]:
        qw = synth.normal(seed, 3, (D,), 0.2, np.float32) + np.float32(1.0)
        kw = synth.normal(seed, 4, (D,), 0.2, np.float32) + np.float32(1.0)
        qn, kn = fa.RmsNorm(qw, None, 1e-6, fa.F32, dev), fa.RmsNorm(kw, None, 1e-6, fa.F32, dev)
    cache = fa.KvCache(2, ctx, fa.F32, dev)
    k0 = v0 = None
    if decode:  # the context the step runs on: `start` cached positions (already rotated keys, as the cache holds them)
        k0 = synth.normal(seed, 5, (B, Hkv, c["start"], D), 1.0, np.float32)
        v0 = synth.normal(seed, 6, (B, Hkv, c["start"], D), 1.0, np.float32)
        cache.append(dev, fa.Tensor.from_numpy(dev, k0, fa.F32), fa.Tensor.from_numpy(dev, v0, fa.F32))
    q_out = fa.Tensor.empty(dev, (B, H, n, D), fa.F32)
    out_buf = fa.Tensor.empty(dev, (B, n, H, D), fa.F32)  # what attention_wo multiplies, as [b, seq, heads * hd]
    mask_table = None
    if decode:  # get_mask(1, pos, None): a [1, pos + 1] row of zeros; one row long enough for every step, narrowed per step
        mask_t = fa.Tensor.from_numpy(dev, np.zeros((1, ctx), np.float32), fa.F32)
    else:       # get_mask(n, 0, None), which MaskCache keeps per (seq_len, window), with the interval table it keeps beside it
        am = fa.MaskCache(fa.F32).get_mask_on_device(n, 0, None, dev)
        mask_t, mask_table = am.mask(), am.intervals()
    # argument blocks, filled once; per step only the position, the cache views and the mask width change
    tables = rope._tables(c["start"], False)
    cq, co, ck, cv = tq._c4(), q_out._c4(), tk._c4(), tv._c4()
    ka, va = fa.CTensor4(), fa.CTensor4()
    cqn, ckn = (qn._c(), kn._c()) if c["norm"] else (None, None)
    pqn, pkn = (ctypes.byref(cqn), ctypes.byref(ckn)) if c["norm"] else (None, None)
    last_len = c["start"] + n * (warmup + 2 * steps + 2) if decode else n
    dummy = fa.Tensor(q_out.buffer, fa.F32, (B, Hkv, last_len, D), (0, 0, 0, 1))  # stands in for the cache views below
    mask_arg = (mask_t.narrow(1, 0, last_len), fa.MaskKind.QKMask) if decode else (mask_t, fa.MaskKind.QKMask, mask_table)
    args = q_out._attn_args(dummy, dummy, D ** -0.5, mask_arg, None, None, None, fa.KERNEL_AUTO, out_buf.transpose(1, 2))
    # one workspace for every step: the split-KV plan, and with it the size, changes with the cache length
    need, most = ctypes.c_size_t(), 16
    for length in (range(c["start"] + n, last_len + 1, n) if decode else [n]):
        args.k.shape[2] = args.v.shape[2] = args.mask.shape[1] = length
        fa.check(L.fhip_flash_attention_workspace_bytes(ctypes.byref(args), dev.compute_units, ctypes.byref(need)))
        most = max(most, need.value)
    ws = fa.Buffer(dev, most)
    args.workspace, args.workspace_bytes = ws.ptr, ws.nbytes
    pos = [c["start"]]

    def step():
        if not decode:
            fa.check(L.fhip_kv_cache_reset(cache.handle))  # a new sequence; the cache keeps its memory
            pos[0] = 0
        tables.start_pos = pos[0]
        fa.check(L.fhip_kv_cache_qkv_rope_append(cache.handle, dev.stream, pqn, pkn, ctypes.byref(tables), ctypes.byref(cq),
                                                 fa.F32, ctypes.byref(co), fa.F32, ctypes.byref(ck), ctypes.byref(cv), fa.F32,
                                                 ctypes.byref(ka), ctypes.byref(va)))
        pos[0] += n
        args.k, args.v = ka, va
        if decode:
            args.mask.shape[1] = pos[0]
        fa.check(L.fhip_flash_attention(dev.stream, ctypes.byref(args)))

    for _ in range(warmup):
        step()
    dev.synchronize()
    len0 = pos[0]
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    dev.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    keys_mean = (len0 + n * (steps + 1) / 2.0) if decode else float(n)  # keys the attention call of a step sees
    # the attention kernel's own duration (events carried by its dispatch), in a second pass
    starts = [Event(fa, dev) for _ in range(steps)]
    dones = [Event(fa, dev) for _ in range(steps)]
    for i in range(steps):
        args.main_kernel_start, args.main_kernel_done = starts[i].h, dones[i].h
        step()
    args.main_kernel_start = args.main_kernel_done = None
    dev.synchronize()
    kernel_ms = np.array([dones[i].ms_since(starts[i]) for i in range(steps)])
    for e in starts + dones:
        L.fhip_event_destroy(e.h)
    kid = ctypes.c_int32()
    fa.check(L.fhip_flash_attention_select(ctypes.byref(args), ctypes.byref(kid)))

    # algorithmic bytes of a step: every tensor a stage must read or write, once
    # (rotation: q in, q out, new k / v in, new k / v into the cache, cos / sin rows; attention: q, K, V, mask tensor, out)
    rot = eb * (2 * B * H * n * D + 4 * B * Hkv * n * D + 2 * n * (D // 2))
    attn_of = lambda keys: eb * (2 * B * H * n * D + 2 * B * Hkv * keys * D + n * keys)  # noqa: E731
    byts = rot + attn_of(keys_mean)
    flops = 4 * D * H * B * (n * keys_mean if decode else n * (n + 1) / 2.0)

    # spot check of one more step against the CPU checker's pieces
    step()
    dev.synchronize()
    f32 = lambda t: np.asarray(t.to_numpy(), np.float32)  # noqa: E731
    view = lambda cten: fa.Tensor(fa._View(dev, cten.ptr, cache), fa.F32, tuple(cten.shape), tuple(cten.stride), cten.offset)  # noqa: E731
    k_all, v_all, q_rot = f32(view(ka)), f32(view(va)), f32(q_out)
    p0 = pos[0] - n
    q_in, k_in = qh.transpose(0, 2, 1, 3), kh.transpose(0, 2, 1, 3)
    if c["norm"]:
        q_in, k_in = oracle.rms_norm(q_in, qw, None, 1e-6), oracle.rms_norm(k_in, kw, None, 1e-6)
    q_ref = oracle.rope(q_in, rope.cos_host, rope.sin_host, p0)
    k_ref = oracle.rope(k_in, rope.cos_host, rope.sin_host, p0)
    bit_exact = bool(np.array_equal(q_rot, q_ref) and np.array_equal(k_all[:, :, -n:], k_ref)
                     and np.array_equal(v_all[:, :, -n:], vh.transpose(0, 2, 1, 3)))
    mask = oracle.get_mask(n, p0, None)
    ref = oracle.flash_attention(q_ref, np.ascontiguousarray(k_all), np.ascontiguousarray(v_all), D ** -0.5, mask, "qk")
    got = f32(out_buf).reshape(B, n, H, D).transpose(0, 2, 1, 3)
    err = float(np.abs(got - ref).max())

    value = byts / (wall_ms * 1e-3) / 1e9
    kmean = float(kernel_ms.mean())
    roof = dict(bound="hbm", achieved=attn_of(keys_mean) / (kmean * 1e-3) / 1e9, peak=PEAK_HBM_GBS, unit="GB/s")
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"], roof["traffic_note"] = measured_traffic(name, fa.KERNEL_NAMES[kid.value])
    roof.update(kernel=fa.KERNEL_NAMES[kid.value], kernel_ms_mean=kmean, kernel_ms_median=float(np.median(kernel_ms)),
                kernel_ms_min=float(kernel_ms.min()),
                note="the attention call's main kernel against the attention call's own algorithmic bytes")
    res = dict(value=value, unit="GB/s", ms_per_step=wall_ms, roofline=roof,
               config=dict(workload=name, kind=c["kind"], batch=B, q_heads=H, kv_heads=Hkv, q_len=n,
                           kv_len=int(round(keys_mean)), head_dim=D, causal=True, q_norm_k_norm=c["norm"],
                           calls_per_step="fhip_kv_cache_qkv_rope_append + fhip_flash_attention (mask tensor, output as "
                                          "[b, seq, heads * hd])" + ("" if decode else " with the mask's interval table, after "
                                                                     "fhip_kv_cache_reset"),
                           algorithmic_flops=int(flops), algorithmic_bytes=int(byts)),
               dtype=c["dtype"], frac_of_roofline=value / PEAK_HBM_GBS, spot_check_max_abs_err=err,
               rope_and_cache_rows_bit_exact=bit_exact)
    if with_cpu:
        # the same step on the CPU checker's restatements (rotation, cache append by concatenation as the reference does,
        # mask, attention), a few steps
        threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        reps = 5 if decode else 3
        ocache = oracle.KvCache(2, ctx)
        if decode:
            ocache.append(k0, v0)
        dts = []
        p = c["start"]
        for _ in range(reps):
            t0 = time.perf_counter()
            if not decode:
                ocache, p = oracle.KvCache(2, ctx), 0
            qi, ki = qh.transpose(0, 2, 1, 3), kh.transpose(0, 2, 1, 3)
            if c["norm"]:
                qi, ki = oracle.rms_norm(qi, qw, None, 1e-6), oracle.rms_norm(ki, kw, None, 1e-6)
            qr = oracle.rope(qi, rope.cos_host, rope.sin_host, p)
            kr = oracle.rope(ki, rope.cos_host, rope.sin_host, p)
            kall, vall = ocache.append(kr, vh.transpose(0, 2, 1, 3))
            m = oracle.get_mask(n, p, None)
            oracle.flash_attention(qr, np.ascontiguousarray(kall), np.ascontiguousarray(vall), D ** -0.5, m, "qk")
            p += n
            dts.append(time.perf_counter() - t0)
        res["cpu_baseline"] = dict(value=byts / float(np.median(dts)) / 1e9, unit="GB/s", cores=threads, kind="port",
                                   sample=f"{reps} whole steps (norm, rotation, cache append by concatenation, mask, attention), median")
    return res


def calibration_copy(mib=256, reps=3):
    """A first KvCache.append is a plain copy of the appended tensor: reads `mib` MiB, writes `mib` MiB."""
    import floneum_amd as fa
    dev = fa.Device.default()
    rows = mib * (1 << 20) // (2 * 128)  # f16 rows of 128 elements
    src = fa.Tensor.empty(dev, (1, 1, rows, 128), fa.F16)
    fa.check(fa.lib().fhip_memset(dev.stream, ctypes.c_void_p(src.buffer.ptr), 0, rows * 256))
    for _ in range(reps):
        cache = fa.KvCache(2, rows, fa.F16, dev)
        cache.append(dev, src, src)  # keys and values: two copies of `mib` MiB each
        dev.synchronize()
        del cache


ISSUE_MIXES = ["matrix instructions only", "a dependent chain of matrix instructions", "+ 4 v_fma", "+ 8 v_fma", "+ 4 v_exp",
               "+ 4 scalar adds", "+ 1 ds_read_b128 (the operand 8 steps later)", "+ 3 ds_read_b128",
               "+ 2 ds_read_b64_tr_b16 (used 8 steps later)", "+ 1 ds_read_b128 + 2 ds_read_b64_tr_b16",
               "+ 1 ds_read_b128 + 2 ds_read_b64_tr_b16 + fma, exp2, add", "+ 2 ds_read_b128 + fma, exp2, add",
               "+ 2 ds_read_b128 + 1/2 ds_read_b64_tr_b16 + 1/4 ds_write_b128"]


def calibration_issue(rounds=20000):
    """What one wavefront per SIMD can issue beside its matrix instructions (fhip_calibration_issue): shader-clock
    cycles per step of one v_mfma_f32_32x32x16_f16 (32 cycles of the matrix pipe) and the named companions."""
    import floneum_amd as fa
    dev = fa.Device.default()
    L = fa.lib()
    cus = dev.compute_units
    nbytes = cus * (256 * 4 + 16)
    scratch = fa.Buffer(dev, nbytes)
    host = np.empty(nbytes, np.uint8)
    rows = []
    for mix, what in enumerate(ISSUE_MIXES):
        for r in (rounds // 10, rounds):  # the first brings the clock to where this load holds it
            fa.check(L.fhip_calibration_issue(dev.stream, mix, r, ctypes.c_void_p(scratch.ptr), nbytes))
        dev.synchronize()
        fa.check(L.fhip_memcpy_d2h(dev.stream, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(scratch.ptr), nbytes))
        ticks = host[cus * 1024:].view(np.uint64).reshape(cus, 2).astype(np.float64)
        steps = 16.0 * rounds
        rows.append(dict(mix=mix, companions=what, cycles_per_step=_r(float(np.median(ticks[:, 0])) / steps, 4),
                         ns_per_step=_r(float(np.median(ticks[:, 1])) * 10.0 / steps, 4),
                         sclk_ghz=_r(float(np.median(ticks[:, 0] / ticks[:, 1])) * 0.1, 4)))
    return rows


def calibration_mfma(seconds=0.0):
    """What the matrix cores deliver with nothing else in the way (fhip_calibration_mfma: a register-only loop of
    the prefill kernel's matrix instruction, one wavefront per SIMD), with the clock the chip held meanwhile.  The
    nominal 2.5 PFLOP/s is 256 CUs x 4 SIMDs x 1024 FLOP/clk at 2.4 GHz; under load the power limit sets the clock.
    seconds > 0: keep the f16 / random-operand / 100 % case running back to back for that long (for sampling socket
    power and clocks from outside) and report only that case."""
    import floneum_amd as fa
    dev = fa.Device.default()
    L = fa.lib()
    cus = dev.compute_units
    nbytes = cus * (256 * 4 + 16)
    scratch = fa.Buffer(dev, nbytes)
    host = np.empty(nbytes, np.uint8)

    def launch(dtype, rand, duty, rounds):
        fa.check(L.fhip_calibration_mfma(dev.stream, dtype, rand, duty, rounds, ctypes.c_void_p(scratch.ptr), nbytes))

    def one(dtype, rand, duty, rounds=60000, repeat=1):
        launch(dtype, rand, duty, rounds)  # brings the clock to where this load holds it
        dev.synchronize()
        e0, e1 = Event(fa, dev), Event(fa, dev)
        e0.record(dev)
        for _ in range(repeat):
            launch(dtype, rand, duty, rounds)
        e1.record(dev)
        e1.sync()
        ms = e1.ms_since(e0)
        fa.check(L.fhip_memcpy_d2h(dev.stream, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(scratch.ptr), nbytes))
        ticks = host[cus * 1024:].view(np.uint64).reshape(cus, 2).astype(np.float64)
        ghz = ticks[:, 0] / ticks[:, 1] * 0.1
        flops = 4.0 * cus * rounds * repeat * 32 * 32768
        for e in (e0, e1):
            L.fhip_event_destroy(e.h)
        return dict(dtype={fa.F16: "f16", fa.BF16: "bf16"}[dtype], operands="random" if rand else "zero",
                    duty_percent=duty, tflops=flops / (ms * 1e-3) / 1e12, ms=ms,
                    sclk_ghz_median=float(np.median(ghz)), sclk_ghz_min=float(ghz.min()), sclk_ghz_max=float(ghz.max()))

    if seconds > 0:
        probe = one(fa.F16, 1, 100)
        return [one(fa.F16, 1, 100, repeat=max(1, int(seconds * 1e3 / probe["ms"])))]
    return [one(fa.F16, 1, 100), one(fa.F16, 1, 84), one(fa.F16, 1, 67), one(fa.F16, 0, 100), one(fa.BF16, 1, 100)]


def calibration_read(mib=256, slices=5, launches=60):
    """What a kernel that only reads reaches (fhip_calibration_read: 16-byte non-temporal loads, eight in flight per
    lane, no arithmetic, no output): `mib` MiB per launch, the launches rotating over `slices` distinct slices so that
    the 256 MB Infinity Cache cannot serve them, back to back.  The size is C2's KV bytes per call."""
    import floneum_amd as fa
    dev = fa.Device.default()
    L = fa.lib()
    nbytes = mib << 20
    buf = fa.Buffer(dev, nbytes * slices)
    sink = fa.Buffer(dev, dev.compute_units * 32)
    fa.check(L.fhip_memset(dev.stream, ctypes.c_void_p(buf.ptr), 0x3c, nbytes * slices))

    def launch(i):
        fa.check(L.fhip_calibration_read(dev.stream, ctypes.c_void_p(buf.ptr + (i % slices) * nbytes), nbytes,
                                         ctypes.c_void_p(sink.ptr), dev.compute_units * 32))

    for i in range(10):
        launch(i)
    dev.synchronize()
    t0 = time.perf_counter()
    for i in range(launches):
        launch(i)
    dev.synchronize()
    us = (time.perf_counter() - t0) * 1e6 / launches
    return dict(mib_per_launch=mib, slices_rotated=slices, launches=launches, us_per_launch=us,
                gbps=nbytes / us / 1e3, frac_of_peak=nbytes / us / 1e3 / PEAK_HBM_GBS)


def calibration_xcd_map(workgroups=1024, show=32):
    """Which XCD the workgroups of a one-dimensional launch run on (fhip_calibration_xcd_map), for a few launches in a
    row with small launches of other sizes in between (a 1-, 3- and 13-workgroup launch of the same kernel), and whether
    workgroups with the same number modulo 8 always share an XCD: what the decode kernels' merge inside the kernel
    relies on."""
    import floneum_amd as fa
    dev = fa.Device.default()
    L = fa.lib()
    buf = fa.Buffer(dev, workgroups)
    host = np.empty(workgroups, np.uint8)
    rows = []
    for before in (0, 1, 3, 13, 0, 5):
        if before:
            fa.check(L.fhip_calibration_xcd_map(dev.stream, before, ctypes.c_void_p(buf.ptr), workgroups))
        fa.check(L.fhip_calibration_xcd_map(dev.stream, workgroups, ctypes.c_void_p(buf.ptr), workgroups))
        fa.check(L.fhip_memcpy_d2h(dev.stream, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(buf.ptr), workgroups))
        rows.append(dict(workgroups_of_the_launch_before=before, xcd_of_first_workgroups="".join(str(int(x)) for x in host[:show]),
                         xcds=int(len(set(host.tolist()))),
                         same_number_modulo_8_same_xcd=bool(all(host[i] == host[i & 7] for i in range(workgroups)))))
    return rows


def record_traffic(name, fetch_csv, write_csv):
    """profiles/traffic.json entry of one configuration from the two counter CSVs (one counter per profiler run).
    The copy kernel of --calibration-copy moves 256 MiB each way; its counts give the bytes per count."""
    import csv

    def per_kernel(path, counter):
        """kernel name -> (mean count over its dispatches, largest count)"""
        sums = {}
        for r in csv.DictReader(open(path)):
            if r["Counter_Name"] == counter:
                sums.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return {k: (float(np.mean(v)), float(np.max(v))) for k, v in sums.items()}

    copied = 256 * (1 << 20)
    out = {}
    kernel = None
    for key, path, counter in (("fetch_bytes", fetch_csv, "FETCH_SIZE"), ("write_bytes", write_csv, "WRITE_SIZE")):
        counts = per_kernel(path, counter)
        # the calibration copies are the largest copies of the run (a workload that appends to a KV cache copies too)
        copy = [v[1] for k, v in counts.items() if "copy_rows_kernel" in k]
        assert copy, f"{path}: no copy_rows_kernel dispatches (run bench.py with --calibration-copy)"
        per_count = copied / max(copy)
        main = {k: v for k, v in counts.items() if any(t in k for t in ("decode_mfma", "decode_vec", "prefill_mfma_kernel",
                                                                       "prefill_mfma_wide_kernel", "prefill_mfma_wide_rows32_kernel",
                                                                       "prefill_mfma_rows64_kernel",
                                                                       "prefill_f32_kernel",
                                                                       "prefill_f32_wide", "attn_generic"))}
        assert len(main) == 1, f"{path}: expected one main kernel, found {sorted(main)}"
        kname, (count, _) = next(iter(main.items()))
        out[key] = count * per_count
        out[key.replace("bytes", "bytes_per_count")] = per_count
        kernel = "decode_splitkv" if "decode" in kname else "prefill_mfma" if "prefill_mfma" in kname else \
            "prefill_f32" if "prefill_f32" in kname else "generic"
        out["kernel_symbol"] = kname
    out["kernel"] = kernel
    # the file the kernel lives in (the wide-head 16-bit prefill kernels have files of their own)
    out["source"] = "attn_prefill_mfma_rows32.hip" if "prefill_mfma_wide_rows32" in out["kernel_symbol"] else \
        "attn_prefill_mfma_rows64.hip" if "prefill_mfma_rows64" in out["kernel_symbol"] else \
        "attn_prefill_mfma_wide.hip" if "prefill_mfma_wide" in out["kernel_symbol"] else KERNEL_SOURCES[kernel]
    out["source_sha256"] = source_hash(kernel, out["source"])
    try:
        rec = json.load(open(TRAFFIC_RECORD))
    except (OSError, ValueError):
        rec = {}
    rec[name] = out
    with open(TRAFFIC_RECORD, "w") as f:
        json.dump(rec, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps({name: out}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="C2", choices=sorted(configs()) + sorted(LAYER_STEPS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the other configurations (C3 under \"prefill\"; C1, C4, C5 under \"configs\")")
    ap.add_argument("--record-traffic", nargs=3, metavar=("CONFIG", "FETCH_CSV", "WRITE_CSV"),
                    help="no benchmark: read the counter_collection CSVs of two `rocprofv3 --pmc FETCH_SIZE` / `--pmc "
                         "WRITE_SIZE` runs of `bench.py --config CONFIG --no-cpu --no-extra --calibration-copy` and "
                         "store the dominant kernel's HBM bytes per launch in profiles/traffic.json")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (the KV-cache row copy kernel) three times, so a "
                         "rocprofv3 --pmc run of this command has a kernel of known traffic to scale FETCH_SIZE / "
                         "WRITE_SIZE with")
    ap.add_argument("--calibration-read", action="store_true",
                    help="no benchmark: run the read-only streaming kernel over 256 MiB slices and print GB/s")
    ap.add_argument("--calibration-xcd", action="store_true",
                    help="no benchmark: print which XCD the workgroups of a few launches in a row run on")
    ap.add_argument("--calibration-issue", action="store_true",
                    help="cycles per step of one matrix instruction and companions, one wavefront per SIMD (fhip_calibration_issue)")
    ap.add_argument("--calibration-mfma", nargs="?", type=float, const=0.0, default=None, metavar="SECONDS",
                    help="no benchmark: run the register-only matrix-core loop (f16 random operands at 100 / 84 / 67 %% "
                         "duty, zero operands, bf16) and print TFLOP/s and the shader clock held; with SECONDS, keep "
                         "the f16 random 100 %% case running that long (to sample socket power from outside)")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this build runs on exactly one GPU (no sharding, no collectives); --gpus {a.gpus} is "
              "not supported", file=sys.stderr)
        sys.exit(2)

    if a.record_traffic:
        record_traffic(*a.record_traffic)
        return
    if a.calibration_read:
        print(json.dumps({"read_calibration": calibration_read(), "nominal_peak_gbps": PEAK_HBM_GBS}))
        return
    if a.calibration_xcd:
        for row in calibration_xcd_map():
            print(json.dumps(row))
        return
    if a.calibration_issue:
        for row in calibration_issue():
            print(json.dumps(row), flush=True)
        return
    if a.calibration_mfma is not None:
        print(json.dumps({"mfma_calibration": calibration_mfma(a.calibration_mfma), "nominal_peak_tflops": PEAK_MFMA_F16_TFLOPS}))
        return

    main_res = (run_layer_step if a.config in LAYER_STEPS else run_config)(a.config, a.steps, a.warmup, with_cpu=not a.no_cpu)
    if a.calibration_copy:
        calibration_copy()
    detail("workload", dict(main_res, steps=a.steps, warmup=a.warmup))
    read_cal = pre = mfma_cal = None
    others = {}
    if not a.no_extra and a.config == "C2":
        # beside the nominal 8 TB/s the roofline is priced against: what a kernel that only reads the same number of
        # bytes per launch reaches on this chip
        read_cal = calibration_read()
        detail("read_calibration", read_cal)
        # the other half of the metric: C3 prefill on the matrix cores
        # the shader clock needs some tens of milliseconds of matrix load to settle: warm the prefill
        # leg up for longer than the (much shorter) decode steps need
        pre = run_config("C3", max(20, a.steps // 2), max(100, a.warmup), with_cpu=not a.no_cpu)
        detail("workload", dict(pre, steps=max(20, a.steps // 2), warmup=max(100, a.warmup)))
        # beside the nominal peak the roofline is priced against: what a register-only loop of the same matrix
        # instruction reaches on this chip under its power limit, and the clock it holds
        mfma_cal = calibration_mfma()
        detail("mfma_calibration", mfma_cal)
        # the remaining benchmark configurations (C1M: C1 with the mask as the tensor kalosm-llama passes; F2: C2's batch
        # with the f32 cache kalosm-llama keeps; M1: C2's batch with four new rows per sequence; L1 / L2: a whole
        # attention layer step around the call; W2 / W3: Gemma-3's key length 256 in f16, no CPU leg)
        for name, (steps, warmup, cpu) in EXTRA_WORKLOADS.items():
            run = run_layer_step if name in LAYER_STEPS else run_config
            r = run(name, steps, warmup, with_cpu=cpu and not a.no_cpu)
            r["steps"], r["warmup"] = steps, warmup
            detail("workload", r)
            others[name] = r
    print(json.dumps(final_line(main_res, a.steps, a.warmup, read_cal, pre, mfma_cal, others)), flush=True)


# workloads beside C2 and C3 on the default run: name -> (steps, warm-up steps, CPU leg)
EXTRA_WORKLOADS = {"C1": (200, 20, True), "C1M": (200, 20, False), "C4": (100, 100, True), "C5": (20, 3, True),
                   "F2": (100, 10, True), "M1": (100, 10, True), "L1": (200, 20, True), "L2": (200, 20, True),
                   "W2": (100, 10, False), "W3": (50, 100, False)}


def detail(kind, obj):
    """One complete record per line, ahead of the final line (which stays short enough for any log tail)."""
    print(json.dumps({"detail": kind, **(obj if isinstance(obj, dict) else {"rows": obj})}), flush=True)


def _r(x, digits=5):
    return float(f"{x:.{digits}g}") if isinstance(x, float) else x


def _short_roofline(roof, keys=("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "kernel_ms_mean")):
    return {k: _r(roof[k]) for k in keys if k in roof}


def _short_config(cfg):
    keep = ("workload", "kind", "batch", "q_heads", "kv_heads", "q_len", "kv_len", "head_dim", "causal", "window",
            "ragged_lens", "kv_sets_rotated", "algorithmic_flops", "algorithmic_bytes")
    return {k: cfg[k] for k in keep if cfg.get(k) is not None}


def _short_cpu(cpu):
    return dict(value=_r(cpu["value"]), unit=cpu["unit"], cores=cpu["cores"], kind=cpu["kind"], sample=cpu["sample"][:100])


def final_line(main_res, steps, warmup, read_cal=None, pre=None, mfma_cal=None, others=None):
    """The last line of stdout: the headline workload in full contract form, C3 under "prefill", one short entry per other
    workload.  Everything else went out earlier as "detail" lines.  Kept under 4 KB."""
    line = {"metric": METRIC, "value": _r(main_res["value"], 6), "unit": main_res["unit"], "n_gpus": 1, "steps": steps,
            "warmup": warmup, "ms_per_step": _r(main_res["ms_per_step"], 6), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": main_res["dtype"], "data": "synthetic (seeded SplitMix64 normals)",
            "config": _short_config(main_res["config"]), "roofline": _short_roofline(main_res["roofline"]),
            "frac_of_roofline": _r(main_res["frac_of_roofline"]),
            "spot_check_max_abs_err": _r(main_res["spot_check_max_abs_err"])}
    if read_cal:
        line["roofline"]["read_calibration_gbps"] = _r(read_cal["gbps"])
    if "cpu_baseline" in main_res:
        line["cpu_baseline"] = _short_cpu(main_res["cpu_baseline"])
    if "imbalance" in main_res:
        line["imbalance"] = {k: _r(v) for k, v in main_res["imbalance"].items() if k != "note"}
    if pre:
        line["prefill"] = dict(value=_r(pre["value"], 6), unit=pre["unit"], ms_per_step=_r(pre["ms_per_step"], 6), dtype=pre["dtype"],
                               frac_of_roofline=_r(pre["frac_of_roofline"]), config=_short_config(pre["config"]),
                               roofline=_short_roofline(pre["roofline"]),
                               spot_check_max_abs_err=_r(pre["spot_check_max_abs_err"]))
        if "cpu_baseline" in pre:
            line["prefill"]["cpu_baseline"] = _short_cpu(pre["cpu_baseline"])
        if mfma_cal:
            row = next((r for r in mfma_cal if r["dtype"] == "f16" and r["operands"] == "random" and r["duty_percent"] == 100), None)
            if row:
                line["prefill"]["mfma_calibration"] = {k: _r(row[k]) for k in ("dtype", "operands", "duty_percent", "tflops",
                                                                               "sclk_ghz_median")}
    if others:
        # value = per step by the wall clock; kernel_frac = the dominant kernel's own duration against its roofline
        line["configs"] = {name: dict(value=_r(r["value"]), unit=r["unit"], ms_per_step=_r(r["ms_per_step"]),
                                      step_frac=_r(r["frac_of_roofline"], 4), kernel_frac=_r(r["roofline"]["frac"], 4),
                                      err=_r(r["spot_check_max_abs_err"], 3)) for name, r in others.items()}
    return line


if __name__ == "__main__":
    main()
