"""Builds libfusor_hip.so (and libfusor_hip.a) for gfx950 from floneum_amd/csrc with hipcc."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
SOURCES = ["api.hip", "attn_generic.hip", "attn_decode.hip", "attn_prefill_mfma.hip", "attn_prefill_mfma_wide.hip", "attn_prefill_mfma_rows32.hip", "attn_prefill_mfma_rows64.hip",
           "attn_prefill_f32.hip",
           "kv_cache.hip", "mask_intervals.hip", "rope.hip", "calibration.hip"]
LIB = os.path.join(HERE, "libfusor_hip.so")
STATIC = os.path.join(HERE, "libfusor_hip.a")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
         # packed-f32 VALU forms are kept out of the generated code on purpose
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


# the rotary embedding must round every product and sum on its own (bit parity with the reference's CPU path)
PER_FILE = {"rope.hip": ["-ffp-contract=off"]}


def _compile(src):
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + PER_FILE.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True):
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    if os.path.exists(STATIC):
        os.remove(STATIC)
    subprocess.check_call(["ar", "rcs", STATIC] + objs)
    # the C++ host mirror's test program (runs on the GPU box, started by tests/test_host_mirror_gpu.py)
    root = os.path.dirname(HERE)
    cpp = os.path.join(root, "tests", "cpp", "test_host_mirror.cpp")
    if os.path.exists(cpp):
        subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(root, "include"), cpp,
                               "-o", os.path.join(root, "tests", "cpp", "test_host_mirror"),
                               "-L", HERE, "-lfusor_hip", "-Wl,-rpath,$ORIGIN/../../floneum_amd"])
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
