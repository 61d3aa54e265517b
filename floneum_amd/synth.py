"""Seeded synthetic inputs for the attention benchmarks and parity tests.

Counter-based SplitMix64: element `i` of stream (seed, tensor_id) is a pure function of
(seed, tensor_id, i), so any slice of any tensor can be regenerated independently and the same
buffers can be handed to the GPU kernels and to the CPU checker.  Normals come from Box-Muller in
float64 and are then rounded to the requested element type.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def splitmix64(seed, start, count):
    """Outputs start .. start+count-1 of SplitMix64 seeded with `seed` (output 0 is the first)."""
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        return _mix(np.uint64(seed) + idx * _GOLDEN)


def stream_seed(seed, tensor_id):
    with np.errstate(over="ignore"):
        return int(_mix(np.array([np.uint64(seed) ^ (np.uint64(tensor_id + 1) * _M2)], dtype=np.uint64))[0])


def uniform(seed, tensor_id, count, start=0):
    """Uniform (0, 1) doubles with 53 random bits."""
    z = splitmix64(stream_seed(seed, tensor_id), start, count)
    return ((z >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, tensor_id, shape, scale=1.0, dtype=np.float32, chunk=1 << 22):
    """i.i.d. N(0, scale^2) of the given shape; element i uses uniforms 2i and 2i+1."""
    n = int(np.prod(shape))
    out = np.empty(n, dtype)
    for s in range(0, n, chunk):
        c = min(chunk, n - s)
        u = uniform(seed, tensor_id, 2 * c, 2 * s)
        r = np.sqrt(-2.0 * np.log(u[0::2]))
        out[s:s + c] = (r * np.cos(2.0 * np.pi * u[1::2]) * scale).astype(dtype)
    return out.reshape(shape)


def integers(seed, tensor_id, count, lo, hi):
    """Integers uniform in [lo, hi] (inclusive)."""
    z = splitmix64(stream_seed(seed, tensor_id), 0, count)
    return (lo + (z % np.uint64(hi - lo + 1)).astype(np.int64)).astype(np.int64)
