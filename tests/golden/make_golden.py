"""Writes tests/golden/attention_cases.json: the inputs of the reference's own attention tests
(fusor-ml/fusor/src/composite/flash_attention.rs:207-358, fusor-ml/core/src/composite/
flash_attention.rs:559-673) with expected outputs from the float64 textbook twin, plus a few
closed-form cases.  Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

NEG = float("-inf")


def case(name, q, k, v, scale, mask=None, kind=None, source=""):
    q, k, v = (np.asarray(a, np.float32) for a in (q, k, v))
    scale = float(np.float32(scale))
    out = oracle.flash_attention_f64(q, k, v, scale, None if mask is None else np.asarray(mask, np.float32), kind)
    enc = lambda a: [None if np.isneginf(x) else float(x) for x in np.asarray(a, np.float64).ravel()]  # noqa: E731
    return dict(name=name, source=source, q_shape=list(q.shape), k_shape=list(k.shape), scale=scale,
                q=enc(q), k=enc(k), v=enc(v), mask_kind=kind,
                mask_shape=None if mask is None else list(np.shape(mask)),
                mask=None if mask is None else enc(mask),  # null encodes -inf
                expected=[float(x) for x in out.ravel()])


def main():
    s2 = 1.0 / np.sqrt(np.float32(2.0))
    eye = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    v12 = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 2, 2)
    cases = [
        case("cpu_2x2", eye, eye, v12, s2, source="fusor flash_attention.rs:207-239"),
        case("cpu_2x2_causal", eye, eye, v12, s2, [[0, NEG], [0, 0]], "qk", "fusor flash_attention.rs:241-276"),
        case("gqa_ramp", (np.arange(16) * 0.1).reshape(1, 4, 2, 2), (np.arange(8) * 0.1 + 1).reshape(1, 2, 2, 2),
             (np.arange(8) * 0.1 + 2).reshape(1, 2, 2, 2), s2, source="fusor flash_attention.rs:278-313"),
        case("batch_key_mask", (np.arange(12) * 0.1).reshape(2, 1, 3, 2), (np.arange(12) * 0.1 + 1).reshape(2, 1, 3, 2),
             (np.arange(12) * 0.1 + 2).reshape(2, 1, 3, 2), s2, [[0, 0, 0], [0, 0, NEG]], "batch_key",
             "fusor flash_attention.rs:315-358"),
        case("core_2x2", np.array([[[[1, 2], [3, 4]]]], np.float32), np.array([[[[1, 2], [3, 4]]]], np.float32),
             np.array([[[[1, 2], [3, 4]]]], np.float32), s2, source="core flash_attention.rs:559-603 (shape)"),
    ]
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_cases.json"), "w") as f:
        json.dump(cases, f, indent=1)
    print(f"wrote {len(cases)} cases")


if __name__ == "__main__":
    main()
