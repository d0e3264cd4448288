#!/usr/bin/env python3
"""Writes tests/golden/quantizer_vectors.npz.

Runs only in the build container, where the reference tree is mounted: it
imports the reference's two pure quantizer functions

    quantize_row_symmetric   src/models/lfm2-5-350m/scripts/quantize_weights.py:53-57
    quantize_row_q4          src/models/lfm2-5-350m/scripts/quantize_q4.py:62-82

feeds them seeded fp16 rows and stores inputs and outputs.  The stored arrays
are data (inputs and expected outputs); no reference source text is kept.
The points that only running the functions can settle are the float32-vs-double
arithmetic of `w / scale` under the installed NumPy, the single rounding of
`np.float16(python_float)` and round-half-to-even at exact .5 ties, so the rows
below include constructed ties, a zero row, a single-spike row and a row whose
scale is a half subnormal.
"""
import importlib.util
import os
import sys

import numpy as np

REF = os.environ.get("ADRENO_REFERENCE", "/root/reference")
LF_SCRIPTS = os.path.join(REF, "src/models/lfm2-5-350m/scripts")


def _load(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def int8_rows(rng, K):
    rows = []
    for sigma in (0.02, 0.02, 0.02, 1.0, 5e-4):
        rows.append((rng.standard_normal(K) * sigma).astype(np.float16))
    rows.append(np.zeros(K, np.float16))                       # all-zero row -> scale 1.0
    spike = np.zeros(K, np.float16); spike[K // 3] = np.float16(-0.7311)
    rows.append(spike)                                         # single spike -> -127
    # exact .5 ties: absmax 127 -> scale 1.0, entries k + 0.5 are exact in fp16 below 1024
    tie = np.array([127.0] + [(-1) ** i * (i % 120 + 0.5) for i in range(K - 1)], np.float16)
    rows.append(tie)
    # scale in the half-subnormal range: absmax ~ 3e-5 -> scale ~ 2.4e-7
    tiny = (rng.standard_normal(K) * 1e-5).astype(np.float16)
    rows.append(tiny)
    # absmax = fp16 max (65504): scale rounds in the normal range, q hits +-127
    big = (rng.standard_normal(K) * 2e4).astype(np.float16); big[5] = np.float16(65504.0)
    rows.append(big)
    return np.stack(rows)


def q4_rows(rng, K):
    rows = []
    for sigma in (0.02, 0.02, 1.0, 5e-4):
        rows.append((rng.standard_normal(K) * sigma).astype(np.float16))
    z = (rng.standard_normal(K) * 0.02).astype(np.float16); z[32:64] = 0   # one all-zero block
    rows.append(z)
    # ties: absmax 7 -> scale 1, inv 1; entries k + 0.5
    tie = np.tile(np.array([7.0] + [(-1) ** i * (i % 7 + 0.5) for i in range(31)], np.float16), K // 32)
    rows.append(tie)
    tiny = (rng.standard_normal(K) * 1e-5).astype(np.float16)
    rows.append(tiny)
    return np.stack(rows)


def main():
    qw = _load(os.path.join(LF_SCRIPTS, "quantize_weights.py"), "ref_quantize_weights")
    q4 = _load(os.path.join(LF_SCRIPTS, "quantize_q4.py"), "ref_quantize_q4")
    rng = np.random.default_rng(20240607)

    out = {}
    for K in (64, 896):
        w = int8_rows(rng, K)
        q = np.empty(w.shape, np.int8)
        s = np.empty(w.shape[0], np.float16)
        for r in range(w.shape[0]):
            q[r], s[r] = qw.quantize_row_symmetric(w[r])
        out[f"int8_w_k{K}"] = w.view(np.uint16)
        out[f"int8_q_k{K}"] = q
        out[f"int8_s_k{K}"] = s.view(np.uint16)

        w = q4_rows(rng, K)
        p = np.empty((w.shape[0], K // 2), np.uint8)
        sc = np.empty((w.shape[0], K // 32), np.float16)
        for r in range(w.shape[0]):
            p[r], sc[r] = q4.quantize_row_q4(w[r].astype(np.float32))
        out[f"q4_w_k{K}"] = w.view(np.uint16)
        out[f"q4_p_k{K}"] = p
        out[f"q4_s_k{K}"] = sc.view(np.uint16)

    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quantizer_vectors.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, {k: v.shape for k, v in out.items()}, "numpy", np.__version__)


if __name__ == "__main__":
    sys.exit(main())
