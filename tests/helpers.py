"""Shared helpers of the test-suite."""
import importlib
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
mil = importlib.import_module("adreno-llms_amd")


def synth_w(seed, N, K, sigma=0.02):
    return mil.synth_normal_f16(seed, sigma, (N, K))


def synth_x(seed, *shape):
    return mil.synth_normal_f16(seed, 1.0, shape)


def assert_tolerance(got_f16, want_f16):
    """The stated bar: max-abs/rel 1e-3 and cosine >= 0.9999 on fp16 outputs."""
    g = np.asarray(got_f16, np.float16).astype(np.float64).ravel()
    w = np.asarray(want_f16, np.float16).astype(np.float64).ravel()
    err = np.abs(g - w)
    assert np.all(err <= 1e-3 + 1e-3 * np.abs(w)), f"max err {err.max()} at {err.argmax()}"
    cos = np.dot(g, w) / max(np.linalg.norm(g) * np.linalg.norm(w), 1e-30)
    assert cos >= 0.9999, f"cosine {cos}"
