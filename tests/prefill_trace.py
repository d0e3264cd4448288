"""Runs a prompt of 2048 tokens (or of as many as the first argument says) through the device decoder on Qwen2.5-0.5B shapes three times: the
program behind profiles/prompt_2048_kernel_trace.txt."""
import importlib, os, sys

import numpy as np
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT); sys.path.insert(0, os.path.join(ROOT, "tests"))
mil = importlib.import_module("adreno-llms_amd")
from decode_harness import QWEN25_05B, GpuDecoder, Model
assert mil.lib().mi_init(0) == 1
queue = mil.Queue()
M = int(sys.argv[1]) if len(sys.argv) > 1 else 2048
m = Model(dict(QWEN25_05B, max_pos=M), seed=2024)
gd = GpuDecoder(m, queue)
ids = [int(t) for t in np.random.default_rng(M).integers(0, QWEN25_05B["vocab"], M)]
for _ in range(3):
    assert gd.dec.prefill(queue, ids)
print("done", gd.dec.read(queue), flush=True)
gd.close()
